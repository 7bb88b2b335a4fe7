// Internal declarations shared by the HIP translation units of libtinygemma_hip.so.
// Nothing here is part of the C ABI (that is include/tinygemma_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/tinygemma_hip.h"

// ---------------------------------------------------------------------------------------------
// Packed int8 weight layout in HBM
//
// The reference keeps W as [in][out] row-major int8 (csrc/include/tensor.hpp:144-192): bytes run
// along the output dimension and the reduction runs across rows.  On the device every matrix is
// re-tiled once at upload into
//
//        P[tile][kg][c][j]      tile = col / 128, kg = row / 4, c = col % 128, j = row % 4
//
// so that (1) one 16-byte lane load holds 4 output columns x 4 consecutive input rows, with the
// 4 rows of one column packed in one dword (the k-contiguous operand shape MFMA wants, and four
// sign-extending byte->float converts for the GEMV), (2) a wave's 64 lane loads are one
// contiguous 1 KiB segment covering two kg rows of a 128-column tile, and (3) everything a
// workgroup streams for its tile is one contiguous slab of K*128 bytes.  The values are the
// reference's bytes, only their addresses change.
// ---------------------------------------------------------------------------------------------
#define TG_CT 128            // output columns per packed tile
#define TG_MAX_K 6912        // largest reduction length (1B down projection)

inline size_t tg_packed_index(int K, int r, int c) {
	return (((size_t)(c / TG_CT) * (size_t)(K / 4) + (size_t)(r / 4)) * TG_CT + (size_t)(c % TG_CT)) * 4 + (size_t)(r % 4);
}

// ---- GEMV launch description --------------------------------------------------------------
enum { TG_PRO_PLAIN = 0, TG_PRO_NORM = 1, TG_PRO_RESNORM = 2, TG_PRO_EMBED = 3 };
enum { TG_EPI_STORE = 0, TG_EPI_GEGLU = 1, TG_EPI_LOGITS = 2 };

struct TgGemv {
	// matrix
	const int8_t *W;       // packed, ntiles tiles of 128 columns
	const float *scales;   // one per (virtual) column, tile order
	int K;                 // reduction length (rows of the reference matrix)
	int ntiles;            // 128-column tiles (grid.x)
	int KS;                // K splits (grid.y)
	int pairs_per_block;   // (K/8)/KS: one "pair" = 8 input rows x 128 columns = 1 KiB
	int tpc;               // tiles per completion group: 1, or 2 for the fused up|gate matrix
	// workspace for the cross-workgroup reduction (unused when KS*tpc == 1)
	float *partial;        // [ntiles][KS][128]
	unsigned *counters;    // [ntiles/tpc], zero between launches
	// prologue: how the input vector is produced
	int pro;
	int hidden;            // length of the residual stream (PRO_NORM/RESNORM/EMBED)
	const float *x;        // PLAIN: the input [K]; NORM: vector to normalise; RESNORM: residual
	const float *pend;     // RESNORM: block output still to be post-normalised and added
	const float *w_post;   // RESNORM: post-norm weights
	const float *w_pre;    // NORM/RESNORM/EMBED: pre-norm weights
	float *xr_out;         // NORM/RESNORM/EMBED: residual stream written by workgroup (0,0); may be null
	const int8_t *wte;     // EMBED: [vocab][hidden] row-major int8 (reference layout)
	const float *wte_scales;
	const int *tok;        // EMBED: device token id (clamped to [0, vocab))
	int vocab;
	float emb_scale;       // EMBED: float(sqrt(hidden))
	// epilogue
	int epi;
	float *y;              // STORE: [N]; GEGLU: [N/2]; LOGITS: [N] or null
	const float *lut;      // GEGLU
	float gmin, geps;
	int lut_size;
	float *blk_val;        // LOGITS: per-workgroup maxima [ntiles]
	int *blk_idx;
	unsigned *argmax_counter;
	int *tok_out;          // LOGITS: winning index (lowest index on ties)
	int *tok_log;          // LOGITS: optional history, tok_log[*step] = winner
	int *step;             // LOGITS: device step counter, incremented by the last workgroup
	int *pos;              // LOGITS: device position counter, incremented by the last workgroup
};

struct TgAttnDecode {
	const float *qkv;        // [n_head*hd + 2*hd]: q | k | v straight out of the fused projection
	const float *rms_q, *rms_k;
	const float *cos_t, *sin_t;  // [n_pos][hd/2]
	float *kc, *vc;          // cache [max_pos][hd]
	int max_pos;             // slots (ring for local layers, linear for global)
	const int *pos;          // device counters: pos[0] = position_ptr, pos[1]/pos[2] = buffer_ptr of local/global layers
	int bp_index;            // 1 (local layer) or 2 (global layer)
	int chunk;               // keys per workgroup
	float *part_acc;         // [nblocks][n_head][hd]
	float *part_ml;          // [nblocks][n_head][2]
	unsigned *counter;
	float *out;              // [n_head*hd]
	int n_head;
};

void tg_launch_gemv(const TgGemv &g, hipStream_t s);
void tg_launch_attn_decode(const TgAttnDecode &a, int max_blocks, hipStream_t s);

// ---- prefill kernels (rows = prompt positions) -----------------------------------------------
void tg_launch_embed_rows(float *x, const int *ids, int S, const int8_t *wte, const float *scales, int hidden, int vocab,
                          hipStream_t s);
// out = rmsnorm(in, w); if resid != null first in = rmsnorm(in, w_post) + resid is formed and stored to resid_out
void tg_launch_norm_rows(float *out, const float *in, const float *w_pre, const float *w_post, const float *resid, float *resid_out,
                         int S, int dim, hipStream_t s);
void tg_launch_qk_norm_rope_rows(float *q, float *k, const float *v, const float *rms_q, const float *rms_k, const float *cos_t,
                                 const float *sin_t, float *kc, float *vc, int max_pos, int S, int n_head, int hd, int ldq, int ldkv,
                                 hipStream_t s);
void tg_launch_attn_prefill(float *o, const float *q, const float *k, const float *v, int S, int n_head, int hd, int ldq, int ldkv,
                            int ldo, int is_sw, int window, hipStream_t s);
// C[m][N] = (A[m][K] . W) * scales, W packed; epi GEGLU writes C[m][N/2]
void tg_launch_gemm(float *C, const float *A, const int8_t *Wp, const float *scales, int m, int K, int ntiles, int epi,
                    const float *lut, float gmin, float geps, int lut_size, hipStream_t s);

// ---- errors -----------------------------------------------------------------------------------
int tg_fail(int code, const std::string &msg);
#define TG_HIP(expr)                                                                           \
	do {                                                                                       \
		hipError_t e_ = (expr);                                                                \
		if (e_ != hipSuccess) return tg_fail(TG_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
	} while (0)

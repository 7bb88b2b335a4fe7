// Internal declarations shared by the HIP translation units of libtinygemma_hip.so.
// Nothing here is part of the C ABI (that is include/tinygemma_hip.h and, for knobs and probes, include/tinygemma_hip_debug.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/tinygemma_hip.h"
#include "../../include/tinygemma_hip_debug.h"

// ---------------------------------------------------------------------------------------------
// Packed int8 weight layout in HBM
//
// The reference keeps W as [in][out] row-major int8 (csrc/include/tensor.hpp:144-192): bytes run
// along the output dimension and the reduction runs across rows.  On the device every matrix is
// re-tiled once at upload into tiles of C output columns,
//
//        P[tile][kg][c][j]      tile = col / C, kg = row / 4, c = col % C, j = row % 4
//
// so that (1) one 16-byte lane load holds 4 output columns x 4 consecutive input rows, with the
// 4 rows of one column packed in one dword (the k-contiguous operand shape MFMA wants, and four
// sign-extending byte->float converts for the GEMV), (2) consecutive lanes read consecutive
// 16-byte pieces, and (3) everything a workgroup streams for its tile is one contiguous slab of
// K*C bytes.  The GEMV uses C = 4 ... 128 per matrix (a tile per workgroup over the whole K, so
// narrow matrices still give hundreds of workgroups); the prefill GEMM uses C = 128.  The values
// are the reference's bytes, only their addresses change.
// ---------------------------------------------------------------------------------------------
#define TG_CT 128            // widest tile (and the GEMM tile width)
#define TG_MAX_K 6912        // largest reduction length (1B down projection)
#define TG_MAX_HIDDEN 1152   // largest residual-stream width
#define TG_ATTN_MERGE_MAX 16 // attention partials the output projection merges in its prologue
#define TG_ATTN_MAX_BLOCKS 1024 // attention workgroups per launch, upper bound
#define TG_ATTN_FOLD 64         // partials the merge launch folds into one

// ---- weight prefetch riding along with a launch ------------------------------------------------
// Batch-1 decode is a chain of ~130 dependent, latency-bound launches per token during which HBM
// is mostly idle.  A launch can therefore carry extra workgroups whose only job is to touch the
// weights of the NEXT launch, pulling them out of HBM into the memory-side cache and the L2 while
// the current launch works through its own latency chain.  A hint only: results do not depend on it.
// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2); a prefetch workgroup on XCD x touches
// the slabs of the consumer tiles t with t % 8 == x, the tiles the consumer's workgroups on the same XCD will
// read.  That matters: the same loads dealt to the XCDs without regard to the consumer gain nothing (measured).
struct TgPrefetch {
	const int8_t *ptr;   // first tile slab of the matrix to prefetch (null: nothing)
	uint32_t slab;       // bytes per tile slab
	int ntiles;          // slabs
	int nblocks;         // extra workgroups appended to the grid (multiple of 8)
};

__device__ __forceinline__ void tg_prefetch_block(const TgPrefetch &p, int first_extra_block) {
	if (p.ptr == nullptr) return;
	const int pb = (int)blockIdx.x - first_extra_block;
	const int x = (int)(blockIdx.x & 7u), q = pb >> 3, Q = p.nblocks >> 3;
	// The workgroups on XCD x share that XCD's tiles t = x, x + 8, ...: the 128-byte lines of those slabs are walked
	// as one flat index, cut into equal shares (a launch waits for its slowest workgroup).  One dword per line
	// brings the line in.
	if (x >= p.ntiles) return;
	const uint32_t nx = (uint32_t)(p.ntiles - x + 7) >> 3;
	const uint32_t lps = p.slab >> 7, total = nx * lps;
	const uint32_t per = (total + (uint32_t)Q - 1) / (uint32_t)Q;
	const uint32_t lo = (uint32_t)q * per, hi = lo + per < total ? lo + per : total;
	for (uint32_t i0 = lo + threadIdx.x; i0 < hi; i0 += 4u * 256u) {
		int sink = 0;
#pragma unroll
		for (uint32_t k = 0; k < 4; k++) {  // four loads in flight per lane: unconditional (clamped), consumed together
			uint32_t i = i0 + k * 256u;
			i = i < hi ? i : i0;
			const uint32_t j = i / lps, line = i - j * lps;
			sink += *(const int *)(p.ptr + (size_t)(x + 8 * (int)j) * p.slab + (size_t)line * 128u);
		}
		asm volatile("" ::"v"(sink));  // the values are not needed, the loads are
	}
}

// Extra workgroups of a launch: the first p1.nblocks of them prefetch p1, the rest p2.
__device__ __forceinline__ void tg_prefetch_dispatch(const TgPrefetch &p1, const TgPrefetch &p2, int first_extra_block) {
	if ((int)blockIdx.x < first_extra_block + p1.nblocks) tg_prefetch_block(p1, first_extra_block);
	else tg_prefetch_block(p2, first_extra_block + p1.nblocks);
}

// ---- GEMV launch description --------------------------------------------------------------
enum { TG_PRO_PLAIN = 0, TG_PRO_NORM = 1, TG_PRO_RESNORM = 2, TG_PRO_EMBED = 3, TG_PRO_ATTN_MERGE = 4 };
enum { TG_EPI_STORE = 0, TG_EPI_GEGLU = 1, TG_EPI_LOGITS = 2 };

struct TgGemv {
	// matrix: ntiles tiles of C columns, each a contiguous [K/4][C][4] slab
	const int8_t *W;
	const float *scales;   // one per (virtual) column, tile order
	int K;                 // reduction length (rows of the reference matrix)
	int ntiles;            // grid.x
	int C;                 // columns per tile: 4, 8, ..., 128
	int lc_shift;          // log2(C/4)
	int max_blocks;        // 0: one workgroup per tile; else workgroups loop over tiles when ntiles exceeds it
	int nmain;             // set by the launcher: workgroups that compute (the rest of the grid prefetches)
	// prologue (the TG_PRO_* mode is fixed by the kernel role)
	int hidden;            // length of the residual stream (NORM/RESNORM/EMBED); equals K there
	const float *x;        // PLAIN: the input [K]; NORM: vector to normalise; RESNORM: residual
	const float *pend;     // RESNORM: block output still to be post-normalised and added
	const float *w_post;   // RESNORM: post-norm weights
	const float *w_pre;    // NORM/RESNORM/EMBED: pre-norm weights
	float *xr_out;         // NORM/RESNORM/EMBED: residual stream written by workgroup 0; may be null
	const int8_t *wte;     // EMBED: [vocab][hidden] row-major int8 (reference layout)
	const float *wte_scales;
	const int *tok;        // EMBED: device token id (clamped to [0, vocab))
	// EMBED, optional: the previous step's greedy pick is still pending as per-workgroup maxima of its LM-head launch.
	// Every workgroup then finishes that argmax itself (am_n pairs) instead of reading *tok, and workgroup 0 does the
	// per-token bookkeeping (token log, counters) that the finishing launch would have done.
	const float *am_val;
	const int *am_idx;
	int am_n;
	int *am_ctr, *am_log;
	int vocab;
	float emb_scale;       // EMBED: float(sqrt(hidden))
	const int *pos;        // ATTN_MERGE: device counters (pos[0] = position of this token)
	int host_pos;          // ATTN_MERGE: the same position as a launch argument, or -1 to read the device counter
	int attn_max_pos;      // ATTN_MERGE: cache slots of this layer
	int attn_chunk;        // ATTN_MERGE: keys per attention workgroup
	int merge_nb;          // ATTN_MERGE, set by the kernel from its leading arguments: partials to merge, or -1 (derive from pos)
	const float *part_acc; // ATTN_MERGE: [nb][4][256]
	const float *part_ml;  // ATTN_MERGE: [nb][4][2]
	// epilogue (the TG_EPI_* mode is fixed by the kernel role)
	float *y;              // STORE: [N]; GEGLU: [N/2]; LOGITS: [N] or null
	const float *lut;      // GEGLU
	float gmin, geps;
	int lut_size;
	float *blk_val;        // LOGITS: per-workgroup maximum and its index, [ntiles]
	int *blk_idx;
	TgPrefetch pf, pf2;    // weights of the next launches (optional); the extra workgroups are split between them
};

struct TgAttnDecode {
	const float *qkv;        // [n_head*hd + 2*hd]: q | k | v straight out of the fused projection
	const float *rms_q, *rms_k;
	const float *cos_t, *sin_t;  // [n_pos][hd/2]
	float *kc, *vc;          // cache [max_pos][hd]
	int max_pos;             // slots (ring for local layers, linear for global)
	const int *pos;          // device counters: pos[0] = position_ptr, pos[1]/pos[2] = buffer_ptr of local/global layers
	int bp_index;            // 1 (local layer) or 2 (global layer)
	int host_pos, host_bp;   // the same counters as launch arguments (saves a dependent load), or -1 to read the device ones
	int host_cur;            // host_bp % max_pos when the host knows it (then nblocks is exactly the workgroups the keys need), else -1
	int chunk;               // keys per workgroup
	float *part_acc;         // [nblocks][n_head][hd]
	float *part_ml;          // [nblocks][n_head][2]
	int n_head;
	int nblocks;             // attention workgroups in the grid; workgroups past them prefetch
	TgPrefetch pf, pf2;      // weights of the next launches (optional)
};

enum { TG_ROLE_PLAIN = 0, TG_ROLE_QKV_EMBED, TG_ROLE_QKV, TG_ROLE_OPROJ, TG_ROLE_UPGATE, TG_ROLE_DOWN, TG_ROLE_LMHEAD,
       TG_ROLE_LMHEAD_PLAIN };
// A launch spelled out: kernel, geometry and the argument list in the form hipLaunchKernel and a graph's kernel node
// take it.  The tg_desc_* functions fill one in place (`args` points into the descriptor itself: it is not copied
// afterwards); tg_launch_* = describe + launch.  A replayed graph of a decode step has its position-dependent nodes
// (attention, its merge, the output projection) re-described before every replay.
struct TgLaunchDesc {
	const void *func;
	dim3 grid, block;
	void *args[12];
	const void *p[6];  // storage of pointer arguments
	int i[6];          // ... of integer arguments
	TgGemv g;          // ... of the descriptor a GEMV kernel takes by value
	TgAttnDecode a;    // ... of the descriptor an attention kernel takes by value
};
void tg_desc_gemv(const TgGemv &g, int role, TgLaunchDesc *d);
void tg_desc_attn_decode(const TgAttnDecode &a, int max_blocks, TgLaunchDesc *d);
void tg_desc_attn_merge(const TgAttnDecode &a, int nblk, float *merged_acc, float *merged_ml, TgLaunchDesc *d);
// which of the position-dependent kernels of a decode step a kernel node's function is: 1 attention, 2 its merge, 3 the
// output projection, 0 none of them
int tg_decode_node_kind(const void *func);
inline void tg_launch_desc(const TgLaunchDesc &d, hipStream_t s) {
	(void)hipLaunchKernel(d.func, d.grid, d.block, const_cast<void **>(d.args), 0, s);
}
void tg_launch_gemv(const TgGemv &g, int role, hipStream_t s);
void tg_launch_attn_decode(const TgAttnDecode &a, int max_blocks, hipStream_t s);
void tg_launch_attn_merge(const TgAttnDecode &a, int nblk, float *merged_acc, float *merged_ml, hipStream_t s);
void tg_launch_argmax_finish(const float *blk_val, const int *blk_idx, int n, int *ctr, int *tok_log, int advance, hipStream_t s);
// min-p sampling (tg_sample.hip): n a multiple of 1024; scratch probs[n], seg[tg_minp_segments(n)], bsum/bmax[tg_minp_blocks(n)];
// mode 0 = decode step (append + advance), 1 = replace the token written last, 2 = out_tok only;
// the draw is randf[rand_idx], or randf[ctr[3] - rand_base (- 1 in mode 1)] when rand_idx < 0
size_t tg_minp_blocks(int n);
size_t tg_minp_segments(int n);
void tg_launch_minp(const float *logits, int n, float minp, float temp, const float *randf, int rand_idx, int rand_base, float *probs,
                    float *seg, float *bsum, float *bmax, int *ctr, int *tok_log, int mode, int *out_tok, hipStream_t s);

// ---- one-kernel decode step (tg_decode_fused.hip) --------------------------------------------------------------
// All layers of a decode step in ONE launch of resident workgroups: `ng` GEMV workgroups that own fixed column tiles of
// every projection (tiles g and g + ng) and TG_FUSED_ATTN_WGS attention workgroups.  Where the launch path has a launch
// boundary, the workgroups hand over through device memory: producers store write-through, arrive on counters, consumers
// poll the counters and then read the data with ordinary loads from a buffer that is written once per launch (a line
// that was never read before cannot be stale in an L1 or in another XCD's L2).  The LM head stays a launch of its own.
#define TG_FUSED_ATTN_WGS TG_ATTN_MERGE_MAX
struct TgFusedMat {
	int K, C, lc_shift, ntiles;
};
struct TgFusedLayer {
	const int8_t *Wqkv, *Wo, *Wug, *Wd;      // GEMV tile layout
	const float *sqkv, *so, *sug, *sd;       // column scales, tile order
	const float *apre, *apost, *mpre, *mpost, *rms_q, *rms_k;
	float *kc, *vc;
	int max_pos, is_sw;
};
struct TgFused {
	const TgFusedLayer *layers;  // device array [L]
	int L, hidden, ng;
	TgFusedMat mqkv, mo, mug, md;
	// first layer: embedding of the device-side token, or of the previous step's pending greedy pick (see TgGemv)
	const int8_t *wte;
	const float *wte_scales;
	const int *tok;
	const float *am_val;
	const int *am_idx;
	int am_n;
	int *am_ctr, *am_log;
	int vocab;
	float emb_scale;
	// attention: tables [n_pos][128] of the global / local layers, counters of this step, keys per attention workgroup
	const float *cos_g, *sin_g, *cos_l, *sin_l;
	int pos, bp_local, bp_global, chunk_local, chunk_global;
	const float *lut;
	float gmin, geps;
	int lut_size;
	float *xr;            // [2L+1][hidden] residual stream after every block (written by GEMV workgroup 0)
	// exchange buffer: per layer qkv | partial outputs | partial (max, sum) | o | h | d, every region 256-byte aligned
	float *xch;
	size_t layer_stride;  // floats
	int off_qkv, off_pacc, off_pml, off_o, off_h, off_d;
	// hand-over state: 8 arrival counters of the GEMV workgroups (one 128-byte line per XCD), 8 copies of the attention
	// counter, one error word; all_base = sum of the GEMV counters at launch, attn_base = value of each attention counter
	unsigned *sync;
	unsigned all_base, attn_base;
	int max_spins;
	unsigned long long *ts;  // optional (debug): [L][24] timestamps of GEMV workgroup 0 (0..15) and attention workgroup 0 (16..18)
};
#define TG_FUSED_SYNC_WORDS (17 * 32)
// Largest number of 4 KiB steps of one tile the kernel keeps in registers, per projection; the launcher picks the
// instantiation: 0 = (2, 1, 9, 7) the 1B shape, 1 = (1, 1, 3, 2) the 270m shape; -1: no instantiation fits
int tg_fused_variant(const TgFused &f);
// returns false when the kernel cannot be co-resident on this device (the caller then uses the launch path)
bool tg_fused_supported(int n_cu);
void tg_launch_decode_fused(const TgFused &f, int variant, hipStream_t s);

// ---- prefill kernels (rows = prompt positions) -----------------------------------------------
void tg_launch_embed_rows(float *x, const int *ids, int S, const int8_t *wte, const float *scales, int hidden, int vocab,
                          hipStream_t s);
// out = rmsnorm(in, w); if resid != null first in = rmsnorm(in, w_post) + resid is formed and stored to resid_out
// apack/rowfac non-null: the normalised rows are also (out == nullptr: only) written as digit planes + row factors for
// tg_launch_gemm_mfma (rowfac as tg_launch_quant_pack lays it out for S rows)
void tg_launch_norm_rows(float *out, const float *in, int nparts, size_t part_stride, const float *w_pre, const float *w_post, const float *resid,
                         float *resid_out, int S, int dim, int8_t *apack, float *rowfac, hipStream_t s,
                         float *clear_rows = nullptr);  // clear_rows: S floats set to 0 (row maxima the next product folds into)
void tg_launch_qk_norm_rope_rows(float *q, float *k, const float *v, const float *rms_q, const float *rms_k, const float *cos_t,
                                 const float *sin_t, float *kc, float *vc, int max_pos, int S, int n_head, int hd, int ldq, int ldkv,
                                 hipStream_t s);
// Balanced work list of a prefill layer (device copies of what tg_attn_prefill_plan returns) + scratch.
struct TgAttnPrefillPlan {
	const int4 *items;  // [nitems] {query tile, first key tile, end key tile, slot or -1}
	const int4 *split;  // [nsplit] {query tile, first slot, chunks}
	const int2 *tiles;  // [query tiles] {first slot, chunks} of a split query tile, {-1, 1} of a whole one
	int nitems, nsplit;
	float *part_o, *part_ml;
};
extern int g_attn_prefill_split;  // prefill attention: 0 = fp32 matrix path, 1 = split-precision matrix path (two fp16 or three bf16 planes), 2 = the same with 32-query workgroups at any length, 3 = the same with 16-query workgroups at any length
int tg_attn_prefill_query_tile(int S, int n_cu);  // query positions per workgroup of the kernel a launch will take
// window < 0: causal layer; else a local layer whose queries see `window` keys before them and themselves
bool tg_attn_prefill_plan(int S, int n_cu, int tq, int window, std::vector<int4> &items, std::vector<int4> &split, int &nslots);
size_t tg_attn_prefill_part_floats(int nslots, int tq);
size_t tg_attn_prefill_ml_floats(int nslots, int tq);
void tg_launch_attn_prefill(float *o, const float *q, const float *k, const float *v, int S, int n_head, int hd, int ldq, int ldkv,
                            int ldo, int is_sw, int window, const TgAttnPrefillPlan *plan, int n_cu, hipStream_t s,
                            bool finish_later = false, void *planes_ws = nullptr, int *range_flag = nullptr);
// range_flag (device, may be null): set to 1 when an operand does not fit the fp16 planes of the split path
extern int g_attn_prefill_f16;
// planes_ws: tg_attn_prefill_planes_bytes(S) bytes of scratch for the pre-split K/V plane images of the split-precision path
// (null: every workgroup splits the tiles it stages itself)
extern int g_attn_prefill_planes;
size_t tg_attn_prefill_planes_bytes(int S);
// The rows of o (S x 1024, 4 heads x 256) -> digit planes + row factors of the int8 MFMA GEMM, merging the partial
// results of split query tiles on the way (instead of attn_prefill_merge_kernel + the two quantising launches);
// tg_launch_attn_prefill must then have been called with finish_later = true
void tg_launch_attn_prefill_finish(const float *o, int S, int ldo, const TgAttnPrefillPlan *plan, int n_cu, int8_t *apack, float *rowfac,
                                   hipStream_t s);
// exact-order GEMM on the GEMV tiling (ntiles tiles of Ct columns): C[m][N] = (A[m][K] . W) * scales; epi GEGLU writes C[m][N/2]
void tg_launch_gemm(float *C, const float *A, const int8_t *Wp, const float *scales, int m, int K, int ntiles, int Ct, int epi,
                    const float *lut, float gmin, float geps, int lut_size, hipStream_t s);

void tg_launch_copy(void *dst, const void *src, size_t bytes, hipStream_t s);

// Load-time re-tiling on the device.  A matrix of N virtual columns is assembled from up to three
// row-major int8 sources (device pointers, reference layout [K][n[i]], scales[i] per source column):
//   half == 0: the sources side by side (n[0] + n[1] + n[2] == N);
//   half  > 0: tiles of 2*half virtual columns = half columns of source 0 followed by the same half
//              columns of source 1 (both n[0] columns wide).
struct TgColMap {
	const int8_t *src[3];
	const float *scales[3];
	int n[3];
	int half;
};
void tg_launch_retile_gemv(int8_t *dst, float *dst_scales, const TgColMap &m, int K, int N, int C, hipStream_t s);
void tg_launch_retile_mfma(int8_t *dst, float *dst_scales, const TgColMap &m, int K, int N, hipStream_t s);

// int8 MFMA prefill GEMM (tg_gemm_mfma.hip): A is first quantised per row into three int8 digit planes in operand order
size_t tg_gemm_mfma_apack_bytes(int M, int K);
size_t tg_gemm_mfma_rows(int M);  // rowfac scratch holds twice this many floats
void tg_launch_quant_pack(const float *A, int lda, int M, int K, int8_t *apack, float *rowfac, const float *rowmax, hipStream_t s);
void tg_launch_gemm_mfma(float *C, const int8_t *apack, const float *rowfac, const int8_t *Wg, const float *scales, int M, int K,
                         int ntiles, int epi, const float *lut, float gmin, float geps, int lut_size, float *rowmax_part,
                         int kparts, size_t part_stride, hipStream_t s);
extern int g_gemm_lds, g_gemm_lds_cus, g_gemm_lds_ksplit;
int tg_gemm_clk_begin(unsigned long long **buf, int n, hipStream_t s);
int tg_gemm_clk_end(unsigned long long *buf, int n, double *clock_mhz, double *workgroup_us, int *workgroups);
extern long g_gemm_launches[3];
// parts of K (1, 2, 4) a plain-epilogue product should run in; part p writes C + p * part_stride, the consumer adds them
int tg_gemm_mfma_k_parts(int M, int K, int ntiles, int n_cu);

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global load of the wave (its fence covers all address spaces), which would drain a software pipeline
// of prefetched tiles at every stage; here loads issued earlier stay in flight across the barrier.
__device__ __forceinline__ void tg_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- cross-lane reductions without the LDS crossbar --------------------------------------------
// __shfl_xor compiles to ds_bpermute_b32 (address arithmetic + an LDS round trip, ~100 clocks of
// dependent latency per step).  The steps of a butterfly reduction have cheaper forms on gfx950:
// quad permutes and row rotations (DPP modifiers on a VALU move) inside a row of 16 lanes,
// v_permlane16_swap / v_permlane32_swap across rows.  tg_red_partner<O>(v) is what a reduction that walks
// O = 32, 16, 8, 4, 2, 1 DOWNWARDS (possibly starting lower) must combine with at step O.  At the 4-step
// the row rotation delivers lane (l - 4) mod 16 instead of l ^ 4; after the 8-step both hold the same
// value, so the reduction is bit-identical to the xor butterfly.  Not a general shuffle.
#if defined(__HIPCC__)
template <int CTRL>
__device__ __forceinline__ unsigned tg_dpp_u32(unsigned v) {
	return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int O>
__device__ __forceinline__ unsigned tg_red_partner_u32(unsigned v) {
	static_assert(O == 32 || O == 16 || O == 8 || O == 4 || O == 2 || O == 1, "butterfly step");
	if constexpr (O == 32) {
		const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);  // r[0] = {lo, lo}, r[1] = {hi, hi}
		return (__lane_id() & 32) ? r[0] : r[1];
	} else if constexpr (O == 16) {
		const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);  // r[0] = rows {0,0,2,2}, r[1] = rows {1,1,3,3}
		return (__lane_id() & 16) ? r[0] : r[1];
	} else if constexpr (O == 8) {
		return tg_dpp_u32<0x128>(v);  // row_ror:8
	} else if constexpr (O == 4) {
		return tg_dpp_u32<0x124>(v);  // row_ror:4
	} else if constexpr (O == 2) {
		return tg_dpp_u32<0x4E>(v);   // quad_perm:[2,3,0,1]
	} else {
		return tg_dpp_u32<0xB1>(v);   // quad_perm:[1,0,3,2]
	}
}
template <int O>
__device__ __forceinline__ float tg_red_partner(float v) { return __uint_as_float(tg_red_partner_u32<O>(__float_as_uint(v))); }
template <int O>
__device__ __forceinline__ int tg_red_partner(int v) { return (int)tg_red_partner_u32<O>((unsigned)v); }

// sums / maxima over the wave, a row of 16 lanes, or the lanes sharing (lane % LC); all lanes get the result
__device__ __forceinline__ float tg_wave_sum(float v) {
	v += tg_red_partner<32>(v);
	v += tg_red_partner<16>(v);
	v += tg_red_partner<8>(v);
	v += tg_red_partner<4>(v);
	v += tg_red_partner<2>(v);
	v += tg_red_partner<1>(v);
	return v;
}
__device__ __forceinline__ float tg_wave_max(float v) {
	v = fmaxf(v, tg_red_partner<32>(v));
	v = fmaxf(v, tg_red_partner<16>(v));
	v = fmaxf(v, tg_red_partner<8>(v));
	v = fmaxf(v, tg_red_partner<4>(v));
	v = fmaxf(v, tg_red_partner<2>(v));
	v = fmaxf(v, tg_red_partner<1>(v));
	return v;
}
__device__ __forceinline__ float tg_row16_sum(float v) {
	v += tg_red_partner<8>(v);
	v += tg_red_partner<4>(v);
	v += tg_red_partner<2>(v);
	v += tg_red_partner<1>(v);
	return v;
}
__device__ __forceinline__ float tg_row16_max(float v) {
	v = fmaxf(v, tg_red_partner<8>(v));
	v = fmaxf(v, tg_red_partner<4>(v));
	v = fmaxf(v, tg_red_partner<2>(v));
	v = fmaxf(v, tg_red_partner<1>(v));
	return v;
}
#endif

// ---- activation quantisation of the int8 MFMA GEMM (shared by the stand-alone pre-pass and fused producers) ----
// A row is scaled by a power of two so that its largest magnitude lies in [2^21, 2^22), rounded to an integer and
// written as three signed base-256 digits (int8 planes), 16 consecutive k per lane, in MFMA operand order:
//   planes [tile of 32 rows][K/32][3][64 lanes][16 bytes], lane = row % 32 + 32 * ((k % 32) / 16).
#if defined(__HIPCC__)
constexpr int TG_QBITS = 22;
__device__ __forceinline__ void tg_row_factors(float amax, float &mul, float &inv) {
	mul = 1.0f;
	inv = 1.0f;
	if (amax > 0.0f && amax < INFINITY) {
		int e;
		(void)frexpf(amax, &e);  // amax = f * 2^e, f in [0.5, 1)
		mul = ldexpf(1.0f, TG_QBITS - e);
		inv = ldexpf(1.0f, e - TG_QBITS);
	}
}
typedef int tg_i32x4 __attribute__((ext_vector_type(4)));
// v[16] consecutive k of one row -> the lane's 16 bytes of each plane
__device__ __forceinline__ void tg_quant16(const float *v, float mul, tg_i32x4 pl[3]) {
#pragma unroll
	for (int q = 0; q < 4; q++) {
		unsigned d0 = 0, d1 = 0, d2 = 0;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			const int xi = (int)rintf(v[4 * q + i] * mul);
			const int a0 = (xi << 24) >> 24;
			const int r1 = (xi - a0) >> 8;
			const int a1 = (r1 << 24) >> 24;
			const int a2 = (r1 - a1) >> 8;
			d0 |= (unsigned)(a0 & 255) << (8 * i);
			d1 |= (unsigned)(a1 & 255) << (8 * i);
			d2 |= (unsigned)(a2 & 255) << (8 * i);
		}
		pl[0][q] = (int)d0;
		pl[1][q] = (int)d1;
		pl[2][q] = (int)d2;
	}
}
// v[8] consecutive k of one row -> the 8 bytes of each plane (half of a lane's piece)
__device__ __forceinline__ void tg_quant8(const float *v, float mul, uint2 pl[3]) {
	unsigned d[3][2];
#pragma unroll
	for (int q = 0; q < 2; q++) {
		unsigned d0 = 0, d1 = 0, d2 = 0;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			const int xi = (int)rintf(v[4 * q + i] * mul);
			const int a0 = (xi << 24) >> 24;
			const int r1 = (xi - a0) >> 8;
			const int a1 = (r1 << 24) >> 24;
			const int a2 = (r1 - a1) >> 8;
			d0 |= (unsigned)(a0 & 255) << (8 * i);
			d1 |= (unsigned)(a1 & 255) << (8 * i);
			d2 |= (unsigned)(a2 & 255) << (8 * i);
		}
		d[0][q] = d0;
		d[1][q] = d1;
		d[2][q] = d2;
	}
#pragma unroll
	for (int p = 0; p < 3; p++) pl[p] = uint2{d[p][0], d[p][1]};
}
// where the 16 bytes of (row m, k0 = multiple of 16) of plane 0 go; planes are 64 pieces apart
__device__ __forceinline__ tg_i32x4 *tg_plane_dst(int8_t *apack, int m, int k0, int K) {
	const int kb = k0 >> 5, hb = (k0 >> 4) & 1;
	return reinterpret_cast<tg_i32x4 *>(apack) + ((size_t)(m >> 5) * (size_t)(K >> 5) + kb) * 3 * 64 + ((m & 31) + 32 * hb);
}
#endif

// ---- errors -----------------------------------------------------------------------------------
int tg_fail(int code, const std::string &msg);
#define TG_HIP(expr)                                                                           \
	do {                                                                                       \
		hipError_t e_ = (expr);                                                                \
		if (e_ != hipSuccess) return tg_fail(TG_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
	} while (0)

// Device-side building blocks of the decode GEMV (tg_gemv.hip) that the one-kernel decode step (tg_decode_fused.hip)
// shares with it, so that both paths do the same arithmetic in the same order and give the same bits.
#pragma once

#include "tg_internal.h"

namespace tgp {

constexpr int NT = 256;     // threads per workgroup (4 waves)
constexpr int NWAVE = 4;
constexpr int LUT_LDS = 1024;  // GeLU tables up to this size are staged in LDS (one 16-byte load per lane)
constexpr uint32_t STEP_BYTES = NT * 16u;  // the workgroup reads 4 KiB of its slab per step

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Cache policy bits of a weight load.  TG_W_NT marks the data as non-temporal (read once): measured on the
// 302 MB LM head, rotating over three copies so that nothing is left in the memory-side cache from the
// previous launch, the stream runs at 6.4 TB/s with it and 5.6 TB/s without.
constexpr int TG_W_DEFAULT = 0, TG_W_NT = 2;
// 16-byte weight loads in flight per lane of the LM head, which streams 36 steps per tile.  The per-layer
// projections cover 1 to 9 steps and are bound by latency, not by loads in flight: measured on whole decode steps, a
// fixed 2 is 4 % faster than a fixed 8 (1B shape; 8 % on the 270m shape); tg_gemv_depth picks theirs per shape.
constexpr int TG_DEPTH_STREAM = 8;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
	return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}
template <int AUX>
__device__ __forceinline__ i32x4 ldw(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
	return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, AUX);
}
__device__ __forceinline__ f32x4 ldx(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
	i32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
	return __builtin_bit_cast(f32x4, t);
}

__device__ __forceinline__ float wave_sum(float v) { return tg_wave_sum(v); }

// Sum over the workgroup; every thread gets the same value (fixed order).
__device__ __forceinline__ float block_sum(float v, float *sred) {
	v = wave_sum(v);
	__syncthreads();
	if ((threadIdx.x & 63) == 0) sred[threadIdx.x >> 6] = v;
	__syncthreads();
	return (sred[0] + sred[1]) + (sred[2] + sred[3]);
}

// The same sum for an `sred` that no thread of the workgroup can still be reading (its first use in a kernel, or one
// separated from the last by another barrier): the leading barrier of block_sum, which only protects such a reader, is
// dropped.  Same order of additions, same bits.
__device__ __forceinline__ float block_sum_fresh(float v, float *sred) {
	v = wave_sum(v);
	if ((threadIdx.x & 63) == 0) sred[threadIdx.x >> 6] = v;
	__syncthreads();
	return (sred[0] + sred[1]) + (sred[2] + sred[3]);
}

__device__ __forceinline__ float b2f(int d, int j) {  // signed byte j of d -> float (exact)
	return (float)(int8_t)(d >> (8 * j));
}

// ops.hpp:41-51: truncating index, below the table -> 0, above -> identity
// A step that is a power of two (the table of the command line: 8 / 1024) has an exact reciprocal: the product equals the
// quotient bit for bit and saves the IEEE division.
__device__ __forceinline__ float gelu_lut(float x, const float *lut, float gmin, float geps, int size) {
	const bool pow2 = (__float_as_uint(geps) & 0x007fffffu) == 0u && geps > 1e-30f && geps < 1e30f;
	const float ginv = __uint_as_float((254u << 23) - __float_as_uint(geps));  // 2^-e for geps = 2^e
	int idx = pow2 ? (int)((x - gmin) * ginv) : (int)((x - gmin) / geps);
	if (idx < 0) return 0.0f;
	if (idx >= size) return x;
	return lut[idx];
}

__device__ __forceinline__ void fma16(float acc[4], const i32x4 v, const f32x4 xv) {
	const int d0 = v.x, d1 = v.y, d2 = v.z, d3 = v.w;
	acc[0] = fmaf(xv.x, b2f(d0, 0), acc[0]); acc[0] = fmaf(xv.y, b2f(d0, 1), acc[0]);
	acc[0] = fmaf(xv.z, b2f(d0, 2), acc[0]); acc[0] = fmaf(xv.w, b2f(d0, 3), acc[0]);
	acc[1] = fmaf(xv.x, b2f(d1, 0), acc[1]); acc[1] = fmaf(xv.y, b2f(d1, 1), acc[1]);
	acc[1] = fmaf(xv.z, b2f(d1, 2), acc[1]); acc[1] = fmaf(xv.w, b2f(d1, 3), acc[1]);
	acc[2] = fmaf(xv.x, b2f(d2, 0), acc[2]); acc[2] = fmaf(xv.y, b2f(d2, 1), acc[2]);
	acc[2] = fmaf(xv.z, b2f(d2, 2), acc[2]); acc[2] = fmaf(xv.w, b2f(d2, 3), acc[2]);
	acc[3] = fmaf(xv.x, b2f(d3, 0), acc[3]); acc[3] = fmaf(xv.y, b2f(d3, 1), acc[3]);
	acc[3] = fmaf(xv.z, b2f(d3, 2), acc[3]); acc[3] = fmaf(xv.w, b2f(d3, 3), acc[3]);
}

// Second stage of the greedy argmax over n per-workgroup (maximum, index) pairs: every thread of the workgroup gets
// the winner (ops.hpp:749-757: strict '>' from index 0, so the lowest index wins ties; no comparison is true for a
// row of NaN and the index stays at the reference's initial -1).  s_bv / s_bi: NWAVE entries of LDS.
__device__ __forceinline__ int argmax_pairs(const float *blk_val, const int *blk_idx, int n, float *s_bv, int *s_bi) {
	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	float bv = -INFINITY;
	int bi = 0x7fffffff;
	// all loads first (clamped indices, no branches), then the comparisons: one memory round trip instead of one per pass
	for (int i0 = 0; i0 < n; i0 += 8 * NT) {
		float ovs[8];
		int ois[8];
#pragma unroll
		for (int u = 0; u < 8; u++) {
			const int i = i0 + u * NT + tid, ic = i < n ? i : n - 1;
			ovs[u] = blk_val[ic];
			ois[u] = blk_idx[ic];
		}
#pragma unroll
		for (int u = 0; u < 8; u++) {
			const bool in = i0 + u * NT + tid < n;
			if (in && (ovs[u] > bv || (ovs[u] == bv && ois[u] < bi))) { bv = ovs[u]; bi = ois[u]; }
		}
	}
#define TG_STEP(O)                                                      \
	{                                                                   \
		const float ov = tg_red_partner<O>(bv);                         \
		const int oi = tg_red_partner<O>(bi);                           \
		if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }     \
	}
	TG_STEP(32) TG_STEP(16) TG_STEP(8) TG_STEP(4) TG_STEP(2) TG_STEP(1)
#undef TG_STEP
	if (lane == 0) { s_bv[w] = bv; s_bi[w] = bi; }
	__syncthreads();
	bv = s_bv[0];
	bi = s_bi[0];
	for (int i = 1; i < NWAVE; i++)
		if (s_bv[i] > bv || (s_bv[i] == bv && s_bi[i] < bi)) { bv = s_bv[i]; bi = s_bi[i]; }
	return bi == 0x7fffffff ? -1 : bi;
}

// Per-token bookkeeping once the pick is known: it becomes the next step's input token, is appended to the id log, and
// KVCache::update_single's counters (decode.hpp:68-69) advance once per token.  One thread.
__device__ __forceinline__ void record_pick(int tok, int *ctr, int *tok_log, int advance) {
	ctr[4] = tok;
	const int st = ctr[3];
	tok_log[st] = tok;
	ctr[3] = st + 1;
	if (advance) {
		ctr[0] += 1;
		ctr[1] += 1;
		ctr[2] += 1;
	}
}

// ---- pieces of the prologues and epilogues, as functions so that every caller rounds the same way ----
constexpr int PER = (TG_MAX_HIDDEN + NT - 1) / NT;  // elements of the residual stream per lane (element d = tid + i * NT)

// scalar store, optionally write-through at device scope: for a consumer inside the same kernel on another XCD, and for
// the outputs of the decode launches, which then leave no dirty line in the L2s for the end of the kernel to write back
// (+0.2 ... 0.5 % decode speed; every consumer runs in a later launch, on any XCD)
template <bool WT>
__device__ __forceinline__ void st_f32(float *p, float v) {
	if (WT) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	else *p = v;
}

__device__ __forceinline__ float sumsq(const float (&v)[PER]) {
	float ss = 0.0f;
#pragma unroll
	for (int i = 0; i < PER; i++) ss = fmaf(v[i], v[i], ss);  // lanes past the vector hold 0
	return ss;
}
// ops.hpp:126-180: 1 / sqrt(mean(x^2) + eps) from the sum of squares.  v_rsq_f32 (1 ulp) instead of an IEEE square root
// and an IEEE division: those are two chains of a dozen dependent instructions in every norm, and every decode launch
// with a norm prologue has two norms in front of its first product (1,594 -> 1,625 tok/s, same picks).
__device__ __forceinline__ float rms_inv(float ss, int h) { return __builtin_amdgcn_rsqf(ss * (1.0f / (float)h) + 1e-06f); }
// modules.hpp:166-168 / 218-219: x = rmsnorm(block_out, post) + residual
__device__ __forceinline__ void post_norm_add(float (&t)[PER], const float (&p)[PER], float irms, const float (&wpo)[PER], const float (&r)[PER]) {
#pragma unroll
	for (int i = 0; i < PER; i++) t[i] = (p[i] * irms) * (wpo[i] + 1.0f) + r[i];
}
// x * rsqrt(mean(x^2) + eps) * (1 + w) into the workgroup's input vector
__device__ __forceinline__ void pre_norm_store(float *xs, const float (&t)[PER], float irms, const float (&wpre)[PER], int h) {
#pragma unroll
	for (int i = 0; i < PER; i++) {
		const int d = threadIdx.x + i * NT;
		if (d < h) xs[d] = (t[i] * irms) * (wpre[i] + 1.0f);
	}
}
// ops.hpp:537-568: one element of the embedding row, s[d] * (sqrt(hidden) * q)
__device__ __forceinline__ float embed_value(float scale, float emb_scale, int8_t q) { return scale * (emb_scale * (float)q); }

// Merge of the flash-decoding partials of the attention that precedes an output projection:
//   out_h = sum_b acc_{b,h} * exp(m_{b,h} - M_h) / sum_b l_{b,h} * exp(m_{b,h} - M_h)
// into xs[4][256].  Wave w merges head w; a lane owns 4 consecutive dims: 16 loads of 16 bytes instead of 64 of 4.
// after_loads() is called once the partials have been requested.  wgt: [4][TG_ATTN_MERGE_MAX] of LDS.
template <class F>
__device__ __forceinline__ void attn_merge_prologue(float *xs, float (*wgt)[TG_ATTN_MERGE_MAX], const float *part_acc, const float *part_ml, int nb,
                                                    F after_loads) {
	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	f32x4 a[TG_ATTN_MERGE_MAX];
	float m = -INFINITY, l = 0.0f;
	if (tid < 4 * TG_ATTN_MERGE_MAX && (tid % TG_ATTN_MERGE_MAX) < nb) {
		const int h = tid / TG_ATTN_MERGE_MAX, b = tid % TG_ATTN_MERGE_MAX;
		m = part_ml[((size_t)b * 4 + h) * 2];
		l = part_ml[((size_t)b * 4 + h) * 2 + 1];
	}
#pragma unroll
	for (int b = 0; b < TG_ATTN_MERGE_MAX; b++) {
		// unconditional load from a clamped index, select afterwards: a load under a branch is waited for
		// at the end of that branch, which would turn these loads into as many round trips
		const int bb = b < nb ? b : 0;
		const f32x4 val = *reinterpret_cast<const f32x4 *>(part_acc + ((size_t)bb * 4 + w) * 256 + 4 * lane);
		a[b] = (b < nb) ? val : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
	}
	after_loads();
	if (tid < 4 * TG_ATTN_MERGE_MAX) {
		const int h = tid / TG_ATTN_MERGE_MAX, b = tid % TG_ATTN_MERGE_MAX;
		const bool ok = b < nb;
		static_assert(TG_ATTN_MERGE_MAX == 16, "one row of 16 lanes per head");
		const float M = tg_row16_max(m);
		const float e = ok ? __builtin_amdgcn_exp2f((m - M) * 1.44269504088896341f) : 0.0f;  // as the attention kernel's weights
		// __fmul_rn: the product must be rounded before the reduction; contracted into the first add
		// (fma(l, e, partner)) the two lanes of a pair would no longer hold the same sum
		const float L = tg_row16_sum(__fmul_rn(l, e));
		wgt[h][b] = e * __builtin_amdgcn_rcpf(L);  // v_rcp_f32 (1 ulp) instead of an IEEE division in front of the product
	}
	__syncthreads();
	{
		f32x4 o = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
		for (int b = 0; b < TG_ATTN_MERGE_MAX; b++) {
			const float wb = wgt[w][b];
#pragma unroll
			for (int e = 0; e < 4; e++) o[e] = fmaf(a[b][e], wb, o[e]);
		}
		*reinterpret_cast<f32x4 *>(&xs[w * 256 + 4 * lane]) = o;
	}
	__syncthreads();
}

// Reduction over the lanes along K (fixed order): lanes l and l' hold partial sums of the same columns iff
// l % LC == l' % LC.  Then lane < LC of every wave leaves its 4 columns in red[wave].
__device__ __forceinline__ void lanes_reduce(float (&acc)[4], int LC, float (*red)[TG_CT]) {
#define TG_STEP(O)                                                   \
	if (LC <= O) {                                                   \
		_Pragma("unroll") for (int j = 0; j < 4; j++) acc[j] += tg_red_partner<O>(acc[j]); \
	}
	TG_STEP(32) TG_STEP(16) TG_STEP(8) TG_STEP(4) TG_STEP(2) TG_STEP(1)
#undef TG_STEP
	const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
	if (lane < LC) *reinterpret_cast<float4 *>(&red[w][lane * 4]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
}
// Epilogues of tile `cur` (after the barrier that follows lanes_reduce): the four waves' sums in a fixed order, the column
// scale applied once (linalg.hpp:83-107).
template <bool WT>
__device__ __forceinline__ void epi_store(const float (*red)[TG_CT], int C, int cur, float sc, float *y) {
	const int tid = threadIdx.x;
	if (tid < C) {
		const int col = cur * C + tid;
		const float sum = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
		st_f32<WT>(&y[col], sum * sc);
	}
}
// modules.hpp:211-215: gelu(gate) * up; the tile holds C/2 up columns, then the same C/2 gate columns
template <bool WT>
__device__ __forceinline__ void epi_geglu(const float (*red)[TG_CT], int C, int cur, float sc_up, float sc_gate, float *y, const float *lut, float gmin,
                                          float geps, int lut_size) {
	const int tid = threadIdx.x, C2 = C >> 1;
	if (tid < C2) {
		const float su = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
		const float sg = (red[0][tid + C2] + red[1][tid + C2]) + (red[2][tid + C2] + red[3][tid + C2]);
		const float up = su * sc_up;
		const float gate = sg * sc_gate;
		st_f32<WT>(&y[cur * C2 + tid], gelu_lut(gate, lut, gmin, geps, lut_size) * up);
	}
}

}  // namespace tgp

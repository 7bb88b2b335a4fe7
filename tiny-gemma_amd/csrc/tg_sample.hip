// min-p / temperature sampling on the device, replacing ops::minp_logits (ops.hpp:762-859): the second
// branch of gemma::generate (transformer.hpp:208-211, 232-235).
//
// What the reference computes, in order (and what is kept here):
//   1. logits /= temp                                                         (ops.hpp:767-769)
//   2. p_i = exp(l_i - max l)                maxp = max p_i                  (ops.hpp:773-799)
//   3. denom = sum of the p_i that are >= minp * maxp                         (ops.hpp:801-834)
//   4. p_i *= float(1.0 / denom) for EVERY i: the reference masks the small p_i only inside the
//      denominator loop and never stores the mask, so tokens below the cut keep their
//      (now over-normalised) probability and can still be drawn                (ops.hpp:836-846)
//   5. index = first idx whose running sum of p reaches randf, 0 if none does (ops.hpp:848-858)
// The reference sums sequentially in fp32 (vocab = 262144 terms); here the sums are blocked, so an index
// can differ from the reference's only where randf lies within fp32 summation error of a boundary of the
// cumulative distribution.
//
// Three launches per token: block maxima; probabilities + masked block sums + sums of 256-element
// segments; one workgroup that finds the crossing segment, re-scans it and does the per-token bookkeeping
// tg_argmax_finish does on the greedy branch.

#include "tg_internal.h"

namespace {

constexpr int SNT = 256;     // threads per workgroup of the first two kernels
constexpr int SEG = 256;     // elements per segment (one wave, 4 consecutive elements per lane)
constexpr int SCHUNK = 1024; // elements per workgroup: 4 segments
constexpr int FNT = 1024;    // threads of the finishing workgroup
constexpr int NONE = 0x7fffffff;

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_max(float v) { return tg_wave_max(v); }
__device__ __forceinline__ float wave_sum(float v) { return tg_wave_sum(v); }

// bmax[b] = max over the workgroup's 1024 elements of logits[i] / temp
__global__ __launch_bounds__(SNT) void minp_max_kernel(const float *logits, float temp, float *bmax) {
	__shared__ float sm[SNT / 64];
	const int tid = threadIdx.x;
	const f32x4 l = *reinterpret_cast<const f32x4 *>(logits + (size_t)blockIdx.x * SCHUNK + 4 * tid);
	float m = fmaxf(fmaxf(l[0] / temp, l[1] / temp), fmaxf(l[2] / temp, l[3] / temp));
	m = wave_max(m);
	if ((tid & 63) == 0) sm[tid >> 6] = m;
	__syncthreads();
	if (tid == 0) bmax[blockIdx.x] = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
}

// probs[i] = exp(logits[i] / temp - rowmax); seg[s] = sum of segment s; bsum[b] = sum of the workgroup's
// probabilities that are >= cut.  maxp is exp(0) = 1 (the maximum element itself), so cut = minp.
__global__ __launch_bounds__(SNT) void minp_prob_kernel(const float *logits, float temp, float minp, const float *bmax, int nblocks,
                                                        float *probs, float *seg, float *bsum) {
	__shared__ float sm[SNT / 64], ss[SNT / 64];
	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	const f32x4 l = *reinterpret_cast<const f32x4 *>(logits + (size_t)blockIdx.x * SCHUNK + 4 * tid);
	float m = -INFINITY;
	for (int i = tid; i < nblocks; i += SNT) m = fmaxf(m, bmax[i]);
	m = wave_max(m);
	if (lane == 0) sm[w] = m;
	__syncthreads();
	const float rowmax = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
	const float cut = minp * 1.0f;
	f32x4 p;
	float all = 0.0f, kept = 0.0f;
#pragma unroll
	for (int e = 0; e < 4; e++) {
		p[e] = expf(l[e] / temp - rowmax);
		all += p[e];
		kept += (p[e] < cut) ? 0.0f : p[e];
	}
	*reinterpret_cast<f32x4 *>(probs + (size_t)blockIdx.x * SCHUNK + 4 * tid) = p;
	all = wave_sum(all);
	kept = wave_sum(kept);
	if (lane == 0) {
		seg[blockIdx.x * (SCHUNK / SEG) + w] = all;
		ss[w] = kept;
	}
	__syncthreads();
	if (tid == 0) bsum[blockIdx.x] = (ss[0] + ss[1]) + (ss[2] + ss[3]);
}

// One workgroup: denominator, scan of the segment sums, re-scan of the crossing segment, bookkeeping.
//   mode 0: decode step  — token -> ctr[4], appended to tok_log, position counters advance
//   mode 1: prefill      — replaces the token the greedy finish wrote last (ctr[4], tok_log[ctr[3] - 1])
//   mode 2: stand-alone  — token -> out_tok only
// randf: the draw of this token is randf[rand_idx], or randf[ctr[3] - rand_base] when rand_idx < 0.
__global__ __launch_bounds__(FNT) void minp_finish_kernel(const float *probs, const float *seg, const float *bsum, int nblocks, int nseg,
                                                          const float *randf, int rand_idx, int rand_base, int *ctr, int *tok_log,
                                                          int mode, int *out_tok) {
	__shared__ float s_w[FNT / 64];
	__shared__ float s_scan[FNT / 64];
	__shared__ int s_seg;
	__shared__ float s_start, s_inv;
	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;

	// denominator: fixed-order sum of the masked block sums
	float d = 0.0f;
	for (int i = tid; i < nblocks; i += FNT) d += bsum[i];
	d = wave_sum(d);
	if (lane == 0) s_w[w] = d;
	if (tid == 0) s_seg = NONE;
	__syncthreads();
	if (tid == 0) {
		float denom = 0.0f;
		for (int i = 0; i < FNT / 64; i++) denom += s_w[i];
		s_inv = (float)(1.0 / (double)denom);  // ops.hpp:836
	}
	__syncthreads();
	const float inv = s_inv;
	int ri = rand_idx;
	if (ri < 0) ri = ctr[3] - rand_base - (mode == 1 ? 1 : 0);
	const float r = randf[ri];

	// running sum over the segments, FNT at a time (nseg <= FNT for a 262144-entry vocabulary)
	float base = 0.0f;
	for (int s0 = 0; s0 < nseg && s_seg == NONE; s0 += FNT) {
		const int s = s0 + tid;
		const float q = (s < nseg) ? seg[s] * inv : 0.0f;
		// inclusive scan inside the wave, then across the 16 waves
		float incl = q;
#pragma unroll
		for (int o = 1; o < 64; o <<= 1) {
			const float t = __shfl_up(incl, o, 64);
			if (lane >= o) incl += t;
		}
		if (lane == 63) s_scan[w] = incl;
		__syncthreads();
		float woff = base;
		for (int i = 0; i < w; i++) woff += s_scan[i];
		const float end = woff + incl, start = end - q;
		// the crossing segment is the first one whose running sum reaches r, as in the sequential scan
		if (s < nseg && end >= r) atomicMin(&s_seg, s);
		float total = base;
		for (int i = 0; i < FNT / 64; i++) total += s_scan[i];
		__syncthreads();
		if (s_seg == s) s_start = start;
		base = total;
		__syncthreads();
	}

	int token = 0;  // ops.hpp:850: index stays 0 when the running sum never reaches randf
	const int cs = s_seg;
	if (cs != NONE && w == 0) {
		// re-scan the crossing segment with the stored probabilities: 4 consecutive elements per lane
		const f32x4 p = *reinterpret_cast<const f32x4 *>(probs + (size_t)cs * SEG + 4 * lane);
		const float q0 = p[0] * inv, q1 = p[1] * inv, q2 = p[2] * inv, q3 = p[3] * inv;
		const float lsum = ((q0 + q1) + q2) + q3;
		float incl = lsum;
#pragma unroll
		for (int o = 1; o < 64; o <<= 1) {
			const float t = __shfl_up(incl, o, 64);
			if (lane >= o) incl += t;
		}
		float c = s_start + (incl - lsum);
		int first = NONE;
		c += q0;
		if (c >= r) first = 4 * lane;
		c += q1;
		if (c >= r && first == NONE) first = 4 * lane + 1;
		c += q2;
		if (c >= r && first == NONE) first = 4 * lane + 2;
		c += q3;
		if (c >= r && first == NONE) first = 4 * lane + 3;
#pragma unroll
		for (int o = 32; o > 0; o >>= 1) first = min(first, __shfl_xor(first, o, 64));
		if (first == NONE) first = SEG - 1;  // rounding: the segment's end reached r, its re-scan did not
		token = cs * SEG + first;
	}
	if (tid == 0) {
		if (out_tok) *out_tok = token;
		if (mode == 0) {
			ctr[4] = token;
			const int st = ctr[3];
			tok_log[st] = token;
			ctr[3] = st + 1;
			ctr[0] += 1;
			ctr[1] += 1;
			ctr[2] += 1;
		} else if (mode == 1) {
			ctr[4] = token;
			tok_log[ctr[3] - 1] = token;
		}
	}
}

}  // namespace

size_t tg_minp_blocks(int n) { return (size_t)n / SCHUNK; }
size_t tg_minp_segments(int n) { return (size_t)n / SEG; }

// logits[n] (n a multiple of 1024) -> token; probs[n], seg[n/256], bsum[n/1024], bmax[n/1024] are scratch
void tg_launch_minp(const float *logits, int n, float minp, float temp, const float *randf, int rand_idx, int rand_base, float *probs,
                    float *seg, float *bsum, float *bmax, int *ctr, int *tok_log, int mode, int *out_tok, hipStream_t s) {
	const int nb = n / SCHUNK, nseg = n / SEG;
	hipLaunchKernelGGL(minp_max_kernel, dim3((unsigned)nb), dim3(SNT), 0, s, logits, temp, bmax);
	hipLaunchKernelGGL(minp_prob_kernel, dim3((unsigned)nb), dim3(SNT), 0, s, logits, temp, minp, bmax, nb, probs, seg, bsum);
	hipLaunchKernelGGL(minp_finish_kernel, dim3(1), dim3(FNT), 0, s, probs, seg, bsum, nb, nseg, randf, rand_idx, rand_base, ctr, tok_log,
	                   mode, out_tok);
}

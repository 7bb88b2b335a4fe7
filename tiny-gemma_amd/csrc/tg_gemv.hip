// Decode-side int8 weight-only GEMV for gfx950 (wave64).
//
// Replaces gemv::qgemv / gemv::qgemv_row_tile (csrc/include/linalg.hpp:41-174 of the reference):
//     y[c] = scales[c] * sum_r x[r] * float(W[r][c])
// with the scale applied once after the whole fp32 reduction (linalg.hpp:83-107).
//
// Work decomposition: grid = (128-column tiles) x (K splits).  Inside a workgroup every lane
// streams 16-byte pieces of the packed tile (4 columns x 4 input rows, see tg_internal.h),
// converts each byte with one sign-extending convert, and keeps one fp32 accumulator per column;
// lanes 0-31 and 32-63 of a wave take alternating row groups.  The lane/wave partials are summed
// through LDS in a fixed order; when the reduction is split over several workgroups the partial
// sums go through a small HBM workspace and the last workgroup to finish (ticket counter) adds
// them in a fixed order and runs the epilogue, so results are run-to-run deterministic.
//
// Prologues fold the work that precedes a projection in modules::attention / modules::mlp
// (modules.hpp:135-220) into the same launch: embedding gather, post-norm + residual add of the
// previous block, pre-norm.  Epilogues fold what follows it: LUT-GeLU(gate) * up, or logits
// write-out plus greedy argmax.

#include "tg_internal.h"

namespace {

constexpr int NW = 4;          // waves per workgroup
constexpr int NT = NW * 64;    // threads per workgroup
constexpr int UNROLL = 4;      // 16-byte loads in flight per lane

typedef int i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
	return v;
}

// Sum over the workgroup; every thread gets the same value (fixed order).
__device__ __forceinline__ float block_sum(float v, float *sred) {
	v = wave_sum(v);
	__syncthreads();
	if ((threadIdx.x & 63) == 0) sred[threadIdx.x >> 6] = v;
	__syncthreads();
	float t = 0.0f;
#pragma unroll
	for (int i = 0; i < NW; i++) t += sred[i];
	return t;
}

__device__ __forceinline__ float b2f(int d, int j) {  // signed byte j of d -> float (exact)
	return (float)(int8_t)(d >> (8 * j));
}

// ops.hpp:41-51: truncating index, below the table -> 0, above -> identity
__device__ __forceinline__ float gelu_lut(float x, const float *lut, float gmin, float geps, int size) {
	int idx = (int)((x - gmin) / geps);
	if (idx < 0) return 0.0f;
	if (idx >= size) return x;
	return lut[idx];
}

__global__ __launch_bounds__(NT) void gemv_kernel(const TgGemv g) {
	__shared__ float xs[TG_MAX_K];
	__shared__ float red[NW * 2 * TG_CT];
	__shared__ float sred[NW];
	__shared__ unsigned s_ticket;
	__shared__ float s_bv[NW];
	__shared__ int s_bi[NW];

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	const int tile = blockIdx.x, ks = blockIdx.y;

	// ---------------- prologue: input vector into LDS ----------------
	if (g.pro == TG_PRO_PLAIN) {
		const int r0 = ks * g.pairs_per_block * 8, n = g.pairs_per_block * 8;
		for (int i = tid; i < n; i += NT) xs[r0 + i] = g.x[r0 + i];
	} else {
		const int h = g.hidden;
		const float eps = 1e-06f;
		if (g.pro == TG_PRO_EMBED) {
			// ops.hpp:537-568: s[d] * (sqrt(hidden) * q)
			int tok = *g.tok;
			tok = tok < 0 ? 0 : (tok >= g.vocab ? g.vocab - 1 : tok);
			const int8_t *row = g.wte + (size_t)tok * h;
			for (int d = tid; d < h; d += NT) xs[d] = g.wte_scales[d] * (g.emb_scale * (float)row[d]);
		} else if (g.pro == TG_PRO_NORM) {
			for (int d = tid; d < h; d += NT) xs[d] = g.x[d];
		} else {
			// modules.hpp:166-168 / 218-219: x = rmsnorm(block_out, post) + residual
			float ss = 0.0f;
			for (int d = tid; d < h; d += NT) {
				float p = g.pend[d];
				xs[d] = p;
				ss = fmaf(p, p, ss);
			}
			ss = block_sum(ss, sred);
			const float irms = 1.0f / sqrtf(ss / (float)h + eps);
			for (int d = tid; d < h; d += NT) xs[d] = (xs[d] * irms) * (g.w_post[d] + 1.0f) + g.x[d];
		}
		if (g.xr_out != nullptr && tile == 0 && ks == 0)
			for (int d = tid; d < h; d += NT) g.xr_out[d] = xs[d];
		// ops.hpp:126-180: x * rsqrt(mean(x^2) + eps) * (1 + w)
		float ss = 0.0f;
		for (int d = tid; d < h; d += NT) ss = fmaf(xs[d], xs[d], ss);
		ss = block_sum(ss, sred);
		const float irms = 1.0f / sqrtf(ss / (float)h + eps);
		for (int d = tid; d < h; d += NT) xs[d] = (xs[d] * irms) * (g.w_pre[d] + 1.0f);
	}
	__syncthreads();

	// ---------------- main loop: stream the packed tile ----------------
	const int half = lane >> 5, cl = lane & 31;
	const int kgs = g.K >> 2;
	const i32x4 *Wt = reinterpret_cast<const i32x4 *>(g.W) + (size_t)tile * kgs * (TG_CT / 4);
	const int p0 = ks * g.pairs_per_block;
	const int np = (g.pairs_per_block - w + NW - 1) / NW;  // pairs p0 + w, p0 + w + NW, ...
	float acc0 = 0.0f, acc1 = 0.0f, acc2 = 0.0f, acc3 = 0.0f;
	for (int i = 0; i < np; i += UNROLL) {
		i32x4 v[UNROLL];
		int kg[UNROLL];
#pragma unroll
		for (int u = 0; u < UNROLL; u++) {
			const bool ok = (i + u) < np;
			kg[u] = ok ? 2 * (p0 + w + (i + u) * NW) + half : 2 * p0;
			v[u] = ok ? __builtin_nontemporal_load(Wt + (size_t)kg[u] * (TG_CT / 4) + cl) : i32x4{0, 0, 0, 0};
		}
#pragma unroll
		for (int u = 0; u < UNROLL; u++) {
			const float4 xv = *reinterpret_cast<const float4 *>(&xs[4 * kg[u]]);
			const int d0 = v[u].x, d1 = v[u].y, d2 = v[u].z, d3 = v[u].w;
			acc0 = fmaf(xv.x, b2f(d0, 0), acc0); acc0 = fmaf(xv.y, b2f(d0, 1), acc0);
			acc0 = fmaf(xv.z, b2f(d0, 2), acc0); acc0 = fmaf(xv.w, b2f(d0, 3), acc0);
			acc1 = fmaf(xv.x, b2f(d1, 0), acc1); acc1 = fmaf(xv.y, b2f(d1, 1), acc1);
			acc1 = fmaf(xv.z, b2f(d1, 2), acc1); acc1 = fmaf(xv.w, b2f(d1, 3), acc1);
			acc2 = fmaf(xv.x, b2f(d2, 0), acc2); acc2 = fmaf(xv.y, b2f(d2, 1), acc2);
			acc2 = fmaf(xv.z, b2f(d2, 2), acc2); acc2 = fmaf(xv.w, b2f(d2, 3), acc2);
			acc3 = fmaf(xv.x, b2f(d3, 0), acc3); acc3 = fmaf(xv.y, b2f(d3, 1), acc3);
			acc3 = fmaf(xv.z, b2f(d3, 2), acc3); acc3 = fmaf(xv.w, b2f(d3, 3), acc3);
		}
	}

	// ---------------- workgroup reduction (fixed order) ----------------
	*reinterpret_cast<float4 *>(&red[(w * 2 + half) * TG_CT + cl * 4]) = make_float4(acc0, acc1, acc2, acc3);
	__syncthreads();
	float sum = 0.0f;
	if (tid < TG_CT) {
#pragma unroll
		for (int i = 0; i < NW * 2; i++) sum += red[i * TG_CT + tid];
	}

	// ---------------- cross-workgroup reduction ----------------
	const int group_n = g.KS * g.tpc;
	int t_first = tile, t_count = 1;
	float val[2] = {sum, 0.0f};
	if (group_n > 1) {
		if (tid < TG_CT) g.partial[((size_t)tile * g.KS + ks) * TG_CT + tid] = sum;
		__threadfence();
		__syncthreads();
		if (tid == 0) s_ticket = atomicAdd(&g.counters[tile / g.tpc], 1u);
		__syncthreads();
		if (s_ticket != (unsigned)(group_n - 1)) return;
		__threadfence();
		t_first = (tile / g.tpc) * g.tpc;
		t_count = g.tpc;
		if (tid < TG_CT) {
			for (int t = 0; t < t_count; t++) {
				float s = 0.0f;
				const float *pp = g.partial + (size_t)(t_first + t) * g.KS * TG_CT + tid;
				for (int k = 0; k < g.KS; k++) s += __builtin_nontemporal_load(pp + (size_t)k * TG_CT);
				val[t] = s;
			}
		}
		if (tid == 0) g.counters[tile / g.tpc] = 0u;
	}

	// ---------------- epilogue ----------------
	if (g.epi == TG_EPI_STORE) {
		if (tid < TG_CT) {
			const int col = t_first * TG_CT + tid;
			g.y[col] = val[0] * g.scales[col];
		}
		return;
	}
	if (g.epi == TG_EPI_GEGLU) {
		// modules.hpp:211-215: gelu(gate) * up ; tiles (2t, 2t+1) hold up | gate columns of block t
		if (tid < TG_CT) {
			const float up = val[0] * g.scales[t_first * TG_CT + tid];
			const float gate = val[1] * g.scales[(t_first + 1) * TG_CT + tid];
			g.y[(t_first / 2) * TG_CT + tid] = gelu_lut(gate, g.lut, g.gmin, g.geps, g.lut_size) * up;
		}
		return;
	}
	// TG_EPI_LOGITS: logits + greedy argmax (ops.hpp:749-757: strict '>' from index 0 => lowest index wins)
	float bv = -INFINITY;
	int bi = 0x7fffffff;
	if (tid < TG_CT) {
		const int col = t_first * TG_CT + tid;
		const float v = val[0] * g.scales[col];
		if (g.y != nullptr) g.y[col] = v;
		if (v > bv) { bv = v; bi = col; }
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) {
		const float ov = __shfl_xor(bv, o, 64);
		const int oi = __shfl_xor(bi, o, 64);
		if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
	}
	if (lane == 0) { s_bv[w] = bv; s_bi[w] = bi; }
	__syncthreads();
	if (tid == 0) {
		for (int i = 1; i < NW; i++)
			if (s_bv[i] > bv || (s_bv[i] == bv && s_bi[i] < bi)) { bv = s_bv[i]; bi = s_bi[i]; }
		g.blk_val[tile] = bv;
		g.blk_idx[tile] = bi;
	}
	__threadfence();
	__syncthreads();
	if (tid == 0) s_ticket = atomicAdd(g.argmax_counter, 1u);
	__syncthreads();
	if (s_ticket != (unsigned)(g.ntiles * g.KS / group_n - 1)) return;
	__threadfence();
	bv = -INFINITY;
	bi = 0x7fffffff;
	for (int i = tid; i < g.ntiles; i += NT) {
		const float ov = __builtin_nontemporal_load(g.blk_val + i);
		const int oi = __builtin_nontemporal_load(g.blk_idx + i);
		if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) {
		const float ov = __shfl_xor(bv, o, 64);
		const int oi = __shfl_xor(bi, o, 64);
		if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
	}
	__syncthreads();
	if (lane == 0) { s_bv[w] = bv; s_bi[w] = bi; }
	__syncthreads();
	if (tid == 0) {
		for (int i = 1; i < NW; i++)
			if (s_bv[i] > bv || (s_bv[i] == bv && s_bi[i] < bi)) { bv = s_bv[i]; bi = s_bi[i]; }
		if (bi == 0x7fffffff) bi = -1;  // all NaN: the reference's scan leaves -1 (ops.hpp:750)
		*g.argmax_counter = 0u;
		*g.tok_out = bi;
		if (g.step != nullptr) {
			const int st = *g.step;
			if (g.tok_log != nullptr) g.tok_log[st] = bi;
			*g.step = st + 1;
		}
		if (g.pos != nullptr) {  // KVCache::update_single's counters (decode.hpp:68-69), once per token
			g.pos[0] += 1;
			g.pos[1] += 1;
			g.pos[2] += 1;
		}
	}
}

}  // namespace

void tg_launch_gemv(const TgGemv &g, hipStream_t s) {
	dim3 grid((unsigned)g.ntiles, (unsigned)g.KS);
	hipLaunchKernelGGL(gemv_kernel, grid, dim3(NT), 0, s, g);
}

// Device-side body of the decode attention (tg_attn.hip), shared with the one-kernel decode step
// (tg_decode_fused.hip) so that both paths do the same arithmetic in the same order and give the same bits.
#pragma once

#include "tg_internal.h"

namespace tga {

constexpr int HD = 256;        // head_dim (config.hpp:47-48); checked on the host
constexpr int NH = 4;          // query heads sharing the single KV head
constexpr int ANT = 256;       // threads per workgroup
constexpr int MAXCHUNK = 256;  // keys per workgroup, upper bound

__device__ __forceinline__ float wsum(float v) { return tg_wave_sum(v); }
__device__ __forceinline__ float wmax(float v) { return tg_wave_max(v); }
__device__ __forceinline__ float sum16(float v) { return tg_row16_sum(v); }  // over aligned groups of 16 lanes

// One wave normalises and rotates one 256-wide head vector (ops.hpp:126-180, decode.hpp:136-211).
// Lane l owns dims {l, l+64, l+128, l+192}: both members of every rotation pair (d, d+128).
// cs/sn point at the [hd/2] table row of this token's position.  Split in two so that a caller can put
// all of the loads in front of other, bulkier loads: the wait for a load also waits for every load
// issued before it.
struct HeadIn {
	float x[4], w[4], c0, c1, s0, s1;
};
__device__ __forceinline__ void head_load(HeadIn &in, const float *src, const float *w, const float *cs, const float *sn, int lane) {
#pragma unroll
	for (int i = 0; i < 4; i++) in.x[i] = src[lane + 64 * i];
#pragma unroll
	for (int i = 0; i < 4; i++) in.w[i] = w[lane + 64 * i];
	in.c0 = cs[lane];
	in.c1 = cs[lane + 64];
	in.s0 = sn[lane];
	in.s1 = sn[lane + 64];
}
__device__ __forceinline__ void head_finish(const HeadIn &in, float mul, float out[4]) {
	float x[4];
	float ss = 0.0f;
#pragma unroll
	for (int i = 0; i < 4; i++) ss = fmaf(in.x[i], in.x[i], ss);
	ss = wsum(ss);
	const float irms = 1.0f / sqrtf(ss / (float)HD + 1e-06f);
#pragma unroll
	for (int i = 0; i < 4; i++) x[i] = (in.x[i] * irms) * (in.w[i] + 1.0f);
	out[0] = fmaf(in.c0, x[0], (-x[2]) * in.s0) * mul;
	out[1] = fmaf(in.c1, x[1], (-x[3]) * in.s1) * mul;
	out[2] = fmaf(in.c0, x[2], x[0] * in.s0) * mul;
	out[3] = fmaf(in.c1, x[3], x[1] * in.s1) * mul;
}
__device__ __forceinline__ void norm_rope_head(const float *src, const float *w, const float *cs, const float *sn, float mul,
                                               float out[4], int lane) {
	HeadIn in;
	head_load(in, src, w, cs, sn, lane);
	head_finish(in, mul, out);
}

// Keys of a chunk whose K rows / V elements are fetched before anything else in the kernel (the rest, for
// chunks longer than this, is fetched inside the loops).
constexpr int PRE = 32;

// WT: the partials are stored write-through at device scope (for a consumer inside the same kernel on another XCD)
template <bool WT>
__device__ __forceinline__ void attn_store(float *p, float v) {
	if (WT) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	else *p = v;
}

// One workgroup's chunk b of the keys: q/k norm + RoPE, cache write (chunk 0), scores, softmax partial, P.V.
// after_loads() is called once the body has issued its up-front loads.
template <bool WT, class F>
__device__ __forceinline__ void attn_decode_body(const TgAttnDecode &a, int b, F after_loads) {
	__shared__ __attribute__((aligned(16))) float qs[NH][HD];
	__shared__ __attribute__((aligned(16))) float knew[HD];
	__shared__ __attribute__((aligned(16))) float vnew[HD];
	__shared__ __attribute__((aligned(16))) float sc[NH][MAXCHUNK];
	__shared__ __attribute__((aligned(16))) float pv[ANT / 64][NH][HD];  // per-wave partial outputs of the first PRE keys
	__shared__ float s_m[NH], s_l[NH];

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, sub = lane >> 4, sl = lane & 15;
	const int pos = a.host_pos >= 0 ? a.host_pos : a.pos[0];          // position_ptr before this token (decode.hpp:154)
	const int bp = a.host_bp >= 0 ? a.host_bp : a.pos[a.bp_index];    // buffer_ptr before this token (decode.hpp:59)
	const int cur = bp % a.max_pos;
	const int valid = (pos + 1 < a.max_pos) ? pos + 1 : a.max_pos;  // decode.hpp:45-47 after update_single
	const int nb = (valid + a.chunk - 1) / a.chunk;
	if (b >= nb) return;
	const int k0 = b * a.chunk;
	const int n = (valid - k0 < a.chunk) ? valid - k0 : a.chunk;

	// Everything is requested up front.  The few values the q/k path needs go first (the previous launch's
	// q|k|v vector, norm weights, RoPE row): a wait for them must not include the cache rows behind them.
	HeadIn qin, kin;
	const float *cs = a.cos_t + (size_t)pos * (HD / 2), *sn = a.sin_t + (size_t)pos * (HD / 2);
	head_load(qin, a.qkv + w * HD, a.rms_q, cs, sn, lane);
	if (w == 0) head_load(kin, a.qkv + NH * HD, a.rms_k, cs, sn, lane);
	const float vnew_r = a.qkv[NH * HD + HD + tid];
	// Cache rows of the first PRE keys of this chunk: they depend on nothing computed here.
	// K: 16 lanes per key row (pass p covers keys 16p + 4w + sub); V: wave w takes keys 8w .. 8w+7, a lane 4 dims.
	float4 kpre[PRE / 16][4];
	float4 vpre[PRE / 4];
	// Rows are addressed as base + constant * row so that the 40 loads cost no per-load address arithmetic; rows
	// past the chunk (and slot `cur`, which workgroup 0 rewrites below) are fetched and ignored: every row index is
	// clamped into the cache, whose max_pos rows are all allocated.
	{
		const int lim = a.max_pos - 1 - k0;  // >= 0: last row of the cache, relative to the chunk
		const float *kbase = a.kc + (size_t)k0 * HD + sl * 4;
		const float *vbase = a.vc + (size_t)k0 * HD + 4 * lane;
#pragma unroll
		for (int p = 0; p < PRE / 16; p++) {
			int jj = 16 * p + w * 4 + sub;
			jj = jj < lim ? jj : lim;
			const float *kr = kbase + (size_t)jj * HD;
#pragma unroll
			for (int i = 0; i < 4; i++) kpre[p][i] = *reinterpret_cast<const float4 *>(kr + i * 64);
		}
#pragma unroll
		for (int u = 0; u < PRE / 4; u++) {
			const int jj = (PRE / 4) * w + u;
			vpre[u] = *reinterpret_cast<const float4 *>(vbase + (size_t)(jj < lim ? jj : lim) * HD);
		}
	}

	after_loads();  // the caller's own loads go out behind this body's: a wait for a load covers every load issued before it

	// q heads: one wave each; k: wave 0 again
	{
		float o[4];
		head_finish(qin, 0.0625f, o);  // ops.hpp:257: q *= 1/sqrt(256)
#pragma unroll
		for (int i = 0; i < 4; i++) qs[w][lane + 64 * i] = o[i];
		if (w == 0) {
			head_finish(kin, 1.0f, o);
#pragma unroll
			for (int i = 0; i < 4; i++) knew[lane + 64 * i] = o[i];
		}
		vnew[tid] = vnew_r;
	}
	__syncthreads();
	if (b == 0) {  // KVCache::update_single, decode.hpp:49-70
		a.kc[(size_t)cur * HD + tid] = knew[tid];
		a.vc[(size_t)cur * HD + tid] = vnew[tid];
	}

	// scores: q_h . k_j for the 4 heads; the token being decoded (slot cur) comes from knew
	{
		float4 q[NH][4];
#pragma unroll
		for (int h = 0; h < NH; h++)
#pragma unroll
			for (int i = 0; i < 4; i++) q[h][i] = *reinterpret_cast<const float4 *>(&qs[h][i * 64 + sl * 4]);
		auto pass = [&](int base, const float4 *kin) {
			const int jj = base + w * 4 + sub;
			const bool ok = jj < n;
			const int j = k0 + (ok ? jj : 0);
			float4 kv[4];
#pragma unroll
			for (int i = 0; i < 4; i++) kv[i] = (j == cur) ? *reinterpret_cast<const float4 *>(&knew[i * 64 + sl * 4]) : kin[i];
#pragma unroll
			for (int h = 0; h < NH; h++) {
				float d = 0.0f;
#pragma unroll
				for (int i = 0; i < 4; i++) {
					d = fmaf(q[h][i].x, kv[i].x, d);
					d = fmaf(q[h][i].y, kv[i].y, d);
					d = fmaf(q[h][i].z, kv[i].z, d);
					d = fmaf(q[h][i].w, kv[i].w, d);
				}
				d = sum16(d);
				if (ok && sl == 0) sc[h][jj] = d;
			}
		};
#pragma unroll
		for (int p = 0; p < PRE / 16; p++)
			if (16 * p < n) pass(16 * p, kpre[p]);
		for (int base = PRE; base < n; base += 16) {
			const int jj = base + w * 4 + sub;
			const int j = k0 + (jj < n ? jj : 0);
			const float *kr = a.kc + (size_t)(j == cur ? k0 : j) * HD;
			float4 kv[4];
#pragma unroll
			for (int i = 0; i < 4; i++) kv[i] = *reinterpret_cast<const float4 *>(kr + i * 64 + sl * 4);
			pass(base, kv);
		}
	}
	__syncthreads();

	// softmax statistics of this chunk: wave h owns head h
	{
		float m = -INFINITY;
		for (int j = lane; j < n; j += 64) m = fmaxf(m, sc[w][j]);
		m = wmax(m);
		float l = 0.0f;
		for (int j = lane; j < n; j += 64) {
			const float p = expf(sc[w][j] - m);
			sc[w][j] = p;
			l += p;
		}
		l = wsum(l);
		if (lane == 0) { s_m[w] = m; s_l[w] = l; }
	}
	__syncthreads();

	// P.V of the first PRE keys: wave w owns keys 8w..8w+7, lane = 4 consecutive dims; summed over the waves via LDS
	{
		float4 part[NH];
#pragma unroll
		for (int h = 0; h < NH; h++) part[h] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
		const int ub = (PRE / 4) * w;
		if (ub < n) {  // entries of sc past n are read with the group but not used
			float4 p[NH][2];
#pragma unroll
			for (int h = 0; h < NH; h++) {
				p[h][0] = *reinterpret_cast<const float4 *>(&sc[h][ub]);
				p[h][1] = *reinterpret_cast<const float4 *>(&sc[h][ub + 4]);
			}
			const float4 vn = *reinterpret_cast<const float4 *>(&vnew[4 * lane]);
#pragma unroll
			for (int u = 0; u < PRE / 4; u++) {
				if (ub + u < n) {
					const float4 vv = (k0 + ub + u == cur) ? vn : vpre[u];
#pragma unroll
					for (int h = 0; h < NH; h++) {
						const float ph = reinterpret_cast<const float *>(&p[h][u >> 2])[u & 3];
						part[h].x = fmaf(ph, vv.x, part[h].x);
						part[h].y = fmaf(ph, vv.y, part[h].y);
						part[h].z = fmaf(ph, vv.z, part[h].z);
						part[h].w = fmaf(ph, vv.w, part[h].w);
					}
				}
			}
		}
#pragma unroll
		for (int h = 0; h < NH; h++) *reinterpret_cast<float4 *>(&pv[w][h][4 * lane]) = part[h];
	}
	__syncthreads();
	// from here on: thread = output dim, 4 heads
	float acc[NH];
#pragma unroll
	for (int h = 0; h < NH; h++) acc[h] = (pv[0][h][tid] + pv[1][h][tid]) + (pv[2][h][tid] + pv[3][h][tid]);
	for (int j0 = PRE; j0 < n; j0 += 8) {
		float vv[8];
#pragma unroll
		for (int u = 0; u < 8; u++) {
			const int jj = j0 + u;
			const int j = k0 + (jj < n ? jj : 0);
			vv[u] = (j == cur) ? vnew[tid] : a.vc[(size_t)j * HD + tid];
		}
#pragma unroll
		for (int u = 0; u < 8; u++) {
			if (j0 + u < n) {
#pragma unroll
				for (int h = 0; h < NH; h++) acc[h] = fmaf(sc[h][j0 + u], vv[u], acc[h]);
			}
		}
	}

	// partial (max, sum, unnormalised output) of this chunk; merged by the consumer
#pragma unroll
	for (int h = 0; h < NH; h++) attn_store<WT>(&a.part_acc[((size_t)b * NH + h) * HD + tid], acc[h]);
	if (tid < NH) {
		attn_store<WT>(&a.part_ml[((size_t)b * NH + tid) * 2 + 0], s_m[tid]);
		attn_store<WT>(&a.part_ml[((size_t)b * NH + tid) * 2 + 1], s_l[tid]);
	}
}

}  // namespace tga

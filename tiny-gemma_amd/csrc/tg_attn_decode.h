// Device-side body of the decode attention (tg_attn.hip), shared with the one-kernel decode step
// (tg_decode_fused.hip) so that both paths do the same arithmetic in the same order and give the same bits.
#pragma once

#include "tg_internal.h"

namespace tga {

// e^x for softmax weights: v_exp_f32 on x * log2(e), two instructions instead of the dozen of expf.  For x in [-10, 0],
// where the weights that matter lie, the result is off by at most 3.3e-7 relative; e^-inf = 0.
__device__ __forceinline__ float attn_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }


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
	const float irms = __builtin_amdgcn_rsqf(ss * (1.0f / (float)HD) + 1e-06f);
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

typedef float af4 __attribute__((ext_vector_type(4)));

// WT: the partials are stored write-through at device scope (for a consumer inside the same kernel on another XCD)
template <bool WT>
__device__ __forceinline__ void attn_store(float *p, float v) {
	if (WT) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	else *p = v;
}

template <int CTRL>
__device__ __forceinline__ float attn_dpp(float v) { return __uint_as_float(tg_dpp_u32<CTRL>(__float_as_uint(v))); }

// 32 partial sums per lane, index 8 * head + key, are summed over the 64 lanes AND dealt out in the same pass: each
// step adds the partner lane's half of the values this lane keeps and hands the other half over, so the value count
// halves while the lane count doubles (70 instructions instead of 32 butterflies of 6).  Afterwards lane l holds the
// complete sum of head l / 16, key (l % 16) / 2 (two neighbouring lanes hold each sum).  Partner lanes: the other
// half-wave and the neighbouring row through the swap instructions; inside a row of 16 lanes l ^ 8 (rotation by 8),
// l ^ 7 (mirror of the 8-lane half), l ^ 3 (quad reversed), l ^ 1.
__device__ __forceinline__ float attn_transpose_reduce(float (&d)[32]) {
	const int lane = (int)__lane_id();
#pragma unroll
	for (int v = 0; v < 16; v++) {  // lanes 32..63 keep heads 2, 3
		const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(d[v]), __float_as_uint(d[v + 16]), false, false);
		d[v] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
	}
#pragma unroll
	for (int v = 0; v < 8; v++) {   // odd rows keep heads 1, 3
		const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(d[v]), __float_as_uint(d[v + 8]), false, false);
		d[v] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
	}
	const bool b3 = (lane & 8) != 0, b2 = (lane & 4) != 0, b1 = (lane & 2) != 0;
#pragma unroll
	for (int v = 0; v < 4; v++) {   // lanes with bit 3 keep keys 4..7
		const float keep = b3 ? d[v + 4] : d[v], send = b3 ? d[v] : d[v + 4];
		d[v] = keep + attn_dpp<0x128>(send);  // row_ror:8
	}
#pragma unroll
	for (int v = 0; v < 2; v++) {   // lanes with bit 2 keep keys 2, 3 (6, 7)
		const float keep = b2 ? d[v + 2] : d[v], send = b2 ? d[v] : d[v + 2];
		d[v] = keep + attn_dpp<0x141>(send);  // row_half_mirror
	}
	const float keep = b1 ? d[1] : d[0], send = b1 ? d[0] : d[1];
	const float s = keep + attn_dpp<0x1B>(send);  // quad_perm:[3,2,1,0]
	return s + attn_dpp<0xB1>(s);                 // quad_perm:[1,0,3,2]
}

// RMSNorm + half-rotation RoPE of one 256-wide head vector spread over a wave, lane l owning dims 4l .. 4l+3
// (ops.hpp:126-180, decode.hpp:136-211); the rotation partner of dim d, d +- 128, sits in lane l ^ 32.
// cs4 / sn4: the table entries of dims (4l .. 4l+3) % 128.
__device__ __forceinline__ af4 attn_head_finish(af4 x, af4 w, af4 cs4, af4 sn4, float mul) {
	float ss = 0.0f;
#pragma unroll
	for (int e = 0; e < 4; e++) ss = fmaf(x[e], x[e], ss);
	ss = wsum(ss);
	const float irms = __builtin_amdgcn_rsqf(ss * (1.0f / (float)HD) + 1e-06f);
	const bool upper = (__lane_id() & 32) != 0;
	af4 out;
#pragma unroll
	for (int e = 0; e < 4; e++) {
		const float xn = (x[e] * irms) * (w[e] + 1.0f);
		const float xp = tg_red_partner<32>(xn);
		out[e] = fmaf(cs4[e], xn, (upper ? xp : -xp) * sn4[e]) * mul;
	}
	return out;
}

// Keys per wave and pass: a wave walks the blocks w, w + 4, ... of 8 keys of the workgroup's chunk.  The first block of
// every wave (32 keys per workgroup) is requested before anything else in the kernel.
constexpr int KB = 8;

// One workgroup's chunk b of the keys: q/k norm + RoPE, cache write (chunk 0), and an exact softmax partial (maximum, sum,
// unnormalised output) of the chunk for the four heads.  Every wave does the whole chain for its own keys and all four
// heads without talking to the others - scores (the K rows are read once per workgroup), softmax over its keys, P.V -
// and the four per-wave partials meet in LDS at the end: two workgroup barriers in all (the q heads, the partials).
// after_loads() is called once the body has issued its up-front loads.
template <bool WT, class F>
__device__ __forceinline__ void attn_decode_body(const TgAttnDecode &a, int b, F after_loads) {
	__shared__ __attribute__((aligned(16))) float pacc[ANT / 64][NH][HD];  // per-wave unnormalised outputs
	__shared__ float pm[ANT / 64][NH], pl[ANT / 64][NH];
	__shared__ __attribute__((aligned(16))) float qs[NH][HD];  // normalised, rotated, scaled q heads

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	const int pos = a.host_pos >= 0 ? a.host_pos : a.pos[0];          // position_ptr before this token (decode.hpp:154)

	// Everything is requested up front.  The few values the q/k path needs go first (the previous launch's
	// q|k|v vector, norm weights, RoPE row): a wait for them must not include the cache rows behind them.  Their
	// addresses come from the launch arguments that the dispatcher preloads into scalar registers, so they go out
	// before anything has to be fetched from the argument block.
	const float *cs = a.cos_t + (size_t)pos * (HD / 2), *sn = a.sin_t + (size_t)pos * (HD / 2);
	const af4 xw = *reinterpret_cast<const af4 *>(a.qkv + w * HD + 4 * lane);  // q head w
	const af4 xk = *reinterpret_cast<const af4 *>(a.qkv + NH * HD + 4 * lane);
	const af4 vnew = *reinterpret_cast<const af4 *>(a.qkv + NH * HD + HD + 4 * lane);
	const af4 wq = *reinterpret_cast<const af4 *>(a.rms_q + 4 * lane), wk = *reinterpret_cast<const af4 *>(a.rms_k + 4 * lane);
	const af4 cs4 = *reinterpret_cast<const af4 *>(cs + 4 * (lane & 31)), sn4 = *reinterpret_cast<const af4 *>(sn + 4 * (lane & 31));
	// The rest of the descriptor is fetched now, in one batch, behind the loads above (a scalar fetch per use, each under
	// its own branch, was three dependent round trips in front of the first vector load).
	asm volatile("" ::"s"(a.max_pos), "s"(a.kc), "s"(a.vc), "s"(a.part_acc), "s"(a.part_ml) : "memory");
	const int bp = a.host_bp >= 0 ? a.host_bp : a.pos[a.bp_index];    // buffer_ptr before this token (decode.hpp:59)
	// with the position known on the host the ring slot and the number of workgroups come with the launch (two integer
	// divisions of 25 instructions each in front of the cache rows' addresses otherwise)
	const int cur = a.host_cur >= 0 ? a.host_cur : bp % a.max_pos;
	const int valid = (pos + 1 < a.max_pos) ? pos + 1 : a.max_pos;  // decode.hpp:45-47 after update_single
	const int nb = a.host_cur >= 0 ? a.nblocks : (valid + a.chunk - 1) / a.chunk;
	if (b >= nb) return;
	const int k0 = b * a.chunk;
	const int n = (valid - k0 < a.chunk) ? valid - k0 : a.chunk;
	const int nblk = (n + KB - 1) / KB;
	// Cache rows of the wave's first block: they depend on nothing computed here.  Rows are addressed as base + constant
	// * row; rows past the chunk (and slot `cur`, which workgroup 0 rewrites below) are fetched and ignored: every row
	// index is clamped into the cache, whose max_pos rows are all allocated.
	const int lim = a.max_pos - 1 - k0;  // >= 0: last row of the cache, relative to the chunk
	const float *kbase = a.kc + (size_t)k0 * HD + 4 * lane, *vbase = a.vc + (size_t)k0 * HD + 4 * lane;
	af4 kr[KB], vr[KB];
	auto load_block = [&](int t) {
#pragma unroll
		for (int jj = 0; jj < KB; jj++) {
			int r = KB * t + jj;
			r = r < lim ? r : lim;
			kr[jj] = *reinterpret_cast<const af4 *>(kbase + (size_t)r * HD);
		}
#pragma unroll
		for (int jj = 0; jj < KB; jj++) {
			int r = KB * t + jj;
			r = r < lim ? r : lim;
			vr[jj] = *reinterpret_cast<const af4 *>(vbase + (size_t)r * HD);
		}
	};
	load_block(w);
	after_loads();  // the caller's own loads go out behind this body's: a wait for a load covers every load issued before it
	__builtin_amdgcn_sched_barrier(0);  // the requests stay in front of the arithmetic below

	// q heads and the new key.  Wave w normalises and rotates q head w; the new key, which every wave needs, is done by
	// every wave for itself (two independent chains that overlap); the q heads are handed round through LDS.  (Every
	// wave doing all five vectors saved the barrier but took 0.86 us: the chains are 100 instructions each.)
	*reinterpret_cast<af4 *>(&qs[w][4 * lane]) = attn_head_finish(xw, wq, cs4, sn4, 0.0625f);  // ops.hpp:257: q *= 1/sqrt(256)
	const af4 knew = attn_head_finish(xk, wk, cs4, sn4, 1.0f);
	__syncthreads();
	af4 q[NH];
#pragma unroll
	for (int h = 0; h < NH; h++) q[h] = *reinterpret_cast<const af4 *>(&qs[h][4 * lane]);
	if (b == 0 && w == 0) {  // KVCache::update_single, decode.hpp:49-70
		if (WT) {
#pragma unroll
			for (int c = 0; c < 4; c++) {
				attn_store<true>(a.kc + (size_t)cur * HD + 4 * lane + c, knew[c]);
				attn_store<true>(a.vc + (size_t)cur * HD + 4 * lane + c, vnew[c]);
			}
		} else {
			*reinterpret_cast<af4 *>(a.kc + (size_t)cur * HD + 4 * lane) = knew;
			*reinterpret_cast<af4 *>(a.vc + (size_t)cur * HD + 4 * lane) = vnew;
		}
	}

	// the wave's blocks: scores, online softmax, P.V; m_run / l_run are those of the head of this lane's row
	float m_run = -INFINITY, l_run = 0.0f;
	af4 acc[NH];
#pragma unroll
	for (int h = 0; h < NH; h++) acc[h] = af4{0.0f, 0.0f, 0.0f, 0.0f};
	const int jl = (lane & 15) >> 1;  // the key (within a block) whose score this lane ends up with
	for (int t = w; t < nblk; t += ANT / 64) {
		if (t != w) load_block(t);
		float d[32];
#pragma unroll
		for (int jj = 0; jj < KB; jj++) {
			const af4 kv = (k0 + KB * t + jj == cur) ? knew : kr[jj];  // the token being decoded comes from registers
#pragma unroll
			for (int h = 0; h < NH; h++) {
				float x = q[h][0] * kv[0];
				x = fmaf(q[h][1], kv[1], x);
				x = fmaf(q[h][2], kv[2], x);
				x = fmaf(q[h][3], kv[3], x);
				d[h * KB + jj] = x;
			}
		}
		float s = attn_transpose_reduce(d);
		const bool ok = KB * t + jl < n;
		s = ok ? s : -INFINITY;
		const float m_new = fmaxf(m_run, tg_row16_max(s));  // finite: the first key of a block is always valid
		const float p = ok ? attn_exp(s - m_new) : 0.0f;
		const float scale = attn_exp(m_run - m_new);        // 0 for the first block
		l_run = fmaf(l_run, scale, 0.5f * tg_row16_sum(p));  // every sum sits in two lanes
		m_run = m_new;
#pragma unroll
		for (int h = 0; h < NH; h++) {
			const float sh = __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)__float_as_uint(scale), 16 * h));
#pragma unroll
			for (int e = 0; e < 4; e++) acc[h][e] *= sh;
		}
#pragma unroll
		for (int jj = 0; jj < KB; jj++) {
			const af4 vv = (k0 + KB * t + jj == cur) ? vnew : vr[jj];
#pragma unroll
			for (int h = 0; h < NH; h++) {
				const float ph = __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)__float_as_uint(p), 16 * h + 2 * jj));
#pragma unroll
				for (int e = 0; e < 4; e++) acc[h][e] = fmaf(ph, vv[e], acc[h][e]);
			}
		}
	}
#pragma unroll
	for (int h = 0; h < NH; h++) *reinterpret_cast<af4 *>(&pacc[w][h][4 * lane]) = acc[h];
	if ((lane & 15) == 0) {
		pm[w][lane >> 4] = m_run;
		pl[w][lane >> 4] = l_run;
	}
	__syncthreads();

	// the four per-wave partials of head w -> the chunk's partial (max, sum, unnormalised output); merged by the consumer
	{
		float mw[ANT / 64], M = -INFINITY;
#pragma unroll
		for (int i = 0; i < ANT / 64; i++) {
			mw[i] = pm[i][w];
			M = fmaxf(M, mw[i]);
		}
		af4 o = af4{0.0f, 0.0f, 0.0f, 0.0f};
		float l = 0.0f;
#pragma unroll
		for (int i = 0; i < ANT / 64; i++) {
			const float e = attn_exp(mw[i] - M);  // a wave without keys: exp(-inf) = 0
			const af4 pa = *reinterpret_cast<const af4 *>(&pacc[i][w][4 * lane]);
#pragma unroll
			for (int c = 0; c < 4; c++) o[c] = fmaf(pa[c], e, o[c]);
			l = fmaf(pl[i][w], e, l);
		}
		float *dst = a.part_acc + ((size_t)b * NH + w) * HD + 4 * lane;
		if (WT) {
#pragma unroll
			for (int c = 0; c < 4; c++) attn_store<true>(dst + c, o[c]);
		} else {
			*reinterpret_cast<af4 *>(dst) = o;
		}
		if (lane == 0) {
			attn_store<WT>(&a.part_ml[((size_t)b * NH + w) * 2 + 0], M);
			attn_store<WT>(&a.part_ml[((size_t)b * NH + w) * 2 + 1], l);
		}
	}
}

}  // namespace tga

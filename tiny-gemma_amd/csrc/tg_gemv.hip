// Decode-side int8 weight-only GEMV for gfx950 (wave64).
//
// Replaces gemv::qgemv / gemv::qgemv_row_tile (csrc/include/linalg.hpp:41-174 of the reference):
//     y[c] = scales[c] * sum_r x[r] * float(W[r][c])
// with the scale applied once after the whole fp32 reduction (linalg.hpp:83-107).
//
// Work decomposition: one workgroup per tile of C output columns, over the WHOLE reduction
// length, so no partial sums ever leave the workgroup: no atomics, no device-scope fences (on
// this multi-XCD part a fence is an L2 write-back + invalidate, tens of microseconds when
// hundreds of workgroups issue one).  C is chosen per matrix (4 ... 128) so that every matrix,
// however narrow, yields a few hundred workgroups.  The tile is stored as one contiguous slab
// [K/4][C][4] (tg_internal.h): the 256 lanes read consecutive 16-byte pieces (4 columns x 4 rows),
// C/4 lanes across the columns and 1024/C lanes along K; each byte is converted with one
// sign-extending convert and fed to an fp32 FMA; lanes that share columns are combined with
// cross-lane shuffles and one small LDS exchange between the 4 waves, in a fixed order, so
// results are run-to-run deterministic.
//
// Prologues fold the work that precedes a projection in modules::attention / modules::mlp
// (modules.hpp:135-220) into the same launch: embedding gather, post-norm + residual add of the
// previous block, pre-norm, or the merge of the attention partials.  Epilogues fold what follows:
// LUT-GeLU(gate) * up, or logits write-out plus the per-workgroup stage of the greedy argmax.

#include "tg_internal.h"

namespace {

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

// DEPTH: 16-byte weight loads in flight per lane
template <int PRO, int EPI, int AUX, int DEPTH>
__device__ __forceinline__ void gemv_body(const TgGemv &g) {
	__shared__ __attribute__((aligned(16))) float xs[TG_MAX_HIDDEN];  // input vector (all prologues but PLAIN)
	__shared__ __attribute__((aligned(16))) float lut_s[(EPI == TG_EPI_GEGLU) ? LUT_LDS : 4];  // GeLU table of the GeGLU epilogue
	__shared__ __attribute__((aligned(16))) float red2[2][NWAVE][TG_CT];  // double buffered across the tile loop
	__shared__ float sred[NWAVE];
	__shared__ float wgt[4][TG_ATTN_MERGE_MAX];
	__shared__ float s_bv[2][NWAVE];
	__shared__ int s_bi[2][NWAVE];

	if ((int)blockIdx.x >= g.nmain) {  // extra workgroups: prefetch the next launch's weights and leave
		tg_prefetch_dispatch(g.pf, g.pf2, g.nmain);
		return;
	}
	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	int tile = blockIdx.x;
	const int C = g.C, LC = C >> 2, lcs = g.lc_shift;  // LC = 1 << lcs lanes across the tile's columns
	const int KL = NT >> lcs;                          // lanes along K
	const int kpos = tid >> lcs;
	const int kgs = g.K >> 2;
	const int nit = (kgs + KL - 1) / KL;  // steps; one step = the 256 lanes reading 4 KiB of the slab

	// The tile slab and (for the PLAIN prologue) the input vector are read through buffer
	// descriptors: the per-step address is a scalar offset, so addressing costs no vector
	// instructions, and pieces past the end of the slab (lanes beyond K in the last step) read as 0.
	const uint32_t slab = (uint32_t)g.K * (uint32_t)C;
	__amdgpu_buffer_rsrc_t rw = make_rsrc(g.W + (size_t)tile * slab, slab);
	const uint32_t xbytes = (PRO == TG_PRO_PLAIN) ? (uint32_t)g.K * 4u : 0u;
	const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.x, xbytes);
	const uint32_t voff = (uint32_t)tid * 16u, xoff = (uint32_t)kpos * 16u, xstep = (uint32_t)KL * 16u;

	// The first DEPTH steps of the weight stream do not depend on the prologue and are requested before
	// its arithmetic ends, but BEHIND the prologue's own (small) loads: a wait for a load also waits for
	// every load issued before it, and the prologue must not wait for the weights to see its inputs.
	i32x4 v[DEPTH];
	f32x4 xq[DEPTH];
	// Column scales of a tile (and, for the GeGLU epilogue, the GeLU table) are requested together with its first
	// weights: fetched in the epilogue they would add one, for the table two, memory round trips at the end.
	float sc_a = 0.0f, sc_b = 0.0f;  // thread tid < C: scale of column tid (GeGLU: up column tid and gate column tid)
	auto load_scales = [&](int t) {
		const int ncol = (EPI == TG_EPI_GEGLU) ? (C >> 1) : C;
		const int c = tid < ncol ? tid : 0;
		sc_a = g.scales[t * C + c];
		if (EPI == TG_EPI_GEGLU) sc_b = g.scales[t * C + (C >> 1) + c];
	};
	f32x4 lutv = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
	const bool lut_in_lds = (EPI == TG_EPI_GEGLU) && g.lut_size <= LUT_LDS && (g.lut_size & 3) == 0;
	auto issue_weights = [&]() {
		load_scales(tile);
		if (lut_in_lds) lutv = *reinterpret_cast<const f32x4 *>(g.lut + (4 * tid < g.lut_size ? 4 * tid : 0));
#pragma unroll
		for (int u = 0; u < DEPTH; u++) {
			xq[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
			v[u] = ldw<AUX>(rw, voff, min((uint32_t)u * STEP_BYTES, slab));  // past the end of the slab: reads as 0
			if (PRO == TG_PRO_PLAIN) xq[u] = ldx(rx, xoff, min((uint32_t)u * xstep, xbytes));
		}
	};
	if (PRO == TG_PRO_PLAIN) issue_weights();

	// ---------------- prologue: input vector ----------------
	// Every global load of a prologue that does not depend on another one is issued up front, next
	// to the weight loads above, so that the prologue costs one memory round trip, not several.
	if (PRO == TG_PRO_ATTN_MERGE) {
		// merge of the flash-decoding partials of the attention launch that precedes this projection:
		//   out_h = sum_b acc_{b,h} * exp(m_{b,h} - M_h) / sum_b l_{b,h} * exp(m_{b,h} - M_h)
		const int pos = g.host_pos >= 0 ? g.host_pos : g.pos[0];
		const int valid = (pos + 1 < g.attn_max_pos) ? pos + 1 : g.attn_max_pos;
		const int nb = (valid + g.attn_chunk - 1) / g.attn_chunk;  // <= TG_ATTN_MERGE_MAX, checked on the host
		// wave w merges head w; a lane owns 4 consecutive dims: 16 loads of 16 bytes instead of 64 of 4
		f32x4 a[TG_ATTN_MERGE_MAX];
		float m = -INFINITY, l = 0.0f;
		if (tid < 4 * TG_ATTN_MERGE_MAX && (tid % TG_ATTN_MERGE_MAX) < nb) {
			const int h = tid / TG_ATTN_MERGE_MAX, b = tid % TG_ATTN_MERGE_MAX;
			m = g.part_ml[((size_t)b * 4 + h) * 2];
			l = g.part_ml[((size_t)b * 4 + h) * 2 + 1];
		}
#pragma unroll
		for (int b = 0; b < TG_ATTN_MERGE_MAX; b++) {
			// unconditional load from a clamped index, select afterwards: a load under a branch is waited for
			// at the end of that branch, which would turn these loads into as many round trips
			const int bb = b < nb ? b : 0;
			const f32x4 val = *reinterpret_cast<const f32x4 *>(g.part_acc + ((size_t)bb * 4 + w) * 256 + 4 * lane);
			a[b] = (b < nb) ? val : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
		}
		issue_weights();
		if (tid < 4 * TG_ATTN_MERGE_MAX) {
			const int h = tid / TG_ATTN_MERGE_MAX, b = tid % TG_ATTN_MERGE_MAX;
			const bool ok = b < nb;
			static_assert(TG_ATTN_MERGE_MAX == 16, "one row of 16 lanes per head");
			const float M = tg_row16_max(m);
			const float e = ok ? expf(m - M) : 0.0f;
			// __fmul_rn: the product must be rounded before the reduction; contracted into the first add
			// (fma(l, e, partner)) the two lanes of a pair would no longer hold the same sum
			const float L = tg_row16_sum(__fmul_rn(l, e));
			wgt[h][b] = e / L;
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
	} else if (PRO != TG_PRO_PLAIN) {
		const int h = g.hidden;
		const float eps = 1e-06f;
		constexpr int PER = (TG_MAX_HIDDEN + NT - 1) / NT;  // elements of the residual stream per lane
		float t[PER], wpre[PER];
#pragma unroll
		for (int i = 0; i < PER; i++) {
			const int d = tid + i * NT;
			const float val = g.w_pre[d < h ? d : h - 1];  // clamped index + select: no branch, no wait per load
			wpre[i] = (d < h) ? val : 0.0f;
		}
		if (PRO == TG_PRO_EMBED) {
			// ops.hpp:537-568: s[d] * (sqrt(hidden) * q)
			int tok;
			if (g.am_val != nullptr) {  // the previous step's pick is finished here, by every workgroup for itself
				tok = argmax_pairs(g.am_val, g.am_idx, g.am_n, s_bv[0], s_bi[0]);
				if (blockIdx.x == 0 && tid == 0) record_pick(tok, g.am_ctr, g.am_log, 1);
			} else {
				tok = *g.tok;
			}
			tok = tok < 0 ? 0 : (tok >= g.vocab ? g.vocab - 1 : tok);
			const int8_t *row = g.wte + (size_t)tok * h;
#pragma unroll
			for (int i = 0; i < PER; i++) {
				const int d = tid + i * NT;
				const int dd = d < h ? d : h - 1;
				const float val = g.wte_scales[dd] * (g.emb_scale * (float)row[dd]);
				t[i] = (d < h) ? val : 0.0f;
			}
			issue_weights();
		} else if (PRO == TG_PRO_NORM) {
#pragma unroll
			for (int i = 0; i < PER; i++) {
				const int d = tid + i * NT;
				const float val = g.x[d < h ? d : h - 1];
				t[i] = (d < h) ? val : 0.0f;
			}
			issue_weights();
		} else {
			// modules.hpp:166-168 / 218-219: x = rmsnorm(block_out, post) + residual
			float p[PER], r[PER], wpo[PER];
#pragma unroll
			for (int i = 0; i < PER; i++) {
				const int d = tid + i * NT;
				const bool ok = d < h;
				const int dd = ok ? d : h - 1;
				const float pv = g.pend[dd], rv = g.x[dd], wv = g.w_post[dd];
				p[i] = ok ? pv : 0.0f;
				r[i] = ok ? rv : 0.0f;
				wpo[i] = ok ? wv : 0.0f;
			}
			// The weight stream of a per-layer projection starts once the prologue's inputs are here (the empty asm
			// keeps the scheduler from hoisting it): requested together with them it made a decode step 0.7 % slower.
			// The LM head, which is bound by its stream, requests it at once.
			constexpr bool late = (AUX == TG_W_DEFAULT);
			if (!late) issue_weights();
			float ss = 0.0f;
#pragma unroll
			for (int i = 0; i < PER; i++) ss = fmaf(p[i], p[i], ss);
			if (late) {
				asm volatile("" : "+v"(ss) : : "memory");
				issue_weights();
			}
			ss = block_sum(ss, sred);
			const float irms = 1.0f / sqrtf(ss / (float)h + eps);
#pragma unroll
			for (int i = 0; i < PER; i++) t[i] = (p[i] * irms) * (wpo[i] + 1.0f) + r[i];
		}
		if (g.xr_out != nullptr && blockIdx.x == 0) {
#pragma unroll
			for (int i = 0; i < PER; i++) {
				const int d = tid + i * NT;
				if (d < h) g.xr_out[d] = t[i];
			}
		}
		// ops.hpp:126-180: x * rsqrt(mean(x^2) + eps) * (1 + w)
		float ss = 0.0f;
#pragma unroll
		for (int i = 0; i < PER; i++) ss = fmaf(t[i], t[i], ss);  // lanes past h hold 0
		ss = block_sum(ss, sred);
		const float irms = 1.0f / sqrtf(ss / (float)h + eps);
#pragma unroll
		for (int i = 0; i < PER; i++) {
			const int d = tid + i * NT;
			if (d < h) xs[d] = (t[i] * irms) * (wpre[i] + 1.0f);
		}
		__syncthreads();
	}

	if (lut_in_lds && 4 * tid < g.lut_size) *reinterpret_cast<f32x4 *>(&lut_s[4 * tid]) = lutv;  // visible after the barrier that precedes the epilogue
	// A workgroup walks tiles blockIdx.x, blockIdx.x + nmain, ...: the prologue above is paid once.
	const int xlast = g.K - 4;
	for (int it = 0;; it++) {
	float(*red)[TG_CT] = red2[it & 1];
	// ---------------- main loop: rotating pipeline of DEPTH loads per lane ----------------
	float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
	auto xval = [&](int u, int step) -> f32x4 {
		if (PRO == TG_PRO_PLAIN) return xq[u];
		int idx = 4 * (kpos + step * KL);
		idx = idx < xlast ? idx : xlast;  // lanes past K: their weights read as 0, any finite x will do
		return *reinterpret_cast<const f32x4 *>(&xs[idx]);
	};
	// One short loop body, executed nit/DEPTH (rounded up) times: a launch of a per-layer projection runs its code
	// once, from a cold instruction cache, so the bytes of code on its path cost more than the loads they would
	// save.  Loads are unconditional: pieces past the end of the slab read as 0 without a memory access (buffer
	// range check) and add nothing to the sums.
	for (int st = 0; st < nit; st += DEPTH) {
#pragma unroll
		for (int u = 0; u < DEPTH; u++) {
			fma16(acc, v[u], xval(u, st + u));
			// the scalar offset never passes the end of the buffer: the range check then sees 0 records left
			const uint32_t nxt = (uint32_t)(st + DEPTH + u);
			v[u] = ldw<AUX>(rw, voff, min(nxt * STEP_BYTES, slab));
			if (PRO == TG_PRO_PLAIN) xq[u] = ldx(rx, xoff, min(nxt * xstep, xbytes));
		}
	}

	// the next tile's first loads go out before this tile's reduction and epilogue
	const int cur = tile;
	tile += g.nmain;
	const bool more = tile < g.ntiles;
	const float sc_cur_a = sc_a, sc_cur_b = sc_b;
	if (more) {
		load_scales(tile);
		rw = make_rsrc(g.W + (size_t)tile * slab, slab);
#pragma unroll
		for (int u = 0; u < DEPTH; u++) {
			v[u] = ldw<AUX>(rw, voff, min((uint32_t)u * STEP_BYTES, slab));
			if (PRO == TG_PRO_PLAIN) xq[u] = ldx(rx, xoff, min((uint32_t)u * xstep, xbytes));
		}
	}

	// ---------------- reduction over the lanes along K (fixed order) ----------------
	// lanes l and l' hold partial sums of the same columns iff l % LC == l' % LC
#define TG_STEP(O)                                                   \
	if (LC <= O) {                                                   \
		_Pragma("unroll") for (int j = 0; j < 4; j++) acc[j] += tg_red_partner<O>(acc[j]); \
	}
	TG_STEP(32) TG_STEP(16) TG_STEP(8) TG_STEP(4) TG_STEP(2) TG_STEP(1)
#undef TG_STEP
	if (lane < LC) *reinterpret_cast<float4 *>(&red[w][lane * 4]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
	__syncthreads();

	// ---------------- epilogue of tile `cur` ----------------
	if (EPI == TG_EPI_STORE) {
		if (tid < C) {
			const int col = cur * C + tid;
			const float sum = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
			g.y[col] = sum * sc_cur_a;
		}
	} else if (EPI == TG_EPI_GEGLU) {
		// modules.hpp:211-215: gelu(gate) * up; the tile holds C/2 up columns, then the same C/2 gate columns
		const int C2 = C >> 1;
		if (tid < C2) {
			const float su = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
			const float sg = (red[0][tid + C2] + red[1][tid + C2]) + (red[2][tid + C2] + red[3][tid + C2]);
			const float up = su * sc_cur_a;
			const float gate = sg * sc_cur_b;
			g.y[cur * C2 + tid] = gelu_lut(gate, lut_in_lds ? lut_s : g.lut, g.gmin, g.geps, g.lut_size) * up;
		}
	} else {
		// TG_EPI_LOGITS: logits + first stage of the greedy argmax
		// (ops.hpp:749-757: strict '>' scan from index 0, so the lowest index wins ties)
		float bv = -INFINITY;
		int bi = 0x7fffffff;
		if (tid < C) {
			const int col = cur * C + tid;
			const float sum = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
			const float val = sum * sc_cur_a;
			if (g.y != nullptr) g.y[col] = val;
			if (val > bv) { bv = val; bi = col; }
		}
#define TG_STEP(O)                                                                  \
	{                                                                               \
		const float ov = tg_red_partner<O>(bv);                                     \
		const int oi = tg_red_partner<O>(bi);                                       \
		if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }                 \
	}
		TG_STEP(32) TG_STEP(16) TG_STEP(8) TG_STEP(4) TG_STEP(2) TG_STEP(1)
#undef TG_STEP
		if (lane == 0) { s_bv[it & 1][w] = bv; s_bi[it & 1][w] = bi; }
		__syncthreads();
		if (tid == 0) {
			for (int i = 1; i < NWAVE; i++)
				if (s_bv[it & 1][i] > bv || (s_bv[it & 1][i] == bv && s_bi[it & 1][i] < bi)) { bv = s_bv[it & 1][i]; bi = s_bi[it & 1][i]; }
			g.blk_val[cur] = bv;
			g.blk_idx[cur] = bi;
		}
	}
	if (!more) break;
	}  // tile loop
}

// One named entry point per role, so that profiles separate the projections.
// The pointers a kernel dereferences first are passed once more in front of the descriptor: leading scalar
// arguments are preloaded into scalar registers by the dispatcher (kernarg preload, enabled with
// -mllvm -amdgpu-kernarg-preload-count), so the first vector loads of a launch do not have to wait for an
// s_load of the argument block (0.35 us on the critical path of every launch).
template <int PRO>
__device__ __forceinline__ TgGemv with_hot_args(const TgGemv &g_in, const void *a0, const void *a1, const void *a2, const void *a3,
                                                const int8_t *W, int hidden, int K) {
	TgGemv g = g_in;
	g.W = W;
	g.hidden = hidden;
	g.K = K;
	if (PRO == TG_PRO_RESNORM || PRO == TG_PRO_NORM) {
		g.pend = (const float *)a0;
		g.x = (const float *)a1;
		g.w_post = (const float *)a2;
		g.w_pre = (const float *)a3;
	} else if (PRO == TG_PRO_ATTN_MERGE) {
		g.part_acc = (const float *)a0;
		g.part_ml = (const float *)a1;
	} else if (PRO == TG_PRO_EMBED) {
		g.wte = (const int8_t *)a0;
		g.wte_scales = (const float *)a1;
		g.tok = (const int *)a2;
		g.w_pre = (const float *)a3;
	} else {
		g.x = (const float *)a1;
	}
	return g;
}
// The per-layer roles are templates over DEPTH (the launcher picks it from the number of steps); the LM head has
// one depth.
#define TG_GEMV_ARGS const void *a0, const void *a1, const void *a2, const void *a3, const int8_t *W, int hidden, int K, const TgGemv g
#define TG_GEMV_KERNEL_T(NAME, PRO, EPI, AUX)                                                         \
	template <int DEPTH>                                                                              \
	__global__ __launch_bounds__(NT) void NAME(TG_GEMV_ARGS) {                                        \
		gemv_body<PRO, EPI, AUX, DEPTH>(with_hot_args<PRO>(g, a0, a1, a2, a3, W, hidden, K));         \
	}
#define TG_GEMV_KERNEL(NAME, PRO, EPI, AUX, DEPTH)                                                    \
	__global__ __launch_bounds__(NT) void NAME(TG_GEMV_ARGS) {                                        \
		gemv_body<PRO, EPI, AUX, DEPTH>(with_hot_args<PRO>(g, a0, a1, a2, a3, W, hidden, K));         \
	}
TG_GEMV_KERNEL_T(tg_gemv_qkv_embed, TG_PRO_EMBED, TG_EPI_STORE, TG_W_DEFAULT)        // layer 0: embedding + pre-norm + Q|K|V
TG_GEMV_KERNEL_T(tg_gemv_qkv, TG_PRO_RESNORM, TG_EPI_STORE, TG_W_DEFAULT)            // post-norm + residual + pre-norm + Q|K|V
TG_GEMV_KERNEL_T(tg_gemv_oproj, TG_PRO_ATTN_MERGE, TG_EPI_STORE, TG_W_DEFAULT)       // attention merge + output projection
TG_GEMV_KERNEL_T(tg_gemv_upgate_geglu, TG_PRO_RESNORM, TG_EPI_GEGLU, TG_W_DEFAULT)   // post-norm + residual + pre-norm + up|gate + gelu*up
TG_GEMV_KERNEL_T(tg_gemv_down, TG_PRO_PLAIN, TG_EPI_STORE, TG_W_DEFAULT)             // down projection
TG_GEMV_KERNEL_T(tg_gemv_plain, TG_PRO_PLAIN, TG_EPI_STORE, TG_W_DEFAULT)            // stand-alone y = s * (x . W)
TG_GEMV_KERNEL(tg_gemv_lmhead_argmax, TG_PRO_RESNORM, TG_EPI_LOGITS, TG_W_NT, TG_DEPTH_STREAM) // last post-norm + final norm + LM head + argmax stage 1
TG_GEMV_KERNEL(tg_gemv_lmhead_plain, TG_PRO_PLAIN, TG_EPI_LOGITS, TG_W_NT, TG_DEPTH_STREAM)    // LM head on an already normalised vector (prefill)
TG_GEMV_KERNEL(tg_gemv_plain_stream, TG_PRO_PLAIN, TG_EPI_STORE, TG_W_NT, TG_DEPTH_STREAM)     // stand-alone, for a matrix too large to stay cached

// Second stage of the greedy argmax and the per-token bookkeeping as a launch of their own: after a prefill, at the
// end of a batch of decode steps, and wherever the next launch is not the first projection of a decode step (which
// otherwise does both itself).
__global__ __launch_bounds__(NT) void tg_argmax_finish(const float *blk_val, const int *blk_idx, int n, int *ctr, int *tok_log,
                                                       int advance) {
	__shared__ float s_bv[NWAVE];
	__shared__ int s_bi[NWAVE];
	const int bi = argmax_pairs(blk_val, blk_idx, n, s_bv, s_bi);
	if (threadIdx.x == 0) record_pick(bi, ctr, tok_log, advance);
}

}  // namespace

// Loads in flight per lane for a launch whose loop covers `nit` steps of 4 KiB per workgroup.  A round of the loop
// costs a memory round trip plus DEPTH steps of arithmetic (the surplus steps of the last round multiply zeros).
// Measured on whole decode steps: 1 or 2 steps want 2, 7 steps 4 (2 and 8 are 1.2 % and 1.4 % of a step slower),
// 9 steps 3; the rule below (a round trip worth 5.5 steps of arithmetic, depth at most 4) reproduces that.  Columns
// of more than 32 steps are a stream and get 8.
int tg_gemv_depth(int K, int C) {
	const int kl = NT / (C >> 2), nit = ((K >> 2) + kl - 1) / kl;
	if (nit <= 2) return 2;
	if (nit > 32) return 8;
	int best = 2;
	float best_cost = 1e30f;
	for (int d : {2, 3, 4}) {
		const int rounds = (nit + d - 1) / d;
		const float cost = (float)rounds * (5.5f + (float)d);
		if (cost < best_cost) { best_cost = cost; best = d; }
	}
	return best;
}

void tg_launch_gemv(const TgGemv &g_in, int role, hipStream_t s) {
	// more than max_blocks tiles: workgroups loop over tiles, so the prologue is paid once per workgroup
	TgGemv g = g_in;
	g.nmain = (g.max_blocks > 0 && g.ntiles > g.max_blocks) ? g.max_blocks : g.ntiles;
	if (g.pf.ptr == nullptr) g.pf.nblocks = 0;
	if (g.pf2.ptr == nullptr) g.pf2.nblocks = 0;
	dim3 grid((unsigned)(g.nmain + g.pf.nblocks + g.pf2.nblocks)), block(NT);
	// hot arguments in the order with_hot_args expects for the role's prologue
	const void *a0 = g.pend, *a1 = g.x, *a2 = g.w_post, *a3 = g.w_pre;
	if (role == TG_ROLE_OPROJ) { a0 = g.part_acc; a1 = g.part_ml; a2 = a3 = nullptr; }
	if (role == TG_ROLE_QKV_EMBED) { a0 = g.wte; a1 = g.wte_scales; a2 = g.tok; a3 = g.w_pre; }
#define TG_LAUNCH(KERNEL) hipLaunchKernelGGL(KERNEL, grid, block, 0, s, a0, a1, a2, a3, g.W, g.hidden, g.K, g)
#define TG_LAUNCH_D(KERNEL)                          \
	switch (depth) {                                 \
		case 2: TG_LAUNCH(KERNEL<2>); break;         \
		case 3: TG_LAUNCH(KERNEL<3>); break;         \
		case 4: TG_LAUNCH(KERNEL<4>); break;         \
		default: TG_LAUNCH(KERNEL<8>); break;        \
	}
	const int depth = tg_gemv_depth(g.K, g.C);
	switch (role) {
		case TG_ROLE_QKV_EMBED: TG_LAUNCH_D(tg_gemv_qkv_embed); break;
		case TG_ROLE_QKV: TG_LAUNCH_D(tg_gemv_qkv); break;
		case TG_ROLE_OPROJ: TG_LAUNCH_D(tg_gemv_oproj); break;
		case TG_ROLE_UPGATE: TG_LAUNCH_D(tg_gemv_upgate_geglu); break;
		case TG_ROLE_DOWN: TG_LAUNCH_D(tg_gemv_down); break;
		case TG_ROLE_LMHEAD: TG_LAUNCH(tg_gemv_lmhead_argmax); break;
		case TG_ROLE_LMHEAD_PLAIN: TG_LAUNCH(tg_gemv_lmhead_plain); break;
		default:
			// a matrix of a quarter of the 256 MB memory-side cache or more is streamed as read-once data
			if ((size_t)g.K * g.C * g.ntiles >= ((size_t)64 << 20)) TG_LAUNCH(tg_gemv_plain_stream);
			else TG_LAUNCH_D(tg_gemv_plain);
			break;
	}
#undef TG_LAUNCH_D
#undef TG_LAUNCH
}

void tg_launch_argmax_finish(const float *blk_val, const int *blk_idx, int n, int *ctr, int *tok_log, int advance, hipStream_t s) {
	hipLaunchKernelGGL(tg_argmax_finish, dim3(1), dim3(NT), 0, s, blk_val, blk_idx, n, ctr, tok_log, advance);
}

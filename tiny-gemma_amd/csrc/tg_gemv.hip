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
#include "tg_gemv_parts.h"

using namespace tgp;

namespace {

// Where the descriptor sits in the argument block of every GEMV kernel: behind the leading arguments of TG_GEMV_ARGS
// (4 pointers, the weight pointer, 4 ints = 56 bytes, which is a multiple of the descriptor's alignment).
constexpr int TG_GEMV_DESC_OFFSET = 4 * 8 + 8 + 4 * 4;
static_assert(TG_GEMV_DESC_OFFSET % alignof(TgGemv) == 0, "the descriptor follows the leading arguments without padding");

// DEPTH: 16-byte weight loads in flight per lane
template <int PRO, int EPI, int AUX, int DEPTH>
__device__ __forceinline__ void gemv_body(const TgGemv &g_in) {
	TgGemv g = g_in;  // the fields fetch_rest() names are not known to the code before it (see there)
	__shared__ __attribute__((aligned(16))) float xs[TG_MAX_HIDDEN];  // input vector (all prologues but PLAIN)
	__shared__ __attribute__((aligned(16))) float lut_s[(EPI == TG_EPI_GEGLU) ? LUT_LDS : 4];  // GeLU table of the GeGLU epilogue
	__shared__ __attribute__((aligned(16))) float red2[2][NWAVE][TG_CT];  // double buffered across the tile loop
	__shared__ float sred[NWAVE], sred2[NWAVE];  // one per norm of a prologue: neither needs a barrier in front of it
	__shared__ float wgt[4][TG_ATTN_MERGE_MAX];
	__shared__ float s_bv[2][NWAVE];
	__shared__ int s_bi[2][NWAVE];

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	int tile = blockIdx.x;
	const int C = g.C, LC = C >> 2, lcs = g.lc_shift;  // LC = 1 << lcs lanes across the tile's columns
	const int KL = NT >> lcs;                          // lanes along K
	const int kpos = tid >> lcs;
	const int kgs = g.K >> 2;
	static_assert(NT == 256, "KL = 2^(8 - lcs)");
	const int nit = (kgs + KL - 1) >> (8 - lcs);  // steps (KL is a power of two: a shift, not a division in front of the first loads); one step = the 256 lanes reading 4 KiB of the slab

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
	auto lut_in_lds_f = [&]() { return (EPI == TG_EPI_GEGLU) && g.lut_size <= LUT_LDS && (g.lut_size & 3) == 0; };
	// Everything the first vector loads need (pointers, K, C, the number of computing workgroups) arrives in scalar
	// registers with the launch (leading arguments, preloaded by the dispatcher).  The rest of the descriptor is fetched
	// from the argument block in ONE batch, by fetch_rest(), which every prologue calls right behind its first vector
	// loads: fetched field by field at first use, each under its own branch, it was two dependent scalar round trips
	// (0.3 us each) in front of the first vector load of every launch.
	auto fetch_rest = [&]() {
		// The fields are read through the address of the argument block, which is made opaque here: the compiler can
		// neither start these fetches earlier (hoisted to the top of the kernel they end up with a wait in front of the
		// vector loads as soon as one of their registers is reused) nor use a field before this point.
		typedef const TgGemv __attribute__((address_space(4))) *KernargDesc;
		KernargDesc gp = (KernargDesc)((const char __attribute__((address_space(4))) *)__builtin_amdgcn_kernarg_segment_ptr() + TG_GEMV_DESC_OFFSET);
		asm volatile("" : "+s"(gp) : : "memory");
		g.scales = gp->scales;
		g.y = gp->y;
		g.xr_out = gp->xr_out;
		g.lut = gp->lut;
		g.lut_size = gp->lut_size;
		g.gmin = gp->gmin;
		g.geps = gp->geps;
		g.ntiles = gp->ntiles;
		g.blk_val = gp->blk_val;
		g.blk_idx = gp->blk_idx;
	};
	auto issue_weights = [&]() {
#pragma unroll
		for (int u = 0; u < DEPTH; u++) {
			xq[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
			v[u] = ldw<AUX>(rw, voff, min((uint32_t)u * STEP_BYTES, slab));  // past the end of the slab: reads as 0
			if (PRO == TG_PRO_PLAIN) xq[u] = ldx(rx, xoff, min((uint32_t)u * xstep, xbytes));
		}
		if (PRO == TG_PRO_PLAIN) fetch_rest();
		load_scales(tile);
		if (lut_in_lds_f()) lutv = *reinterpret_cast<const f32x4 *>(g.lut + (4 * tid < g.lut_size ? 4 * tid : 0));
	};
	if (PRO == TG_PRO_PLAIN) issue_weights();

	// ---------------- prologue: input vector ----------------
	// Every global load of a prologue that does not depend on another one is issued up front, next
	// to the weight loads above, so that the prologue costs one memory round trip, not several.
	if (PRO == TG_PRO_ATTN_MERGE) {
		// merge of the flash-decoding partials of the attention launch that precedes this projection
		int nb = g.merge_nb;  // <= TG_ATTN_MERGE_MAX, checked on the host
		if (nb < 0) {         // a captured step is replayed at other positions: the count follows the device-side counter
			const int pos = g.pos[0];
			const int valid = (pos + 1 < g.attn_max_pos) ? pos + 1 : g.attn_max_pos;
			nb = (valid + g.attn_chunk - 1) / g.attn_chunk;
		}
		attn_merge_prologue(xs, wgt, g.part_acc, g.part_ml, nb, [&] {
			fetch_rest();
			issue_weights();
		});
	} else if (PRO != TG_PRO_PLAIN) {
		const int h = g.hidden;
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
				const float val = embed_value(g.wte_scales[dd], g.emb_scale, row[dd]);
				t[i] = (d < h) ? val : 0.0f;
			}
			fetch_rest();
			issue_weights();
		} else if (PRO == TG_PRO_NORM) {
#pragma unroll
			for (int i = 0; i < PER; i++) {
				const int d = tid + i * NT;
				const float val = g.x[d < h ? d : h - 1];
				t[i] = (d < h) ? val : 0.0f;
			}
			fetch_rest();
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
			fetch_rest();
			// The weight stream of a per-layer projection starts once the prologue's inputs are here (the empty asm
			// keeps the scheduler from hoisting it): requested together with them it made a decode step 0.7 % slower.
			// The LM head, which is bound by its stream, requests it at once.
			constexpr bool late = (AUX == TG_W_DEFAULT);
			if (!late) issue_weights();
			float ss = sumsq(p);
			if (late) {
				asm volatile("" : "+v"(ss) : : "memory");
				issue_weights();
			}
			ss = block_sum_fresh(ss, sred);
			post_norm_add(t, p, rms_inv(ss, h), wpo, r);
		}
		if (g.xr_out != nullptr && blockIdx.x == 0) {
#pragma unroll
			for (int i = 0; i < PER; i++) {
				const int d = tid + i * NT;
				if (d < h) st_f32<true>(&g.xr_out[d], t[i]);
			}
		}
		// ops.hpp:126-180: x * rsqrt(mean(x^2) + eps) * (1 + w)
		const float ss = block_sum_fresh(sumsq(t), sred2);
		pre_norm_store(xs, t, rms_inv(ss, h), wpre, h);
		__syncthreads();
	}

	const bool lut_in_lds = lut_in_lds_f();
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
	lanes_reduce(acc, LC, red);
	__syncthreads();

	// ---------------- epilogue of tile `cur` ----------------
	if (EPI == TG_EPI_STORE) {
		epi_store<true>(red, C, cur, sc_cur_a, g.y);
	} else if (EPI == TG_EPI_GEGLU) {
		epi_geglu<true>(red, C, cur, sc_cur_a, sc_cur_b, g.y, lut_in_lds ? lut_s : g.lut, g.gmin, g.geps, g.lut_size);
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
			st_f32<true>(&g.blk_val[cur], bv);
			__hip_atomic_store(&g.blk_idx[cur], bi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
                                                const int8_t *W, int hidden, int K, int nmain, int aux) {
	TgGemv g = g_in;
	g.W = W;
	g.hidden = hidden;
	g.K = K;
	g.nmain = nmain;
	g.C = aux;  // tile width: what the addresses of the weight stream need first
	g.lc_shift = 29 - __builtin_clz((unsigned)aux);  // log2(C / 4)
	if (PRO == TG_PRO_RESNORM || PRO == TG_PRO_NORM) {
		g.pend = (const float *)a0;
		g.x = (const float *)a1;
		g.w_post = (const float *)a2;
		g.w_pre = (const float *)a3;
	} else if (PRO == TG_PRO_ATTN_MERGE) {
		g.part_acc = (const float *)a0;
		g.part_ml = (const float *)a1;
		g.merge_nb = hidden;  // partials to merge, or -1: from the device-side position
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
#define TG_GEMV_ARGS \
	const void *a0, const void *a1, const void *a2, const void *a3, const int8_t *W, int hidden, int K, int nmain, int aux, const TgGemv g
#define TG_GEMV_BODY(PRO, EPI, AUX, DEPTH)                                                            \
	if (__builtin_expect((int)blockIdx.x >= nmain, 0)) { /* extra workgroups: prefetch the next launch's weights and leave */ \
		tg_prefetch_dispatch(g.pf, g.pf2, nmain);                                                     \
		return;                                                                                       \
	}                                                                                                 \
	gemv_body<PRO, EPI, AUX, DEPTH>(with_hot_args<PRO>(g, a0, a1, a2, a3, W, hidden, K, nmain, aux));
#define TG_GEMV_KERNEL_T(NAME, PRO, EPI, AUX)                                                         \
	template <int DEPTH>                                                                              \
	__global__ __launch_bounds__(NT) void NAME(TG_GEMV_ARGS) {                                        \
		TG_GEMV_BODY(PRO, EPI, AUX, DEPTH)                                                            \
	}
#define TG_GEMV_KERNEL(NAME, PRO, EPI, AUX, DEPTH)                                                    \
	__global__ __launch_bounds__(NT) void NAME(TG_GEMV_ARGS) {                                        \
		TG_GEMV_BODY(PRO, EPI, AUX, DEPTH)                                                            \
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

void tg_desc_gemv(const TgGemv &g_in, int role, TgLaunchDesc *d) {
	// more than max_blocks tiles: workgroups loop over tiles, so the prologue is paid once per workgroup
	TgGemv &g = d->g;
	g = g_in;
	g.nmain = (g.max_blocks > 0 && g.ntiles > g.max_blocks) ? g.max_blocks : g.ntiles;
	if (g.pf.ptr == nullptr) g.pf.nblocks = 0;
	if (g.pf2.ptr == nullptr) g.pf2.nblocks = 0;
	d->grid = dim3((unsigned)(g.nmain + g.pf.nblocks + g.pf2.nblocks));
	d->block = dim3(NT);
	// hot arguments in the order with_hot_args expects for the role's prologue
	d->p[0] = g.pend;
	d->p[1] = g.x;
	d->p[2] = g.w_post;
	d->p[3] = g.w_pre;
	if (role == TG_ROLE_OPROJ) { d->p[0] = g.part_acc; d->p[1] = g.part_ml; d->p[2] = d->p[3] = nullptr; }
	if (role == TG_ROLE_QKV_EMBED) { d->p[0] = g.wte; d->p[1] = g.wte_scales; d->p[2] = g.tok; d->p[3] = g.w_pre; }
	d->p[4] = g.W;
	int hot_hidden = g.hidden;
	if (role == TG_ROLE_OPROJ) {  // the number of attention partials to merge rides in the slot of `hidden`
		hot_hidden = -1;
		if (g.host_pos >= 0) {
			const int valid = (g.host_pos + 1 < g.attn_max_pos) ? g.host_pos + 1 : g.attn_max_pos;
			hot_hidden = (valid + g.attn_chunk - 1) / g.attn_chunk;
		}
	}
	d->i[0] = hot_hidden;
	d->i[1] = g.K;
	d->i[2] = g.nmain;
	d->i[3] = g.C;
	// TG_GEMV_ARGS: a0, a1, a2, a3, W, hidden, K, nmain, aux, g
	for (int k = 0; k < 5; k++) d->args[k] = &d->p[k];
	for (int k = 0; k < 4; k++) d->args[5 + k] = &d->i[k];
	d->args[9] = &d->g;
#define TG_FUNC(KERNEL) d->func = reinterpret_cast<const void *>(&KERNEL)
#define TG_FUNC_D(KERNEL)                          \
	switch (depth) {                               \
		case 2: TG_FUNC(KERNEL<2>); break;         \
		case 3: TG_FUNC(KERNEL<3>); break;         \
		case 4: TG_FUNC(KERNEL<4>); break;         \
		default: TG_FUNC(KERNEL<8>); break;        \
	}
	const int depth = tg_gemv_depth(g.K, g.C);
	switch (role) {
		case TG_ROLE_QKV_EMBED: TG_FUNC_D(tg_gemv_qkv_embed); break;
		case TG_ROLE_QKV: TG_FUNC_D(tg_gemv_qkv); break;
		case TG_ROLE_OPROJ: TG_FUNC_D(tg_gemv_oproj); break;
		case TG_ROLE_UPGATE: TG_FUNC_D(tg_gemv_upgate_geglu); break;
		case TG_ROLE_DOWN: TG_FUNC_D(tg_gemv_down); break;
		case TG_ROLE_LMHEAD: TG_FUNC(tg_gemv_lmhead_argmax); break;
		case TG_ROLE_LMHEAD_PLAIN: TG_FUNC(tg_gemv_lmhead_plain); break;
		default:
			// a matrix of a quarter of the 256 MB memory-side cache or more is streamed as read-once data
			if ((size_t)g.K * g.C * g.ntiles >= ((size_t)64 << 20)) TG_FUNC(tg_gemv_plain_stream);
			else TG_FUNC_D(tg_gemv_plain);
			break;
	}
#undef TG_FUNC_D
#undef TG_FUNC
}

bool tg_gemv_is_oproj(const void *func) {
	return func == reinterpret_cast<const void *>(&tg_gemv_oproj<2>) || func == reinterpret_cast<const void *>(&tg_gemv_oproj<3>) ||
	       func == reinterpret_cast<const void *>(&tg_gemv_oproj<4>) || func == reinterpret_cast<const void *>(&tg_gemv_oproj<8>);
}

void tg_launch_gemv(const TgGemv &g, int role, hipStream_t s) {
	TgLaunchDesc d;
	tg_desc_gemv(g, role, &d);
	tg_launch_desc(d, s);
}

void tg_launch_argmax_finish(const float *blk_val, const int *blk_idx, int n, int *ctr, int *tok_log, int advance, hipStream_t s) {
	hipLaunchKernelGGL(tg_argmax_finish, dim3(1), dim3(NT), 0, s, blk_val, blk_idx, n, ctr, tok_log, advance);
}

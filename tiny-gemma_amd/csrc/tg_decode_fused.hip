// All layers of a decode step in one launch of resident workgroups (transformer.hpp:75-97 of the reference: the layer loop
// of forward_decode; modules.hpp:135-220: the five all-to-all dependency points of a layer).
//
// The launch path (tg_api.hip: enqueue_decode_step) turns every dependency point into a kernel boundary: 5 launches per
// layer, each of which costs 2.5 us before its first instruction and another 1.4 us until its inputs have arrived.  Here
// the workgroups stay resident for the whole step and hand over through device memory:
//
//   * `ng` GEMV workgroups own fixed column tiles of every projection (tiles g and g + ng of the same tiling the launch
//     path uses, so every column is summed in the same order and the results are bit-identical).  They keep the residual
//     stream in registers (every workgroup computes the norms redundantly, as the launch path does) and request the
//     weights of a projection into registers one phase ahead, so that the weight stream is not on the critical path.
//   * TG_FUSED_ATTN_WGS attention workgroups run the decode attention body of tg_attn_decode.h, one chunk of keys each.
//   * A producer stores its results write-through at device scope, waits for the acknowledgements, and arrives on a
//     counter; there is one counter line per XCD so that no line takes more than 32 arrivals.  A consumer polls the 8
//     counters with one load instruction (their sum tells how many have arrived) and then reads the data with ordinary
//     loads.  That is only correct because every region of the exchange buffer is written and read ONCE per launch: the
//     8 XCDs have separate, mutually incoherent L2s, a launch starts with clean caches, and a line that nobody has read
//     yet cannot be stale anywhere.
//   * Every wait is bounded: after max_spins polls a workgroup sets the error word, which every other poll also looks
//     at, and all workgroups leave.  The host then reports TG_ERR_STATE and goes back to the launch path.
//
// The LM head remains a launch of its own (tg_gemv.hip: tg_gemv_lmhead_argmax): it wants 2048 workgroups.

#include "tg_attn_decode.h"
#include "tg_gemv_parts.h"
#include "tg_internal.h"

using namespace tgp;

namespace {

constexpr int SL = 32;          // words per 128-byte line of the hand-over state
constexpr int SYNC_ALL = 0;     // lines 0..7: arrivals of the GEMV workgroups, by XCD
constexpr int SYNC_ATTN = 8;    // lines 8..15: arrivals of the attention workgroups, one copy per XCD
constexpr int SYNC_ERR = 16;    // line 16: set when a wait timed out

__device__ __forceinline__ int fused_xcc_id() {
	unsigned v;
	asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(v));
	return (int)(v & 7u);
}

// A producer's results are in memory (its write-through stores acknowledged) before its arrival is.
// kind 0: a GEMV workgroup adds to its XCD's counter; kind 1: an attention workgroup adds to all 8 copies.
__device__ __forceinline__ void fused_arrive(unsigned *sync, int kind, int xcd, bool counted) {
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
	__syncthreads();
	if (kind == 0) {
		if (threadIdx.x == 0) __hip_atomic_fetch_add(&sync[(SYNC_ALL + xcd) * SL], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	} else {
		if (counted && threadIdx.x < 8) __hip_atomic_fetch_add(&sync[(SYNC_ATTN + threadIdx.x) * SL], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
}

// Wave 0 polls, everybody leaves through the barrier.  kind 0: the sum of the 8 GEMV counters has reached `target`;
// kind 1: this XCD's copy of the attention counter has.  Returns false once any workgroup has given up.
__device__ __forceinline__ bool fused_wait(unsigned *sync, int kind, unsigned target, int xcd, int max_spins, int *s_dead) {
	if (threadIdx.x < 64) {
		const int lane = threadIdx.x;
		const unsigned *p = lane < 8 ? &sync[((kind ? SYNC_ATTN : SYNC_ALL) + lane) * SL] : &sync[SYNC_ERR * SL];
		int spins = 0;
		bool dead = false;
		for (;;) {
			unsigned v = 0;
			if (lane <= 8) v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			const unsigned err = (unsigned)__builtin_amdgcn_readlane((int)v, 8);
			unsigned have;
			if (kind == 0) {
				unsigned s = lane < 8 ? v : 0u;  // butterfly over the row of 16 lanes: every lane ends up with the sum
				s += tg_red_partner_u32<8>(s);
				s += tg_red_partner_u32<4>(s);
				s += tg_red_partner_u32<2>(s);
				s += tg_red_partner_u32<1>(s);
				have = (unsigned)__builtin_amdgcn_readlane((int)s, 0);
			} else {
				have = (unsigned)__builtin_amdgcn_readlane((int)v, xcd);
			}
			if (err != 0u) {
				dead = true;
				break;
			}
			if ((int)(have - target) >= 0) break;
			if (++spins >= max_spins) {
				if (lane == 0) __hip_atomic_store(&sync[SYNC_ERR * SL], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				dead = true;
				break;
			}
			__builtin_amdgcn_s_sleep(1);
		}
		if (lane == 0 && dead) *s_dead = 1;
	}
	__syncthreads();
	return *s_dead == 0;
}

// The column tiles a GEMV workgroup owns of one projection, held in registers: tiles g and g + ng, NS steps of 4 KiB
// each (a step past the end of the slab, or a tile past the matrix, reads as zeros through the buffer range check).
template <int NS>
struct WTiles {
	i32x4 v[2][NS];
	float sa[2], sb[2];  // thread tid < C: scale of column tid (GeGLU: of up column tid and of gate column tid)
};
template <int NS, bool GEGLU>
__device__ __forceinline__ void tiles_issue(WTiles<NS> &w, const int8_t *W, const float *scales, const TgFusedMat &m, int g, int ng) {
	const uint32_t slab = (uint32_t)m.K * (uint32_t)m.C;
	const int ncol = GEGLU ? (m.C >> 1) : m.C;
	const int c = (int)threadIdx.x < ncol ? (int)threadIdx.x : 0;
#pragma unroll
	for (int t = 0; t < 2; t++) {
		const int tile = g + t * ng;
		const bool have = tile < m.ntiles;
		const int tl = have ? tile : m.ntiles - 1;
		w.sa[t] = scales[tl * m.C + c];
		w.sb[t] = GEGLU ? scales[tl * m.C + (m.C >> 1) + c] : 0.0f;
		const __amdgpu_buffer_rsrc_t rw = make_rsrc(W + (size_t)tl * slab, have ? slab : 0u);
#pragma unroll
		for (int u = 0; u < NS; u++) w.v[t][u] = ldw<TG_W_DEFAULT>(rw, (uint32_t)threadIdx.x * 16u, min((uint32_t)u * STEP_BYTES, slab));
	}
}
// y = scales * (x . W) for the workgroup's tiles; xval(u) = the 4 inputs of this lane's rows in step u
template <int NS, int EPI, class XF>
__device__ __forceinline__ void tiles_compute(const WTiles<NS> &w, const TgFusedMat &m, int g, int ng, XF xval, float (*red2)[NWAVE][TG_CT], float *y,
                                              const float *lut, float gmin, float geps, int lut_size) {
	const int LC = m.C >> 2;
#pragma unroll
	for (int t = 0; t < 2; t++) {
		const int tile = g + t * ng;
		if (tile < m.ntiles) {  // uniform over the workgroup
			float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
			for (int u = 0; u < NS; u++) fma16(acc, w.v[t][u], xval(u));
			lanes_reduce(acc, LC, red2[t]);
			__syncthreads();
			if (EPI == TG_EPI_STORE) epi_store<true>(red2[t], m.C, tile, w.sa[t], y);
			else epi_geglu<true>(red2[t], m.C, tile, w.sa[t], w.sb[t], y, lut, gmin, geps, lut_size);
		}
	}
}

template <int NQ, int NO, int NU, int ND>
__global__ __launch_bounds__(NT) void decode_fused_kernel(const TgFused f) {
	__shared__ __attribute__((aligned(16))) float xs[TG_MAX_HIDDEN];
	__shared__ __attribute__((aligned(16))) float lut_s[LUT_LDS];
	__shared__ __attribute__((aligned(16))) float red2[2][NWAVE][TG_CT];
	__shared__ float sred[NWAVE];
	__shared__ float wgt[4][TG_ATTN_MERGE_MAX];
	__shared__ float s_bv[NWAVE];
	__shared__ int s_bi[NWAVE];
	__shared__ int s_dead;

	const int tid = threadIdx.x;
	const int xcd = fused_xcc_id();
	const int ng = f.ng, h = f.hidden;
	if (tid == 0) s_dead = 0;
	// optional timestamps (100 MHz counter) of GEMV workgroup 0 and attention workgroup 0: ts[layer][24]
	auto stamp = [&](int l, int e) {
		if (f.ts != nullptr && tid == 0 && ((int)blockIdx.x == 0 || (int)blockIdx.x == ng)) f.ts[l * 24 + e] = __builtin_amdgcn_s_memrealtime();
	};
	// keys and attention workgroups of a layer at this position
	auto layer_chunk = [&](int is_sw) { return is_sw ? f.chunk_local : f.chunk_global; };
	auto layer_nb = [&](int max_pos, int is_sw) {
		const int valid = (f.pos + 1 < max_pos) ? f.pos + 1 : max_pos;
		const int c = layer_chunk(is_sw);
		return (valid + c - 1) / c;
	};
	__syncthreads();

	if ((int)blockIdx.x >= ng) {
		// ---------------- attention workgroup ----------------
		const int a = (int)blockIdx.x - ng;
		for (int l = 0; l < f.L; l++) {
			const TgFusedLayer Ld = f.layers[l];
			float *xl = f.xch + (size_t)l * f.layer_stride;
			TgAttnDecode ad;
			ad.qkv = xl + f.off_qkv;
			ad.rms_q = Ld.rms_q;
			ad.rms_k = Ld.rms_k;
			ad.cos_t = Ld.is_sw ? f.cos_l : f.cos_g;
			ad.sin_t = Ld.is_sw ? f.sin_l : f.sin_g;
			ad.kc = Ld.kc;
			ad.vc = Ld.vc;
			ad.max_pos = Ld.max_pos;
			ad.pos = nullptr;
			ad.bp_index = 0;
			ad.host_pos = f.pos;
			ad.host_bp = Ld.is_sw ? f.bp_local : f.bp_global;
			ad.chunk = layer_chunk(Ld.is_sw);
			ad.part_acc = xl + f.off_pacc;
			ad.part_ml = xl + f.off_pml;
			ad.n_head = 4;
			ad.nblocks = 0;
			ad.host_cur = -1;
			const int nb = layer_nb(Ld.max_pos, Ld.is_sw);
			if (!fused_wait(f.sync, 0, f.all_base + (unsigned)(4 * l + 1) * (unsigned)ng, xcd, f.max_spins, &s_dead)) return;
			stamp(l, 16);
			tga::attn_decode_body<true>(ad, a, [] {});
			stamp(l, 17);
			fused_arrive(f.sync, 1, xcd, a < nb);
			stamp(l, 18);
		}
		return;
	}

	// ---------------- GEMV workgroup ----------------
	const int g = blockIdx.x;
	const bool lut_in_lds = f.lut_size <= LUT_LDS && (f.lut_size & 3) == 0;
	const float *lut = lut_in_lds ? lut_s : f.lut;
	float res[PER];  // the residual stream, element d = tid + i * NT
	WTiles<NQ> wq;
	WTiles<NO> wo;
	WTiles<NU> wu;
	WTiles<ND> wd;
	float wpo[PER], wpre[PER];
	auto load_vec = [&](float (&dst)[PER], const float *src) {
#pragma unroll
		for (int i = 0; i < PER; i++) {
			const int d = tid + i * NT;
			const float val = src[d < h ? d : h - 1];  // clamped index + select: no branch, no wait per load
			dst[i] = (d < h) ? val : 0.0f;
		}
	};
	auto xs_val = [&](const TgFusedMat &m) {
		const int kpos = tid >> m.lc_shift, KL = NT >> m.lc_shift, xlast = m.K - 4;
		return [=](int u) -> f32x4 {
			int idx = 4 * (kpos + u * KL);
			idx = idx < xlast ? idx : xlast;  // lanes past K: their weights read as 0, any finite x will do
			return *reinterpret_cast<const f32x4 *>(&xs[idx]);
		};
	};
	unsigned attn_target = f.attn_base;

	// ---- first layer: embedding of the token (ops.hpp:537-568); the previous step's pick may still be pending ----
	{
		int tok;
		if (f.am_val != nullptr) {
			tok = argmax_pairs(f.am_val, f.am_idx, f.am_n, s_bv, s_bi);
			if (g == 0 && tid == 0) record_pick(tok, f.am_ctr, f.am_log, 1);
		} else {
			tok = *f.tok;
		}
		tok = tok < 0 ? 0 : (tok >= f.vocab ? f.vocab - 1 : tok);
		const int8_t *row = f.wte + (size_t)tok * h;
#pragma unroll
		for (int i = 0; i < PER; i++) {
			const int d = tid + i * NT;
			const int dd = d < h ? d : h - 1;
			const float val = embed_value(f.wte_scales[dd], f.emb_scale, row[dd]);
			res[i] = (d < h) ? val : 0.0f;
		}
		load_vec(wpre, f.layers[0].apre);
		if (lut_in_lds) {
			const f32x4 lv = *reinterpret_cast<const f32x4 *>(f.lut + (4 * tid < f.lut_size ? 4 * tid : 0));
			if (4 * tid < f.lut_size) *reinterpret_cast<f32x4 *>(&lut_s[4 * tid]) = lv;
		}
		tiles_issue<NQ, false>(wq, f.layers[0].Wqkv, f.layers[0].sqkv, f.mqkv, g, ng);
	}

	for (int l = 0; l < f.L; l++) {
		const TgFusedLayer Ld = f.layers[l];
		float *xl = f.xch + (size_t)l * f.layer_stride;
		const unsigned base = f.all_base + (unsigned)(4 * l) * (unsigned)ng;

		// ---- pre-norm + Q|K|V (modules.hpp:137-144) ----
		stamp(l, 0);
		if (l > 0) {
			// post-norm of the previous layer's MLP + residual (modules.hpp:218-219)
			float p[PER];
			load_vec(p, f.xch + (size_t)(l - 1) * f.layer_stride + f.off_d);
			const float ss = block_sum(sumsq(p), sred);
			float t[PER];
			post_norm_add(t, p, rms_inv(ss, h), wpo, res);
#pragma unroll
			for (int i = 0; i < PER; i++) res[i] = t[i];
		}
		if (g == 0) {
			float *xr_in = f.xr + (size_t)(2 * l) * h;
#pragma unroll
			for (int i = 0; i < PER; i++) {
				const int d = tid + i * NT;
				if (d < h) xr_in[d] = res[i];
			}
		}
		{
			const float ss = block_sum(sumsq(res), sred);
			pre_norm_store(xs, res, rms_inv(ss, h), wpre, h);
			__syncthreads();
		}
		stamp(l, 1);
		tiles_compute<NQ, TG_EPI_STORE>(wq, f.mqkv, g, ng, xs_val(f.mqkv), red2, xl + f.off_qkv, nullptr, 0.0f, 0.0f, 0);
		stamp(l, 2);
		fused_arrive(f.sync, 0, xcd, true);
		stamp(l, 3);
		// the weights of the next two projections are requested now: they arrive while the attention workgroups work
		tiles_issue<NO, false>(wo, Ld.Wo, Ld.so, f.mo, g, ng);
		tiles_issue<NU, true>(wu, Ld.Wug, Ld.sug, f.mug, g, ng);
		load_vec(wpo, Ld.apost);
		load_vec(wpre, Ld.mpre);

		// ---- merge of the attention partials + output projection (modules.hpp:161-164) ----
		const int nb = layer_nb(Ld.max_pos, Ld.is_sw);
		attn_target += (unsigned)nb;
		if (!fused_wait(f.sync, 1, attn_target, xcd, f.max_spins, &s_dead)) return;
		stamp(l, 4);
		attn_merge_prologue(xs, wgt, xl + f.off_pacc, xl + f.off_pml, nb, [] {});
		stamp(l, 5);
		tiles_compute<NO, TG_EPI_STORE>(wo, f.mo, g, ng, xs_val(f.mo), red2, xl + f.off_o, nullptr, 0.0f, 0.0f, 0);
		stamp(l, 6);
		fused_arrive(f.sync, 0, xcd, true);
		stamp(l, 7);
		tiles_issue<ND, false>(wd, Ld.Wd, Ld.sd, f.md, g, ng);
		if (!fused_wait(f.sync, 0, base + 2u * (unsigned)ng, xcd, f.max_spins, &s_dead)) return;
		stamp(l, 8);

		// ---- post-norm + residual of the attention block, pre-norm, up|gate, gelu(gate) * up (modules.hpp:166-168, 205-215) ----
		{
			float p[PER];
			load_vec(p, xl + f.off_o);
			const float ss = block_sum(sumsq(p), sred);
			float t[PER];
			post_norm_add(t, p, rms_inv(ss, h), wpo, res);
#pragma unroll
			for (int i = 0; i < PER; i++) res[i] = t[i];
			if (g == 0) {
				float *xr_mid = f.xr + (size_t)(2 * l + 1) * h;
#pragma unroll
				for (int i = 0; i < PER; i++) {
					const int d = tid + i * NT;
					if (d < h) xr_mid[d] = res[i];
				}
			}
			const float ss2 = block_sum(sumsq(res), sred);
			pre_norm_store(xs, res, rms_inv(ss2, h), wpre, h);
			__syncthreads();
		}
		stamp(l, 9);
		tiles_compute<NU, TG_EPI_GEGLU>(wu, f.mug, g, ng, xs_val(f.mug), red2, xl + f.off_h, lut, f.gmin, f.geps, f.lut_size);
		stamp(l, 10);
		fused_arrive(f.sync, 0, xcd, true);
		stamp(l, 11);
		if (l + 1 < f.L) {
			tiles_issue<NQ, false>(wq, f.layers[l + 1].Wqkv, f.layers[l + 1].sqkv, f.mqkv, g, ng);
			load_vec(wpre, f.layers[l + 1].apre);
		}
		load_vec(wpo, Ld.mpost);
		if (!fused_wait(f.sync, 0, base + 3u * (unsigned)ng, xcd, f.max_spins, &s_dead)) return;
		stamp(l, 12);

		// ---- down projection (modules.hpp:216-217): the input comes straight from the exchange buffer ----
		{
			const int kpos = tid >> f.md.lc_shift, KL = NT >> f.md.lc_shift;
			const uint32_t xbytes = (uint32_t)f.md.K * 4u;
			const __amdgpu_buffer_rsrc_t rx = make_rsrc(xl + f.off_h, xbytes);
			f32x4 xq[ND];
#pragma unroll
			for (int u = 0; u < ND; u++) xq[u] = ldx(rx, (uint32_t)kpos * 16u, min((uint32_t)u * (uint32_t)KL * 16u, xbytes));
			tiles_compute<ND, TG_EPI_STORE>(wd, f.md, g, ng, [&](int u) -> f32x4 { return xq[u]; }, red2, xl + f.off_d, nullptr, 0.0f, 0.0f, 0);
		}
		stamp(l, 13);
		fused_arrive(f.sync, 0, xcd, true);
		stamp(l, 14);
		if (l + 1 < f.L) {
			if (!fused_wait(f.sync, 0, base + 4u * (unsigned)ng, xcd, f.max_spins, &s_dead)) return;
		}
		stamp(l, 15);
	}
}

int steps_of(const TgFusedMat &m) { return (m.K * m.C + (int)STEP_BYTES - 1) / (int)STEP_BYTES; }

}  // namespace

int tg_fused_variant(const TgFused &f) {
	const TgFusedMat *ms[4] = {&f.mqkv, &f.mo, &f.mug, &f.md};
	for (const TgFusedMat *m : ms)
		if (m->ntiles > 2 * f.ng || m->C < 4 || m->C > TG_CT || (m->K & 3)) return -1;
	if (f.hidden > TG_MAX_HIDDEN || f.mqkv.K != f.hidden || f.mug.K != f.hidden || f.mo.K != 4 * 256 || f.mo.K > TG_MAX_HIDDEN) return -1;
	if (f.ng < 8 || f.L < 1) return -1;
	const int q = steps_of(f.mqkv), o = steps_of(f.mo), u = steps_of(f.mug), d = steps_of(f.md);
	if (q <= 1 && o <= 1 && u <= 3 && d <= 2) return 1;
	if (q <= 2 && o <= 1 && u <= 9 && d <= 7) return 0;
	return -1;
}

bool tg_fused_supported(int n_cu) {
	// every workgroup must be resident at once: one per compute unit
	int per_cu0 = 0, per_cu1 = 0;
	if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu0, decode_fused_kernel<2, 1, 9, 7>, NT, 0) != hipSuccess) return false;
	if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu1, decode_fused_kernel<1, 1, 3, 2>, NT, 0) != hipSuccess) return false;
	return per_cu0 >= 1 && per_cu1 >= 1 && n_cu >= 64;
}

void tg_launch_decode_fused(const TgFused &f, int variant, hipStream_t s) {
	const dim3 grid((unsigned)(f.ng + TG_FUSED_ATTN_WGS)), block(NT);
	if (variant == 0) hipLaunchKernelGGL((decode_fused_kernel<2, 1, 9, 7>), grid, block, 0, s, f);
	else hipLaunchKernelGGL((decode_fused_kernel<1, 1, 3, 2>), grid, block, 0, s, f);
}

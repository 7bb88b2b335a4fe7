// Attention over the fp32 KV cache, plus the per-token work the reference does between the
// Q/K/V projections and the attention itself (modules.hpp:146-159): per-head RMSNorm of q and k,
// half-rotation RoPE, and the KV-cache write.
//
//   decode : ops::attention_decode (ops.hpp:224-370) — one query token, 4 heads sharing 1 KV head,
//            keys = the valid slots of a ring (local layers) or linear (global layers) cache.
//            The reference walks the slots sequentially with a renormalising online softmax; here
//            the slots are split across workgroups (flash-decoding), each writing an exact softmax
//            partial (max, sum, unnormalised output) of its chunk; the partials are merged in the
//            prologue of the output projection (tg_gemv.hip) — via attn_merge_kernel first when
//            there are many.  Softmax is order independent, so only fp32 rounding differs.
//   prefill: the per-row q/k work only (qk_norm_rope_rows_kernel); the attention itself is in
//            tg_attn_prefill.hip.

#include "tg_internal.h"
#include "tg_attn_decode.h"

using namespace tga;

namespace {

// The leading arguments repeat the descriptor's first-used fields so that the dispatcher preloads them into
// scalar registers (kernarg preload): the q/k-path loads go out without waiting for an s_load of the descriptor.
__global__ __launch_bounds__(ANT) void attn_decode_kernel(const float *qkv, const float *rms_q, const float *rms_k, const float *cos_t,
                                                          const float *sin_t, int host_pos, int host_bp, int nblocks, int chunk,
                                                          const TgAttnDecode a_in) {
	if (__builtin_expect((int)blockIdx.x >= nblocks, 0)) {  // extra workgroups: prefetch the next launch's weights and leave
		tg_prefetch_dispatch(a_in.pf, a_in.pf2, nblocks);
		return;
	}
	TgAttnDecode a = a_in;
	a.qkv = qkv;
	a.rms_q = rms_q;
	a.rms_k = rms_k;
	a.cos_t = cos_t;
	a.sin_t = sin_t;
	a.host_pos = host_pos;
	a.host_bp = host_bp;
	a.chunk = chunk;
	a.nblocks = nblocks;
	attn_decode_body<true>(a, (int)blockIdx.x, [] {});
}

// Long contexts only: folds every TG_ATTN_FOLD consecutive partials into one partial of the same form (maximum, sum,
// un-normalised output relative to that maximum), so that the consumer's merge stays at TG_ATTN_MERGE_MAX partials of
// TG_ATTN_FOLD * chunk keys each.  Workgroup = (head, 64 of its 256 dims, group of partials); lane = dim, the four waves
// share the group's partials round-robin and meet in LDS.
__global__ __launch_bounds__(ANT) void attn_merge_kernel(const TgAttnDecode a, float *merged_acc, float *merged_ml) {
	__shared__ float wg[TG_ATTN_FOLD];
	__shared__ float osum[4][64];
	__shared__ float s_ml[2];
	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, h = blockIdx.x, d = 64 * (int)blockIdx.y + lane, grp = blockIdx.z;
	const int pos = a.host_pos >= 0 ? a.host_pos : a.pos[0];
	const int valid = (pos + 1 < a.max_pos) ? pos + 1 : a.max_pos;
	const int b_lo = grp * TG_ATTN_FOLD;
	const int nb = min((valid + a.chunk - 1) / a.chunk - b_lo, TG_ATTN_FOLD);  // partials of this group
	if (nb <= 0) return;  // uniform over the workgroup: a fixed-size grid launched for a longer context
	// the wave's partials are requested before their weights are known: wave w takes b_lo + w, + 4, ...
	constexpr int U = TG_ATTN_FOLD / 4;
	float v[U];
#pragma unroll
	for (int u = 0; u < U; u++) {
		const int b = w + 4 * u;
		v[u] = a.part_acc[((size_t)(b_lo + (b < nb ? b : 0)) * NH + h) * HD + d];
	}
	if (w == 0) {
		const bool ok = lane < nb;  // TG_ATTN_FOLD == 64: one partial per lane
		const float m = ok ? a.part_ml[((size_t)(b_lo + lane) * NH + h) * 2] : -INFINITY;
		const float l = ok ? a.part_ml[((size_t)(b_lo + lane) * NH + h) * 2 + 1] : 0.0f;
		const float M = wmax(m);
		const float e = ok ? attn_exp(m - M) : 0.0f;  // as the attention kernel's own weights
		const float L = wsum(l * e);
		wg[lane] = e;
		if (lane == 0) {
			s_ml[0] = M;
			s_ml[1] = L;
		}
	}
	__syncthreads();
	float o = 0.0f;
#pragma unroll
	for (int u = 0; u < U; u++) o = fmaf(v[u], wg[w + 4 * u], o);  // weight 0 beyond nb
	osum[w][lane] = o;
	__syncthreads();
	if (w == 0) {
		merged_acc[((size_t)grp * NH + h) * HD + d] = (osum[0][lane] + osum[1][lane]) + (osum[2][lane] + osum[3][lane]);
		if (lane == 0 && blockIdx.y == 0) {
			merged_ml[((size_t)grp * NH + h) * 2 + 0] = s_ml[0];
			merged_ml[((size_t)grp * NH + h) * 2 + 1] = s_ml[1];
		}
	}
}

// ---------------------------------------------------------------------------------------------
// prefill
// ---------------------------------------------------------------------------------------------

// One workgroup per prompt position: q heads and k normalised + rotated in place
// (modules.hpp:115-119), k/v rows of the last min(S, max_pos) positions copied to cache slots
// 0.. (KVCache::update_prefill, decode.hpp:72-105).
__global__ __launch_bounds__(ANT) void qk_norm_rope_rows_kernel(float *q, float *k, const float *v, const float *rms_q,
                                                                const float *rms_k, const float *cos_t, const float *sin_t,
                                                                float *kc, float *vc, int max_pos, int S, int ldq, int ldkv) {
	const int s = blockIdx.x, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	const float *cs = cos_t + (size_t)s * (HD / 2), *sn = sin_t + (size_t)s * (HD / 2);
	float o[4];
	float *qrow = q + (size_t)s * ldq + w * HD;
	norm_rope_head(qrow, rms_q, cs, sn, 1.0f, o, lane);
#pragma unroll
	for (int i = 0; i < 4; i++) qrow[lane + 64 * i] = o[i];
	const int start = (S >= max_pos) ? S - max_pos : 0;
	float *krow = k + (size_t)s * ldkv;
	if (w == 0) {
		norm_rope_head(krow, rms_k, cs, sn, 1.0f, o, lane);
#pragma unroll
		for (int i = 0; i < 4; i++) {
			krow[lane + 64 * i] = o[i];
			if (s >= start) kc[(size_t)(s - start) * HD + lane + 64 * i] = o[i];
		}
	}
	if (s >= start) vc[(size_t)(s - start) * HD + tid] = v[(size_t)s * ldkv + tid];
}


}  // namespace

void tg_desc_attn_decode(const TgAttnDecode &a_in, int max_blocks, TgLaunchDesc *d) {
	TgAttnDecode &a = d->a;
	a = a_in;
	a.nblocks = max_blocks;
	if (a.pf.ptr == nullptr) a.pf.nblocks = 0;
	if (a.pf2.ptr == nullptr) a.pf2.nblocks = 0;
	d->func = reinterpret_cast<const void *>(&attn_decode_kernel);
	d->grid = dim3((unsigned)(max_blocks + a.pf.nblocks + a.pf2.nblocks));
	d->block = dim3(ANT);
	// qkv, rms_q, rms_k, cos_t, sin_t, host_pos, host_bp, nblocks, chunk, a
	d->p[0] = a.qkv;
	d->p[1] = a.rms_q;
	d->p[2] = a.rms_k;
	d->p[3] = a.cos_t;
	d->p[4] = a.sin_t;
	d->i[0] = a.host_pos;
	d->i[1] = a.host_bp;
	d->i[2] = a.nblocks;
	d->i[3] = a.chunk;
	for (int k = 0; k < 5; k++) d->args[k] = &d->p[k];
	for (int k = 0; k < 4; k++) d->args[5 + k] = &d->i[k];
	d->args[9] = &d->a;
}

// nblk: workgroups of the attention launch whose partials are folded
void tg_desc_attn_merge(const TgAttnDecode &a, int nblk, float *merged_acc, float *merged_ml, TgLaunchDesc *d) {
	static_assert(TG_ATTN_FOLD == 64 && TG_ATTN_MAX_BLOCKS == TG_ATTN_FOLD * TG_ATTN_MERGE_MAX, "one partial per lane; the consumer merges the rest");
	d->a = a;
	d->func = reinterpret_cast<const void *>(&attn_merge_kernel);
	d->grid = dim3(NH, HD / 64, (unsigned)((nblk + TG_ATTN_FOLD - 1) / TG_ATTN_FOLD));
	d->block = dim3(ANT);
	d->p[0] = merged_acc;
	d->p[1] = merged_ml;
	d->args[0] = &d->a;
	d->args[1] = &d->p[0];
	d->args[2] = &d->p[1];
}

bool tg_gemv_is_oproj(const void *func);  // tg_gemv.hip
int tg_decode_node_kind(const void *func) {
	if (func == reinterpret_cast<const void *>(&attn_decode_kernel)) return 1;
	if (func == reinterpret_cast<const void *>(&attn_merge_kernel)) return 2;
	return tg_gemv_is_oproj(func) ? 3 : 0;
}

void tg_launch_attn_decode(const TgAttnDecode &a, int max_blocks, hipStream_t s) {
	TgLaunchDesc d;
	tg_desc_attn_decode(a, max_blocks, &d);
	tg_launch_desc(d, s);
}

void tg_launch_attn_merge(const TgAttnDecode &a, int nblk, float *merged_acc, float *merged_ml, hipStream_t s) {
	TgLaunchDesc d;
	tg_desc_attn_merge(a, nblk, merged_acc, merged_ml, &d);
	tg_launch_desc(d, s);
}

void tg_launch_qk_norm_rope_rows(float *q, float *k, const float *v, const float *rms_q, const float *rms_k, const float *cos_t,
                                 const float *sin_t, float *kc, float *vc, int max_pos, int S, int n_head, int hd, int ldq, int ldkv,
                                 hipStream_t s) {
	(void)n_head;
	(void)hd;
	hipLaunchKernelGGL(qk_norm_rope_rows_kernel, dim3((unsigned)S), dim3(ANT), 0, s, q, k, v, rms_q, rms_k, cos_t, sin_t, kc, vc,
	                   max_pos, S, ldq, ldkv);
}


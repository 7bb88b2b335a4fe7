// Prefill attention (ops::attention_prefill, ops.hpp:377-526) on the fp32 matrix cores.
//
// The reference walks every (query, head) pair over its keys with a renormalising online softmax.
// Here a workgroup owns 16 consecutive query positions and all 4 query heads (one wave per head: the
// heads share the single KV head, so each K/V tile is fetched once per workgroup) and streams the
// keys in tiles of 32 through LDS.  Both products run on v_mfma_f32_16x16x4_f32: fp32 operands, exact
// fp32 products, fp32 accumulation, so only the summation order differs from the reference.
//
//   scores, transposed:  S^T[key][query] = K[key][:] . Q[query][:]      A = K tile (LDS), B = Q (registers)
//   lane (c = lane % 16, g = lane / 16) then holds S^T[4g + i][c], i = 0..3: the scores of query c,
//   which is exactly the A-operand order the second product needs:
//   output:              O[query][d] += P[query][key] * V[key][d]       A = P (registers), B = V tile (LDS)
//
// The k index of an MFMA step is arbitrary as long as A and B agree, so step (t, i) of the score product
// uses k = 16 t + 4 g + i: every lane fetches 4 consecutive floats of its K row with one 16-byte LDS
// read, and the Q registers are filled with 16-byte global loads.  LDS rows are 260 floats apart: the 16
// rows of a read hit 16 different groups of 4 banks (scores) and the 4 rows of a V read are 16 banks
// apart.  Keys outside a query's range (causal; local layers: qs-window .. qs, ops.hpp:437-443) get a
// score of -inf.
//
// Balance.  A causal layer gives query tile i about i/2 key tiles of work, and at a few thousand tokens there
// is only about one query tile per compute unit, so the last tile would set the pace at twice the mean.  Long
// key ranges are therefore cut into chunks of at most `chunk` key tiles: a work item = (query tile, chunk),
// listed by the host heaviest first.  An item of a split query tile leaves its un-normalised output rows with
// their running maximum and sum in scratch, and attn_prefill_merge_kernel folds the chunks of a row together
// (the flash-decoding merge: weights exp(m_c - max m) / sum).

#include "tg_internal.h"

#include <algorithm>
#include <vector>

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int HD = 256;    // head_dim
constexpr int NH = 4;      // query heads (= waves per workgroup)
constexpr int TQ = 16;     // query positions per workgroup
constexpr int TK = 32;     // keys per LDS tile
constexpr int LDS_LD = 260;
constexpr int PNT = 256;

// items == nullptr: workgroup b owns query tile gridDim.x - 1 - b and all its keys.
// items != nullptr (causal layers only): items[b] = {query tile, first key tile, end key tile, slot}; slot < 0: the
// item is the whole key range of its query tile and writes o; else it writes part_o[slot][16][NH][HD] (un-normalised)
// and part_ml[slot][16][NH][2] (running maximum, running sum).
__global__ __launch_bounds__(PNT) void attn_prefill_mfma_kernel(float *o, const float *q, const float *k, const float *v, int S, int ldq,
                                                               int ldkv, int ldo, int is_sw, int window, const int4 *items,
                                                               float *part_o, float *part_ml, float *rowmax_part, int Mpad) {
	__shared__ __attribute__((aligned(16))) float Ks[TK][LDS_LD];
	__shared__ __attribute__((aligned(16))) float Vs[TK][LDS_LD];

	const int tid = threadIdx.x, lane = tid & 63, head = tid >> 6, c = lane & 15, g = lane >> 4;
	// late query tiles of a causal layer see the most keys: start them first
	int q0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * TQ, slot = -1;
	int4 item = int4{0, 0, 0, -1};
	if (items != nullptr) {
		item = items[blockIdx.x];
		q0 = item.x * TQ;
		slot = item.w;
	}
	const int qpos = q0 + c;                         // the query whose scores this lane holds
	const int qrow = qpos < S ? qpos : S - 1;
	int kb = (is_sw && q0 > window) ? q0 - window : 0;
	int ke = (q0 + TQ < S) ? q0 + TQ : S;            // exclusive
	if (items != nullptr) {
		kb = item.y * TK;
		ke = min(ke, item.z * TK);
	}
	const int ntiles = (ke - kb + TK - 1) / TK;
	const int klo = is_sw ? qpos - window : 0;       // this query's first key (may be negative)

	// K/V tile staging: thread covers rows (tid/64) + 4u, 16-byte piece tid % 64
	const int ld_row = tid >> 6, ld_piece = tid & 63;
	f32x4 kpre[TK / 4], vpre[TK / 4];
	auto fetch = [&](int tile) {
#pragma unroll
		for (int u = 0; u < TK / 4; u++) {
			int j = kb + tile * TK + ld_row + 4 * u;
			j = j < ke ? j : ke - 1;
			kpre[u] = *reinterpret_cast<const f32x4 *>(k + (size_t)j * ldkv + 4 * ld_piece);
			vpre[u] = *reinterpret_cast<const f32x4 *>(v + (size_t)j * ldkv + 4 * ld_piece);
		}
	};
	fetch(0);

	// Q as B operand: qreg[t][i] = Q[qrow][16 t + 4 g + i] / sqrt(hd)   (ops.hpp:406,463)
	f32x4 qreg[HD / 16];
	{
		const float *qp = q + (size_t)qrow * ldq + head * HD + 4 * g;
#pragma unroll
		for (int t = 0; t < HD / 16; t++) {
			const float4 x = *reinterpret_cast<const float4 *>(qp + 16 * t);
			qreg[t] = f32x4{x.x * 0.0625f, x.y * 0.0625f, x.z * 0.0625f, x.w * 0.0625f};
		}
	}

	f32x4 oacc[HD / 16];  // oacc[dt][i] = O[query 4 g + i][16 dt + c]
#pragma unroll
	for (int dt = 0; dt < HD / 16; dt++) oacc[dt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
	float m_run = -INFINITY, l_run = 0.0f;  // of query c (replicated in the 4 lanes sharing c)

	for (int tile = 0; tile < ntiles; tile++) {
		tg_lds_barrier();  // everyone is done with the previous tile
#pragma unroll
		for (int u = 0; u < TK / 4; u++) {
			*reinterpret_cast<f32x4 *>(&Ks[ld_row + 4 * u][4 * ld_piece]) = kpre[u];
			*reinterpret_cast<f32x4 *>(&Vs[ld_row + 4 * u][4 * ld_piece]) = vpre[u];
		}
		tg_lds_barrier();
		if (tile + 1 < ntiles) fetch(tile + 1);  // in flight during the products

		// ---- scores of the tile's two groups of 16 keys ----
		f32x4 s0 = f32x4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;
#pragma unroll
		for (int t = 0; t < HD / 16; t++) {
			const f32x4 a0 = *reinterpret_cast<const f32x4 *>(&Ks[c][16 * t + 4 * g]);
			const f32x4 a1 = *reinterpret_cast<const f32x4 *>(&Ks[16 + c][16 * t + 4 * g]);
#pragma unroll
			for (int i = 0; i < 4; i++) {
				s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[i], qreg[t][i], s0, 0, 0, 0);
				s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[i], qreg[t][i], s1, 0, 0, 0);
			}
		}
		// ---- mask + online softmax for query c ----
		const int j0 = kb + tile * TK + 4 * g;
		float tmax = -INFINITY;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			const int ja = j0 + i, jb = j0 + 16 + i;
			if (ja > qpos || ja < klo) s0[i] = -INFINITY;
			if (jb > qpos || jb < klo) s1[i] = -INFINITY;
			tmax = fmaxf(tmax, fmaxf(s0[i], s1[i]));
		}
		tmax = fmaxf(tmax, tg_red_partner<16>(tmax));
		tmax = fmaxf(tmax, tg_red_partner<32>(tmax));
		const float m_new = fmaxf(m_run, tmax);  // finite from the first tile on: it holds a valid key of every query
		const float alpha = expf(m_run - m_new);
		float psum = 0.0f;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			s0[i] = expf(s0[i] - m_new);
			s1[i] = expf(s1[i] - m_new);
			psum += s0[i] + s1[i];
		}
		psum += tg_red_partner<16>(psum);
		psum += tg_red_partner<32>(psum);
		l_run = fmaf(l_run, alpha, psum);
		m_run = m_new;
		// rescale the output rows this lane holds (queries 4 g + i)
		float ar[4];
#pragma unroll
		for (int i = 0; i < 4; i++) ar[i] = __shfl(alpha, 4 * g + i, 64);
#pragma unroll
		for (int dt = 0; dt < HD / 16; dt++) {
#pragma unroll
			for (int i = 0; i < 4; i++) oacc[dt][i] *= ar[i];
		}
		// ---- O += P V : step i of key group kt uses key 16 kt + 4 g + i ----
#pragma unroll
		for (int dt = 0; dt < HD / 16; dt++) {
#pragma unroll
			for (int i = 0; i < 4; i++) {
				oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(s0[i], Vs[4 * g + i][16 * dt + c], oacc[dt], 0, 0, 0);
			}
#pragma unroll
			for (int i = 0; i < 4; i++) {
				oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(s1[i], Vs[16 + 4 * g + i][16 * dt + c], oacc[dt], 0, 0, 0);
			}
		}
	}

	if (slot >= 0) {  // one chunk of a split query tile: un-normalised rows + (m, l) per (query, head)
		float *po = part_o + (size_t)slot * TQ * NH * HD;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			float *op = po + ((size_t)(4 * g + i) * NH + head) * HD + c;
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) op[16 * dt] = oacc[dt][i];
		}
		if (g == 0) {
			float *pm = part_ml + (((size_t)slot * TQ + c) * NH + head) * 2;
			pm[0] = m_run;
			pm[1] = l_run;
		}
		return;
	}
	float lr[4];
#pragma unroll
	for (int i = 0; i < 4; i++) lr[i] = __shfl(l_run, 4 * g + i, 64);
#pragma unroll
	for (int i = 0; i < 4; i++) {
		const int qo = q0 + 4 * g + i;
		float omax = 0.0f;
		if (qo < S) {
			float *op = o + (size_t)qo * ldo + head * HD + c;
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) {
				const float val = oacc[dt][i] / lr[i];
				op[16 * dt] = val;
				omax = fmaxf(omax, fabsf(val));
			}
		}
		// the output projection quantises these rows next: leave max|row| over this head's columns for it
		if (rowmax_part != nullptr) {
			omax = tg_row16_max(omax);
			if (c == 0 && qo < S) rowmax_part[(size_t)head * Mpad + qo] = omax;
		}
	}
}

// One workgroup per query position of a split query tile; wave = head, lane = 4 consecutive dims.
// split[b] = {query tile, first slot, number of chunks}.
__global__ __launch_bounds__(PNT) void attn_prefill_merge_kernel(float *o, int S, int ldo, const int4 *split, const float *part_o,
                                                                const float *part_ml, float *rowmax_part, int Mpad) {
	const int4 sp = split[blockIdx.x / TQ];
	const int qi = blockIdx.x % TQ, qpos = sp.x * TQ + qi;
	if (qpos >= S) return;
	const int lane = threadIdx.x & 63, head = threadIdx.x >> 6;
	float M = -INFINITY;
	for (int ch = 0; ch < sp.z; ch++) M = fmaxf(M, part_ml[(((size_t)(sp.y + ch) * TQ + qi) * NH + head) * 2]);
	float L = 0.0f;
	f32x4 acc = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
	for (int ch = 0; ch < sp.z; ch++) {
		const size_t row = ((size_t)(sp.y + ch) * TQ + qi) * NH + head;
		const float wgt = expf(part_ml[row * 2] - M);
		L = fmaf(part_ml[row * 2 + 1], wgt, L);
		const f32x4 x = *reinterpret_cast<const f32x4 *>(part_o + row * HD + 4 * lane);
		acc += x * wgt;
	}
	const f32x4 res = acc / L;
	*reinterpret_cast<f32x4 *>(o + (size_t)qpos * ldo + head * HD + 4 * lane) = res;
	if (rowmax_part != nullptr) {
		const float omax = tg_wave_max(fmaxf(fmaxf(fabsf(res[0]), fabsf(res[1])), fmaxf(fabsf(res[2]), fabsf(res[3]))));
		if (lane == 0) rowmax_part[(size_t)head * Mpad + qpos] = omax;
	}
}

}  // namespace

// Work list of a causal layer of S tokens, for tg_launch_attn_prefill.  Returns false when no query tile needs
// splitting (then the plain launch is already balanced).  items: one int4 per workgroup, heaviest first;
// split: one int4 per split query tile; nslots: chunks that go through scratch.
bool tg_attn_prefill_plan(int S, int n_cu, std::vector<int4> &items, std::vector<int4> &split, int &nslots) {
	const int nq = (S + TQ - 1) / TQ;
	auto ntiles_of = [&](int qt) { return (std::min(qt * TQ + TQ, S) + TK - 1) / TK; };
	long total = 0;
	for (int qt = 0; qt < nq; qt++) total += ntiles_of(qt);
	// about 8 items per compute unit, and never chunks below 16 key tiles (512 keys)
	const int chunk = (int)std::max<long>(16, total / ((long)n_cu * 8));
	items.clear();
	split.clear();
	nslots = 0;
	for (int qt = 0; qt < nq; qt++) {
		const int nt = ntiles_of(qt), nc = (nt + chunk - 1) / chunk;
		if (nc == 1) {
			items.push_back(int4{qt, 0, nt, -1});
			continue;
		}
		split.push_back(int4{qt, nslots, nc, 0});
		for (int ch = 0; ch < nc; ch++) {  // equal chunks
			const int tb = (int)((long)nt * ch / nc), te = (int)((long)nt * (ch + 1) / nc);
			items.push_back(int4{qt, tb, te, nslots++});
		}
	}
	if (split.empty()) return false;
	std::stable_sort(items.begin(), items.end(), [](const int4 &a, const int4 &b) { return a.z - a.y > b.z - b.y; });
	return true;
}
size_t tg_attn_prefill_part_floats(int nslots) { return (size_t)nslots * TQ * NH * HD; }
size_t tg_attn_prefill_ml_floats(int nslots) { return (size_t)nslots * TQ * NH * 2; }

// q/k/v: rows of S tokens (q already normalised and rotated, ldq floats apart; k, v ldkv apart); o [S][ldo]
void tg_launch_attn_prefill(float *o, const float *q, const float *k, const float *v, int S, int n_head, int hd, int ldq, int ldkv,
                            int ldo, int is_sw, int window, const TgAttnPrefillPlan *plan, float *rowmax_part, hipStream_t s) {
	(void)n_head;
	(void)hd;
	const int Mpad = (int)tg_gemm_mfma_rows(S);  // rowmax_part (may be null): [4 heads][Mpad], max|o[row][head's columns]|
	if (plan == nullptr || is_sw) {
		hipLaunchKernelGGL(attn_prefill_mfma_kernel, dim3((unsigned)((S + TQ - 1) / TQ)), dim3(PNT), 0, s, o, q, k, v, S, ldq, ldkv, ldo,
		                   is_sw, window, (const int4 *)nullptr, (float *)nullptr, (float *)nullptr, rowmax_part, Mpad);
		return;
	}
	hipLaunchKernelGGL(attn_prefill_mfma_kernel, dim3((unsigned)plan->nitems), dim3(PNT), 0, s, o, q, k, v, S, ldq, ldkv, ldo, 0, window,
	                   plan->items, plan->part_o, plan->part_ml, rowmax_part, Mpad);
	hipLaunchKernelGGL(attn_prefill_merge_kernel, dim3((unsigned)(plan->nsplit * TQ)), dim3(PNT), 0, s, o, S, ldo, plan->split,
	                   plan->part_o, plan->part_ml, rowmax_part, Mpad);
}

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
#include <functional>
#include <map>
#include <queue>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int HD = 256;    // head_dim
constexpr int NH = 4;      // query heads (= waves per workgroup)
constexpr int TQ = 16;     // query positions per workgroup
constexpr int TK = 32;     // keys per LDS tile
constexpr int LDS_LD = 260;
constexpr int PNT = 256;

// Query tile of workgroup b of a launch without a work list.  Causal layer: late tiles see the most keys and start
// first.  Local layer (all tiles cost the same): workgroups go to the 8 XCDs round-robin, and XCD x takes a contiguous
// run of tiles, so that the workgroups it runs side by side have nearly the same key window and find each other's K/V
// tiles in its L2.
__device__ __forceinline__ int plain_query_tile(int is_sw) {
	const int n = (int)gridDim.x, b = (int)blockIdx.x;
	if (!is_sw) return n - 1 - b;
	const int x = b & 7, k = b >> 3, base = n >> 3, rem = n & 7;
	return x * base + (x < rem ? x : rem) + k;
}

// items == nullptr: workgroup b owns query tile plain_query_tile() and all its keys.
// items != nullptr (a work list, see tg_attn_prefill_plan): items[b] = {query tile, first key tile, end key tile, slot}; slot < 0: the
// item is the whole key range of its query tile and writes o; else it writes part_o[slot][16][NH][HD] (un-normalised)
// and part_ml[slot][16][NH][2] (running maximum, running sum).
__global__ __launch_bounds__(PNT) void attn_prefill_mfma_kernel(float *o, const float *q, const float *k, const float *v, int S, int ldq,
                                                               int ldkv, int ldo, int is_sw, int window, const int4 *items,
                                                               float *part_o, float *part_ml) {
	__shared__ __attribute__((aligned(16))) float Ks[TK][LDS_LD];
	__shared__ __attribute__((aligned(16))) float Vs[TK][LDS_LD];

	const int tid = threadIdx.x, lane = tid & 63, head = tid >> 6, c = lane & 15, g = lane >> 4;
	// late query tiles of a causal layer see the most keys: start them first
	int q0 = plain_query_tile(is_sw) * TQ, slot = -1;
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
		const float m_new = fmaxf(m_run, tmax);
		// A chunk of a local layer's work list may start a few keys before a query's window: nothing valid yet, the
		// running maximum stays -inf and every weight of the tile must come out as 0, not as exp(-inf + inf).
		const float m_ref = (m_new == -INFINITY) ? 0.0f : m_new;
		const float alpha = expf(m_run - m_ref);
		float psum = 0.0f;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			s0[i] = expf(s0[i] - m_ref);
			s1[i] = expf(s1[i] - m_ref);
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
	float lr[4];  // 1 / l of the lane's four query rows: one division per row, then multiplications
#pragma unroll
	for (int i = 0; i < 4; i++) lr[i] = 1.0f / __shfl(l_run, 4 * g + i, 64);
#pragma unroll
	for (int i = 0; i < 4; i++) {
		const int qo = q0 + 4 * g + i;
		if (qo < S) {
			float *op = o + (size_t)qo * ldo + head * HD + c;
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) op[16 * dt] = oacc[dt][i] * lr[i];
		}
	}
}

// ---- the same computation on the bf16 matrix cores, fp32-accurate -------------------------------------------
// An fp32 number is the sum of three bf16 numbers (8 + 8 + 8 significant bits): x = h + m + l with h = bf16(x),
// m = bf16(x - h), l = bf16(x - h - m), the two differences exact.  A product of two such sums keeps fp32 accuracy
// with six of the nine cross terms (hh, hm, mh, mm, hl, lh; the dropped ones are below 2^-24 of the product), every
// bf16 x bf16 product is exact in fp32 and the matrix core accumulates in fp32: measured error of a 32-term dot
// product 5e-8 of the sum of magnitudes, against 1.3e-7 for an fp32 fused chain.  v_mfma_f32_16x16x32_bf16 does 8
// times the work of v_mfma_f32_16x16x4_f32 in half the cycles, so six of them per product still run 2.7 times
// faster than the fp32 matrix path.
//
// Layout of v_mfma_f32_16x16x32_bf16: lane (r = lane % 16, g = lane / 16) holds A[r][8g..8g+7], B[8g..8g+7][r] and
// C[4g..4g+3][r].  As above only the pairing of A and B slots matters, so
//   scores:  A = K tile, lane holds dims 32t + 8g .. + 7 of key r (+16 for the second half), B = Q likewise:
//            C[4g+i][c] = S^T[key 4g+i][query c]: lane again holds 4 keys of query c per half;
//   output:  A = P, lane's 8 slots = its 8 scores: keys 4g..4g+3 and 16+4g..16+4g+3; B = V with the same key order,
//            so V is stored in LDS dim-major with those 8 keys of a group adjacent (one 16-byte read per operand).
// K and V tiles are split into their three planes once per workgroup when they are staged (shared by the 4 heads
// and 16 queries); Q is split once, P once per tile and wave.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Operand formats of the split path.
//   FmtBf16x3: three bf16 planes, six products, as described above.  bf16 has fp32's exponent range: no input can
//              fall outside it.
//   FmtF16x2 : x = h + l with h = fp16(x), l = fp16(x - h): 11 + 11 significant bits, three products (hh, hl, lh; the
//              dropped ll is below 2^-22 of the product), half the matrix instructions and two thirds of the LDS traffic
//              of the bf16 form.  The matrix cores take fp16 subnormals as they are (checked on the MI355X: 2^-24 x
//              16384 summed 32 times gives 2^-5), so small values only lose what lies below 2^-25 in absolute terms;
//              an element of magnitude 0.25 or more keeps 22 bits, i.e. 1.2e-7 relative, next to fp32's 6e-8.  The price
//              is the range: an operand beyond +-65504 does not fit.  q and k are RMS-normalised (|x| <= 16 |1 + w|)
//              and p lies in [0, 1]; v is a projection of a normalised vector.  The kernels track the largest
//              magnitude they convert and raise a flag if it does not fit, which the forward turns into an error.
struct FmtBf16x3 {
	typedef bf16x8 vec;
	typedef bf16x2 vec2;
	static constexpr int NP = 3;
	static constexpr float QSCALE = 0.0625f, SSCALE = 1.0f;  // 1/sqrt(head_dim) goes onto q before the split (exact: a power of two)
	static constexpr bool RANGE_CHECK = false;
};
struct FmtF16x2 {
	typedef f16x8 vec;
	typedef f16x2 vec2;
	static constexpr int NP = 2;
	static constexpr float QSCALE = 1.0f, SSCALE = 0.0625f;  // ... or onto the scores: q stays where fp16 resolves it best
	static constexpr bool RANGE_CHECK = true;
};
constexpr float F16_MAX = 65504.0f;

template <typename F>
struct PlanesT {
	typename F::vec p[F::NP];  // leading part, then the successive remainders
};
template <typename F>
__device__ __forceinline__ PlanesT<F> split8(const float *x) {
	PlanesT<F> o;
#pragma unroll
	for (int i = 0; i < 8; i += 2) {
		f32x2 r = {x[i], x[i + 1]};
#pragma unroll
		for (int pl = 0; pl < F::NP; pl++) {
			const typename F::vec2 a = __builtin_convertvector(r, typename F::vec2);  // round to nearest even
			o.p[pl][i] = a[0];
			o.p[pl][i + 1] = a[1];
			if (pl + 1 < F::NP) r = r - __builtin_convertvector(a, f32x2);  // exact
		}
	}
	return o;
}
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
// acc += a . b with the significant cross terms, smallest first
template <typename F>
__device__ __forceinline__ f32x4 mfma_terms(const PlanesT<F> &a, const PlanesT<F> &b, f32x4 acc) {
	if constexpr (F::NP == 3) {
		acc = mfma16(a.p[2], b.p[0], acc);
		acc = mfma16(a.p[0], b.p[2], acc);
		acc = mfma16(a.p[1], b.p[1], acc);
	}
	acc = mfma16(a.p[1], b.p[0], acc);
	acc = mfma16(a.p[0], b.p[1], acc);
	acc = mfma16(a.p[0], b.p[0], acc);
	return acc;
}
// largest magnitude among 8 values about to be converted (formats with a limited range only)
template <typename F>
__device__ __forceinline__ void track_range(unsigned &rmax, const float *x) {
	// largest magnitude as a bit pattern: unsigned order is magnitude order, and every NaN sorts above infinity
	if constexpr (F::RANGE_CHECK) {
#pragma unroll
		for (int i = 0; i < 8; i++) rmax = max(rmax, __float_as_uint(x[i]) & 0x7fffffffu);
	}
}
template <typename F>
__device__ __forceinline__ void report_range(unsigned rmax, int *range_flag) {
	if constexpr (F::RANGE_CHECK) {
		if (range_flag != nullptr && rmax > __float_as_uint(F16_MAX)) *range_flag = 1;  // too large, infinite or NaN
	}
}

// e^x for the softmax weights of the split-precision kernels: v_exp_f32 on x * log2(e), two instructions instead of
// the dozen of expf (range checks, extended-precision argument), which at nine exponentials per lane and key tile cost
// as much as the P.V matrix instructions (16,384 tokens of the 270m shape: 1.0 of 19.4 ms).  The product is rounded
// once: for x in [-10, 0], where the weights that matter lie, the exponent is off by at most 2^-21, i.e. the result by
// 3.3e-7 relative, a few units in the last place like the vectorised expf of the reference build; e^-inf = 0.
__device__ __forceinline__ float softmax_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }

constexpr int NT32 = HD / 32;  // k steps of a score product

// Same arguments and outputs as attn_prefill_mfma_kernel.  QG = groups of 16 query positions per workgroup, each
// with its own four waves (heads).  QG = 2: a K/V tile is fetched, split and staged once for 32 queries x 4 heads,
// and the two waves a SIMD then holds overlap each other's LDS reads, matrix and vector work; the launcher takes it
// for prompts long enough to keep the compute units busy with such workgroups, else QG = 1.
template <int QG, typename F>
__global__ __launch_bounds__(256 * QG) void attn_prefill_split_kernel(float *o, const float *q, const float *k, const float *v, int S, int ldq,
                                                                int ldkv, int ldo, int is_sw, int window, const int4 *items,
                                                                float *part_o, float *part_ml, int *range_flag) {
	typedef typename F::vec vec;
	typedef PlanesT<F> Planes;
	extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
	// Kb[plane][t][key][g]: dims 32t + 8g .. + 7 of a key; Vb[plane][g][dim]: the 8 keys of group g at one dim
	vec(*Kb)[NT32][TK][4] = reinterpret_cast<vec(*)[NT32][TK][4]>(smem);
	vec(*Vb)[4][HD] = reinterpret_cast<vec(*)[4][HD]>(smem + sizeof(vec) * F::NP * NT32 * TK * 4);
	unsigned rmax = 0u;
	constexpr int BQ = 16 * QG;   // query positions per workgroup
	constexpr int SU = 4 / QG;    // staging units per thread and operand

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, head = w & 3, qh = w >> 2, c = lane & 15, g = lane >> 4;
	int q0 = plain_query_tile(is_sw) * BQ, slot = -1;
	int4 item = int4{0, 0, 0, -1};
	if (items != nullptr) {
		item = items[blockIdx.x];
		q0 = item.x * BQ;
		slot = item.w;
	}
	const int q0w = q0 + 16 * qh;  // first query of this wave's group
	const int qpos = q0w + c;
	const int qrow = qpos < S ? qpos : S - 1;
	int kb = (is_sw && q0 > window) ? q0 - window : 0;
	int ke = (q0 + BQ < S) ? q0 + BQ : S;  // exclusive
	if (items != nullptr) {
		kb = item.y * TK;
		ke = min(ke, item.z * TK);
	}
	const int ntiles = (ke - kb + TK - 1) / TK;
	const int klo = is_sw ? qpos - window : 0;

	// staging.  K: thread = (key, g) of k steps t = tid / 128 + 2 QG u: 8 consecutive dims, two 16-byte loads.
	// V: thread = (dim 64 QG u + 64 (w / 4) + lane, group w % 4): the group's 8 keys at one dim, 4-byte loads (a wave
	// reads 256 contiguous bytes of a key row).
	const int sk_g = tid & 3, sk_key = (tid >> 2) & 31, sk_t0 = tid >> 7;
	const int sv_g = w & 3, sv_d = 64 * (w >> 2) + lane;
	f32x4 kpre[SU][2];
	float vpre[SU][8];
	auto key_row = [&](int tile, int key) {
		int j = kb + tile * TK + key;
		return (size_t)(j < ke ? j : ke - 1) * ldkv;
	};
	auto fetch = [&](int tile) {
		const float *kp = k + key_row(tile, sk_key) + 8 * sk_g;
#pragma unroll
		for (int u = 0; u < SU; u++) {
			kpre[u][0] = *reinterpret_cast<const f32x4 *>(kp + 32 * (sk_t0 + 2 * QG * u));
			kpre[u][1] = *reinterpret_cast<const f32x4 *>(kp + 32 * (sk_t0 + 2 * QG * u) + 4);
		}
#pragma unroll
		for (int sl = 0; sl < 8; sl++) {
			const float *vp = v + key_row(tile, (sl < 4 ? 4 * sv_g + sl : 12 + 4 * sv_g + sl)) + sv_d;
#pragma unroll
			for (int u = 0; u < SU; u++) vpre[u][sl] = vp[64 * QG * u];
		}
	};
	fetch(0);

	// Q planes: qp[t] = dims 32t + 8g .. + 7 of query c, scaled by 1/sqrt(hd) (a power of two: commutes with the split)
	Planes qp[NT32];
	{
		const float *qsrc = q + (size_t)qrow * ldq + head * HD + 8 * g;
#pragma unroll
		for (int t = 0; t < NT32; t++) {
			const f32x4 x0 = *reinterpret_cast<const f32x4 *>(qsrc + 32 * t), x1 = *reinterpret_cast<const f32x4 *>(qsrc + 32 * t + 4);
			float x[8];
#pragma unroll
			for (int e = 0; e < 4; e++) {
				x[e] = x0[e] * F::QSCALE;
				x[4 + e] = x1[e] * F::QSCALE;
			}
			track_range<F>(rmax, x);
			qp[t] = split8<F>(x);
		}
	}

	f32x4 oacc[HD / 16];  // oacc[dt][i] = O[query 4 g + i][16 dt + c]
#pragma unroll
	for (int dt = 0; dt < HD / 16; dt++) oacc[dt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
	float m_run = -INFINITY, l_run = 0.0f;

	for (int tile = 0; tile < ntiles; tile++) {
		tg_lds_barrier();  // everyone is done with the previous tile
#pragma unroll
		for (int u = 0; u < SU; u++) {
			float x[8];
#pragma unroll
			for (int e = 0; e < 4; e++) {
				x[e] = kpre[u][0][e];
				x[4 + e] = kpre[u][1][e];
			}
			track_range<F>(rmax, x);
			const Planes pl = split8<F>(x);
			const int t = sk_t0 + 2 * QG * u;
#pragma unroll
			for (int pn = 0; pn < F::NP; pn++) Kb[pn][t][sk_key][sk_g] = pl.p[pn];
		}
#pragma unroll
		for (int u = 0; u < SU; u++) {
			track_range<F>(rmax, vpre[u]);
			const Planes pl = split8<F>(vpre[u]);
#pragma unroll
			for (int pn = 0; pn < F::NP; pn++) Vb[pn][sv_g][64 * QG * u + sv_d] = pl.p[pn];
		}
		tg_lds_barrier();
		if (tile + 1 < ntiles) fetch(tile + 1);  // in flight during the products
		// a tile that starts behind this group's last query holds none of its keys (the other group still needs it)
		if (kb + tile * TK > q0w + 15) continue;

		// ---- scores of the tile's two groups of 16 keys; even and odd k steps in separate accumulators ----
		f32x4 sa[2][2];
#pragma unroll
		for (int hf = 0; hf < 2; hf++) sa[hf][0] = sa[hf][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
		for (int t = 0; t < NT32; t++) {
#pragma unroll
			for (int hf = 0; hf < 2; hf++) {
				Planes kf;
#pragma unroll
				for (int pn = 0; pn < F::NP; pn++) kf.p[pn] = Kb[pn][t][16 * hf + c][g];
				sa[hf][t & 1] = mfma_terms<F>(kf, qp[t], sa[hf][t & 1]);
			}
		}
		f32x4 s0 = (sa[0][0] + sa[0][1]) * F::SSCALE, s1 = (sa[1][0] + sa[1][1]) * F::SSCALE;
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
		const float m_new = fmaxf(m_run, tmax);
		const float m_ref = (m_new == -INFINITY) ? 0.0f : m_new;  // no valid key yet (see the fp32 kernel)
		const float alpha = softmax_exp(m_run - m_ref);
		float psum = 0.0f;
		float pv[8];  // the lane's 8 key slots: keys 4g + i, then 16 + 4g + i
#pragma unroll
		for (int i = 0; i < 4; i++) {
			pv[i] = softmax_exp(s0[i] - m_ref);
			pv[4 + i] = softmax_exp(s1[i] - m_ref);
			psum += pv[i] + pv[4 + i];
		}
		psum += tg_red_partner<16>(psum);
		psum += tg_red_partner<32>(psum);
		l_run = fmaf(l_run, alpha, psum);
		m_run = m_new;
		float ar[4];
#pragma unroll
		for (int i = 0; i < 4; i++) ar[i] = __shfl(alpha, 4 * g + i, 64);
#pragma unroll
		for (int dt = 0; dt < HD / 16; dt++) {
#pragma unroll
			for (int i = 0; i < 4; i++) oacc[dt][i] *= ar[i];
		}
		// ---- O += P V ----
		const Planes pp = split8<F>(pv);
#pragma unroll
		for (int dt = 0; dt < HD / 16; dt++) {
			Planes vf;
#pragma unroll
			for (int pn = 0; pn < F::NP; pn++) vf.p[pn] = Vb[pn][g][16 * dt + c];
			oacc[dt] = mfma_terms<F>(pp, vf, oacc[dt]);
		}
	}

	report_range<F>(rmax, range_flag);
	if (slot >= 0) {
		float *po = part_o + (size_t)slot * BQ * NH * HD;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			float *op = po + ((size_t)(16 * qh + 4 * g + i) * NH + head) * HD + c;
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) op[16 * dt] = oacc[dt][i];
		}
		if (g == 0) {
			float *pm = part_ml + (((size_t)slot * BQ + 16 * qh + c) * NH + head) * 2;
			pm[0] = m_run;
			pm[1] = l_run;
		}
		return;
	}
	float lr[4];  // 1 / l of the lane's four query rows: one division per row, then multiplications
#pragma unroll
	for (int i = 0; i < 4; i++) lr[i] = 1.0f / __shfl(l_run, 4 * g + i, 64);
#pragma unroll
	for (int i = 0; i < 4; i++) {
		const int qo = q0w + 4 * g + i;
		if (qo < S) {
			float *op = o + (size_t)qo * ldo + head * HD + c;
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) op[16 * dt] = oacc[dt][i] * lr[i];
		}
	}
}
template <typename F>
constexpr size_t split_lds_bytes() {
	return sizeof(typename F::vec) * F::NP * (NT32 * TK * 4 + 4 * HD);  // 96 KB with three planes, 64 KB with two
}

// ---- the same kernel fed from pre-split planes by a producer wave ------------------------------------------------
// In the kernel above every workgroup splits every K/V tile it uses into bf16 planes itself while staging it:
// measured, that staging (conversions + LDS writes through registers) is a third of a tile's time, and a K/V element
// is split again by each of the S/16 query tiles that see it.  Here a pre-pass (attn_planes_kernel) splits the K and V
// rows of a layer once and stores every 32-key tile as the exact image of the LDS arrays Kb and Vb (48 KB each); the
// attention workgroup then only copies images, with loads that write straight into LDS (no registers, no vector
// ALU work).  The images are used one per phase in the order K(0), V(0), K(1), V(1), ... (scores of a tile, then its
// P.V); LDS holds a ring of three of them (144 KB): every wave requests its share of image i + 2 when phase i starts,
// into the buffer phase i - 1 has just released, so every copy has two phases to arrive.  One workgroup barrier per
// phase keeps the waves in step.
constexpr size_t PLANE_BYTES = 16 * NT32 * TK * 4;  // one plane of a K image = one plane of a V image (16 KB)
static_assert(PLANE_BYTES == 16 * 4 * HD, "K and V images have the same size");
template <typename F>
constexpr size_t plane_img() {
	return F::NP * PLANE_BYTES;  // bytes of a K image = bytes of a V image: 48 KB with three planes, 32 KB with two
}
template <int N>
__device__ __forceinline__ void wait_loads_in_flight() {  // until at most N of this wave's vector memory loads are outstanding
	asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// One workgroup per 32-key tile: planes[tile] = K image, then V image.  Keys past S are written as zeros.
template <typename F>
__global__ __launch_bounds__(PNT) void attn_planes_kernel(unsigned char *planes, const float *k, const float *v, int S, int ldkv,
                                                         int *range_flag) {
	typedef typename F::vec vec;
	typedef PlanesT<F> Planes;
	constexpr size_t PLANE_IMG = plane_img<F>();
	const int tile = blockIdx.x, tid = threadIdx.x;
	vec *Kimg = reinterpret_cast<vec *>(planes + (size_t)tile * 2 * PLANE_IMG);
	vec *Vimg = reinterpret_cast<vec *>(planes + (size_t)tile * 2 * PLANE_IMG + PLANE_IMG);
	unsigned rmax = 0u;
	// K: unit = (t, key, g): dims 32t + 8g .. + 7 of a key -> Kb[plane][t][key][g]
#pragma unroll
	for (int u = 0; u < 4; u++) {
		const int unit = tid + PNT * u, g = unit & 3, key = (unit >> 2) & 31, t = unit >> 7;
		const int j = tile * TK + key;
		float x[8];
		const float *src = k + (size_t)(j < S ? j : S - 1) * ldkv + 32 * t + 8 * g;
		const f32x4 a = *reinterpret_cast<const f32x4 *>(src), b = *reinterpret_cast<const f32x4 *>(src + 4);
#pragma unroll
		for (int e = 0; e < 4; e++) {
			x[e] = j < S ? a[e] : 0.0f;
			x[4 + e] = j < S ? b[e] : 0.0f;
		}
		track_range<F>(rmax, x);
		const Planes pl = split8<F>(x);
		const size_t at = ((size_t)t * TK + key) * 4 + g;
#pragma unroll
		for (int pn = 0; pn < F::NP; pn++) Kimg[(size_t)pn * NT32 * TK * 4 + at] = pl.p[pn];
	}
	// V: unit = (g, dim): keys 4g .. 4g+3 and 16+4g .. 16+4g+3 at one dim -> Vb[plane][g][dim]
#pragma unroll
	for (int u = 0; u < 4; u++) {
		const int unit = tid + PNT * u, d = unit & 255, g = unit >> 8;
		float x[8];
#pragma unroll
		for (int sl = 0; sl < 8; sl++) {
			const int j = tile * TK + (sl < 4 ? 4 * g + sl : 12 + 4 * g + sl);
			const float val = v[(size_t)(j < S ? j : S - 1) * ldkv + d];
			x[sl] = j < S ? val : 0.0f;
		}
		track_range<F>(rmax, x);
		const Planes pl = split8<F>(x);
		const size_t at = (size_t)g * HD + d;
#pragma unroll
		for (int pn = 0; pn < F::NP; pn++) Vimg[(size_t)pn * 4 * HD + at] = pl.p[pn];
	}
	report_range<F>(rmax, range_flag);
}

// A wave's share of the copy of one 48 KB image into LDS: loads of 64 lanes x 16 bytes, each landing at
// (wave-uniform base) + 16 * lane; the NW waves of a workgroup take every NW-th kilobyte.
template <int NW, int KB>
__device__ __forceinline__ void copy_image_to_lds(const unsigned char *img, unsigned char *lds, int lane, int w) {
#pragma unroll
	for (int c = 0; c < KB / NW; c++)
		__builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(img + (size_t)(c * NW + w) * 1024 + 16 * lane),
		                                 (__attribute__((address_space(3))) void *)(lds + (c * NW + w) * 1024), 16, 0, 0);
}

// One piece (kilobyte c * NW + w) of the same copy, for callers that spread the pieces between other instructions: a
// wave issues in order, and a burst of copies from eight waves fills the queue they go into and holds what follows back.
template <int NW>
__device__ __forceinline__ void copy_image_piece(const unsigned char *img, unsigned char *lds, int lane, int w, int c) {
	__builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(img + (size_t)(c * NW + w) * 1024 + 16 * lane),
	                                 (__attribute__((address_space(3))) void *)(lds + (c * NW + w) * 1024), 16, 0, 0);
}

// LDS reads of the matrix operands as the instruction itself.  The compiler cannot tell which LDS bytes a load that
// writes straight into LDS will touch, so before every LDS read it can see it waits for ALL such loads in flight,
// which would serialise the copy of a later image with the work on the current one.  These reads it does not see;
// the wait for them is lds_wait(), which names the registers so that it stays between the reads and their use.
// Between such a read and its wait the compiler believes the register already holds the value: keep the two in one
// basic block.  Where control flow merges in between it may copy the "value" to another register before the data has
// arrived (seen with a read issued ahead of an if/else: a few lanes of the later-running waves got stale data).
// tests/test_isa_hazards.py checks the compiled kernels for any instruction that touches such a register early.
template <typename V, int OFF>
__device__ __forceinline__ V lds_read16(unsigned addr) {
	V r;
	asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
	return r;
}
__device__ __forceinline__ void lds_wait(PlanesT<FmtBf16x3> &a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.p[0]), "+v"(a.p[1]), "+v"(a.p[2])); }
__device__ __forceinline__ void lds_wait(PlanesT<FmtF16x2> &a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.p[0]), "+v"(a.p[1])); }
template <typename P>
__device__ __forceinline__ void lds_wait(P &a, P &b) {  // LDS reads return in order: both have arrived after these two
	lds_wait(a);
	lds_wait(b);
}
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f) {
	(f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
	static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
// byte offsets inside an image: Kb[plane][t][key][g], Vb[plane][g][dim], 16-byte elements
constexpr int KOFF_T = TK * 4 * 16, KOFF_HALF = 16 * 4 * 16, VOFF_DT = 16 * 16;
template <typename F, int T, int HF>
__device__ __forceinline__ PlanesT<F> read_k(unsigned kaddr) {
	PlanesT<F> f;
	f.p[0] = lds_read16<typename F::vec, T * KOFF_T + HF * KOFF_HALF>(kaddr);
	f.p[1] = lds_read16<typename F::vec, (int)PLANE_BYTES + T * KOFF_T + HF * KOFF_HALF>(kaddr);
	if constexpr (F::NP == 3) f.p[2] = lds_read16<typename F::vec, 2 * (int)PLANE_BYTES + T * KOFF_T + HF * KOFF_HALF>(kaddr);
	return f;
}
template <typename F, int DT>
__device__ __forceinline__ PlanesT<F> read_v(unsigned vaddr) {
	PlanesT<F> f;
	f.p[0] = lds_read16<typename F::vec, DT * VOFF_DT>(vaddr);
	f.p[1] = lds_read16<typename F::vec, (int)PLANE_BYTES + DT * VOFF_DT>(vaddr);
	if constexpr (F::NP == 3) f.p[2] = lds_read16<typename F::vec, 2 * (int)PLANE_BYTES + DT * VOFF_DT>(vaddr);
	return f;
}

// Same arguments and outputs as attn_prefill_split_kernel, except that K and V come as plane images (attn_planes_kernel).
// Every wave computes (head = wave % 4, query group = wave / 4) and issues its share of the image copies.
template <int QG, typename F>
__global__ __launch_bounds__(256 * QG) void attn_prefill_planes_kernel(float *o, const float *q, const unsigned char *planes, int S, int ldq,
                                                                     int ldo, int is_sw, int window, const int4 *items, float *part_o,
                                                                     float *part_ml, int *range_flag) {
	typedef PlanesT<F> Planes;
	extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // ring of three images
	constexpr size_t PLANE_IMG = plane_img<F>();
	constexpr int BQ = 16 * QG, NW = 4 * QG, IMG_KB = (int)(PLANE_IMG / 1024);
	constexpr int SHARE = IMG_KB / NW;  // loads per wave and image (12, 8, 6 or 4)
	unsigned rmax = 0u;

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, head = w & 3, qh = w >> 2, c = lane & 15, g = lane >> 4;
	int q0 = plain_query_tile(is_sw) * BQ, slot = -1;
	int4 item = int4{0, 0, 0, -1};
	if (items != nullptr) {
		item = items[blockIdx.x];
		q0 = item.x * BQ;
		slot = item.w;
	}
	// whole tiles only: a local layer's range starts at the tile that holds its first key (earlier keys are masked)
	int kb = (is_sw && q0 > window) ? ((q0 - window) / TK) * TK : 0;
	int ke = (q0 + BQ < S) ? q0 + BQ : S;  // exclusive
	if (items != nullptr) {
		kb = item.y * TK;
		ke = min(ke, item.z * TK);
	}
	const int ntiles = (ke - kb + TK - 1) / TK;
	// image i (K of tile i / 2 for even i, V for odd i) is the i-th 48 KB piece of the tile sequence; it lives in buffer i % 3
	const unsigned char *img0 = planes + (size_t)(kb / TK) * 2 * PLANE_IMG;
	const int nimg = 2 * ntiles;

	const int q0w = q0 + 16 * qh;  // first query of this wave's group
	const int qpos = q0w + c;
	const int qrow = qpos < S ? qpos : S - 1;
	const int klo = is_sw ? qpos - window : 0;

	// Q planes: qp[t] = dims 32t + 8g .. + 7 of query c, scaled by 1/sqrt(hd) (a power of two: commutes with the split)
	Planes qp[NT32];
	{
		const float *qsrc = q + (size_t)qrow * ldq + head * HD + 8 * g;
#pragma unroll
		for (int t = 0; t < NT32; t++) {
			const f32x4 x0 = *reinterpret_cast<const f32x4 *>(qsrc + 32 * t), x1 = *reinterpret_cast<const f32x4 *>(qsrc + 32 * t + 4);
			float x[8];
#pragma unroll
			for (int e = 0; e < 4; e++) {
				x[e] = x0[e] * F::QSCALE;
				x[4 + e] = x1[e] * F::QSCALE;
			}
			track_range<F>(rmax, x);
			qp[t] = split8<F>(x);
		}
	}
	f32x4 oacc[HD / 16];  // oacc[dt][i] = O[query 4 g + i][16 dt + c]
#pragma unroll
	for (int dt = 0; dt < HD / 16; dt++) oacc[dt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
	float m_run = -INFINITY, l_run = 0.0f;

	// The Q loads have been consumed above: from here on the only loads this wave has in flight are image copies, in
	// the order it issues them, so "at most SHARE outstanding" means "all but the youngest image's share have arrived".
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
	copy_image_to_lds<NW, IMG_KB>(img0, smem, lane, w);
	copy_image_to_lds<NW, IMG_KB>(img0 + PLANE_IMG, smem + PLANE_IMG, lane, w);
	wait_loads_in_flight<SHARE>();
	tg_lds_barrier();  // image 0 is complete

	const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;
	const unsigned k_lane = (unsigned)((c * 4 + g) * 16), v_lane = (unsigned)((g * HD + c) * 16);
	int kbuf = 0;  // buffer of image 2 * tile; the V image follows in the next one, and the one after is free
	for (int tile = 0; tile < ntiles; tile++) {
		const int vbuf = kbuf == 2 ? 0 : kbuf + 1, fbuf = vbuf == 2 ? 0 : vbuf + 1;
		const unsigned kaddr = lds0 + (unsigned)kbuf * (unsigned)PLANE_IMG + k_lane;
		const unsigned vaddr = lds0 + (unsigned)vbuf * (unsigned)PLANE_IMG + v_lane;
		// a tile that starts behind this group's last query holds none of its keys (the other group still needs it)
		const bool mine = kb + tile * TK <= q0w + 15;

		// ---- phase 2 * tile: scores.  Image 2 * tile + 2 (the next K) goes into the free buffer meanwhile ----
		const bool copy_k = 2 * tile + 2 < nimg, copy_v = 2 * tile + 3 < nimg;
		const unsigned char *next_k = img0 + (size_t)(2 * tile + 2) * PLANE_IMG, *next_v = img0 + (size_t)(2 * tile + 3) * PLANE_IMG;
		unsigned char *k_dst = smem + fbuf * PLANE_IMG, *v_dst = smem + kbuf * PLANE_IMG;
		f32x4 s0 = f32x4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;
		if (!mine && copy_k) copy_image_to_lds<NW, IMG_KB>(next_k, k_dst, lane, w);
		if (mine) {
			// the two groups of 16 keys; even and odd k steps in separate accumulators; the fragments of step t + 1 are
			// requested before the matrix instructions of step t
			f32x4 sa[2][2];
#pragma unroll
			for (int hf = 0; hf < 2; hf++) sa[hf][0] = sa[hf][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
			Planes ka = read_k<F, 0, 0>(kaddr), kc = read_k<F, 0, 1>(kaddr);
			static_for<NT32>([&](auto tc) {
				constexpr int t = decltype(tc)::value;
				lds_wait(ka, kc);
				const Planes a = ka, b = kc;
				if constexpr (t + 1 < NT32) {
					ka = read_k<F, t + 1, 0>(kaddr);
					kc = read_k<F, t + 1, 1>(kaddr);
				}
				sa[0][t & 1] = mfma_terms<F>(a, qp[t], sa[0][t & 1]);
				sa[1][t & 1] = mfma_terms<F>(b, qp[t], sa[1][t & 1]);
				// this wave's pieces of the next K image, one (two where there are more pieces than k steps) behind each of the
				// first k steps
				constexpr int PK = (SHARE + NT32 - 1) / NT32;
#pragma unroll
				for (int pc = t * PK; pc < (t + 1) * PK && pc < SHARE; pc++) {
					if (copy_k) copy_image_piece<NW>(next_k, k_dst, lane, w, pc);
				}
			});
			s0 = (sa[0][0] + sa[0][1]) * F::SSCALE;
			s1 = (sa[1][0] + sa[1][1]) * F::SSCALE;
		}
		// this wave's share of image 2 * tile + 1 (issued one phase ago) has arrived once at most the share just issued is outstanding
		if (2 * tile + 2 < nimg) {
			wait_loads_in_flight<SHARE>();
		} else {
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
		}
		tg_lds_barrier();  // the K image is released, the V image is complete

		// ---- phase 2 * tile + 1: softmax and P.V.  Image 2 * tile + 3 (the next V) goes into the buffer the K image has left ----
		if (!mine && copy_v) copy_image_to_lds<NW, IMG_KB>(next_v, v_dst, lane, w);
		if (mine) {
			Planes va = read_v<F, 0>(vaddr);  // in flight during the softmax
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
			const float m_new = fmaxf(m_run, tmax);
			const float m_ref = (m_new == -INFINITY) ? 0.0f : m_new;  // no valid key yet (see the fp32 kernel)
			const float alpha = softmax_exp(m_run - m_ref);
			float psum = 0.0f;
			float pv[8];  // the lane's 8 key slots: keys 4g + i, then 16 + 4g + i
#pragma unroll
			for (int i = 0; i < 4; i++) {
				pv[i] = softmax_exp(s0[i] - m_ref);
				pv[4 + i] = softmax_exp(s1[i] - m_ref);
				psum += pv[i] + pv[4 + i];
			}
			psum += tg_red_partner<16>(psum);
			psum += tg_red_partner<32>(psum);
			l_run = fmaf(l_run, alpha, psum);
			m_run = m_new;
			float ar[4];
#pragma unroll
			for (int i = 0; i < 4; i++) ar[i] = __shfl(alpha, 4 * g + i, 64);
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) {
#pragma unroll
				for (int i = 0; i < 4; i++) oacc[dt][i] *= ar[i];
			}
			// ---- O += P V ----
			const Planes pp = split8<F>(pv);
			static_for<HD / 16>([&](auto dc) {
				constexpr int dt = decltype(dc)::value;
				lds_wait(va);
				const Planes vf = va;
				if constexpr (dt + 1 < HD / 16) va = read_v<F, dt + 1>(vaddr);
				oacc[dt] = mfma_terms<F>(pp, vf, oacc[dt]);
				if constexpr (dt < SHARE) {  // the pieces of the next V image, likewise
					if (copy_v) copy_image_piece<NW>(next_v, v_dst, lane, w, dt);
				}
			});
		}
		if (2 * tile + 3 < nimg) {
			wait_loads_in_flight<SHARE>();
		} else {
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
		}
		tg_lds_barrier();  // the V image is released, the next K image is complete
		kbuf = fbuf;
	}

	report_range<F>(rmax, range_flag);
	if (slot >= 0) {
		float *po = part_o + (size_t)slot * BQ * NH * HD;
#pragma unroll
		for (int i = 0; i < 4; i++) {
			float *op = po + ((size_t)(16 * qh + 4 * g + i) * NH + head) * HD + c;
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) op[16 * dt] = oacc[dt][i];
		}
		if (g == 0) {
			float *pm = part_ml + (((size_t)slot * BQ + 16 * qh + c) * NH + head) * 2;
			pm[0] = m_run;
			pm[1] = l_run;
		}
		return;
	}
	float lr[4];  // 1 / l of the lane's four query rows: one division per row, then multiplications
#pragma unroll
	for (int i = 0; i < 4; i++) lr[i] = 1.0f / __shfl(l_run, 4 * g + i, 64);
#pragma unroll
	for (int i = 0; i < 4; i++) {
		const int qo = q0w + 4 * g + i;
		if (qo < S) {
			float *op = o + (size_t)qo * ldo + head * HD + c;
#pragma unroll
			for (int dt = 0; dt < HD / 16; dt++) op[16 * dt] = oacc[dt][i] * lr[i];
		}
	}
}

// ---- 32 query positions per matrix instruction ---------------------------------------------------------------------
// In the kernels above a wave multiplies 16 queries with every K and V fragment it reads from LDS: 64 KB of fragments
// per wave and key tile, with bank conflicts on the V reads in 13 % of the LDS cycles (SQ_LDS_BANK_CONFLICT).
// v_mfma_f32_32x32x16_f16 takes fragments of the same size (64 lanes x 16 bytes) and does twice the work with them:
// 32 keys x 32 queries x 16 dims.  A wave that owned 32 queries of a head alone would need 128 registers for its Q
// planes and 128 for its output rows; here two waves share a head and split the HEAD DIMENSION: wave (head, dh) keeps
// dims 128 dh .. + 127 of Q (64 registers) and of the output (64 registers), computes the scores' partial sums over
// its dims, and the two swap those partial sums through LDS (4 KB each way, next to the 16 + 16 KB of fragments a
// wave reads per tile, all of them conflict-free 1 KB rows).  A sum of two addends is the same in either order, so
// both hold the same scores, weights and running sums, and each multiplies the weights with its half of V.  fp16
// planes only (the bf16 form needs three planes of everything: 96 registers of Q).
// Measured against the 16-query kernel on the same box (kernel trace): causal layer of 16,384 tokens 1,920-1,955 ->
// 1,725-1,760 us, local layer 145-150 -> 137-142 us, local layer of 4,096 tokens 54-55 -> 50-52 us; the matrix cores
// are busy 45 % of the kernel's clocks (41 %).
//
// Layout of v_mfma_f32_32x32x16_f16: lane (r = lane % 32, h = lane / 32) holds A[r][8h .. 8h + 7], B[8h .. 8h + 7][r]
// and C[8j + 4h + i][r] in register 4j + i (j, i = 0..3).  Only the pairing of A and B slots matters, so
//   scores:  A = K, lane holds dims 16 ks + 8h .. + 7 of key r, B = Q likewise for query r:
//            C[8j + 4h + i][c] = S^T[key 8j + 4h + i][query c]: a lane holds 16 keys of query c = lane % 32;
//   output:  B = P^T, step s = 0, 1 takes the lane's registers 8s .. 8s + 7 (keys 16s + 4h + i, then 16s + 8 + 4h + i);
//            A = V^T with the same key order, lane r = dim: C[8j + 4h + i][c] = O^T[dim 32 dt + 8j + 4h + i][query c].
// The output is kept transposed so that a lane owns one query in both products: its running maximum, running sum and
// rescaling factor never leave the lane.
// Plane images for this kernel (attn_planes_wide_kernel), 16-byte elements, every fragment 1 KB in lane order:
//   Kw[plane][ks = 0..15][lane], Vw[plane][s = 0..1][dt = 0..7][lane].
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int WIDE_BQ = 32;                                        // query positions per workgroup
constexpr size_t WIDE_IMG = 2 * PLANE_BYTES;                       // an image of two fp16 planes, 32 KB
constexpr size_t WIDE_LDS = 4 * WIDE_IMG + 8 * 4096;               // ring of four images + the waves' partial scores: all 160 KB
static_assert(PLANE_BYTES == (HD / 16) * 64 * 16 && PLANE_BYTES == 2 * (HD / 32) * 64 * 16, "one plane of Kw and of Vw");

__global__ __launch_bounds__(PNT) void attn_planes_wide_kernel(unsigned char *planes, const float *k, const float *v, int S, int ldkv,
                                                              int *range_flag) {
	typedef FmtF16x2 F;
	typedef F::vec vec;
	const int tile = blockIdx.x, tid = threadIdx.x;
	vec *Kimg = reinterpret_cast<vec *>(planes + (size_t)tile * 2 * WIDE_IMG);
	vec *Vimg = reinterpret_cast<vec *>(planes + (size_t)tile * 2 * WIDE_IMG + WIDE_IMG);
	unsigned rmax = 0u;
	// one workgroup for the K image of a tile (blockIdx.y == 0), one for its V image: a prompt of 4096 tokens has only 128 tiles
	// K: unit = (key, piece of 8 dims): 32 consecutive threads read one key's 1 KB row
#pragma unroll
	for (int u = 0; u < 4; u++) {
		if (blockIdx.y != 0) break;
		const int unit = tid + PNT * u, piece = unit & 31, key = unit >> 5;
		const int j = tile * TK + key;
		float x[8];
		const float *src = k + (size_t)(j < S ? j : S - 1) * ldkv + 8 * piece;
		const f32x4 a = *reinterpret_cast<const f32x4 *>(src), b = *reinterpret_cast<const f32x4 *>(src + 4);
#pragma unroll
		for (int e = 0; e < 4; e++) {
			x[e] = j < S ? a[e] : 0.0f;
			x[4 + e] = j < S ? b[e] : 0.0f;
		}
		track_range<F>(rmax, x);
		const PlanesT<F> pl = split8<F>(x);
		const size_t at = (size_t)(piece >> 1) * 64 + (piece & 1) * 32 + key;  // ks = piece / 2, h = piece % 2
#pragma unroll
		for (int pn = 0; pn < 2; pn++) Kimg[pn * (PLANE_BYTES / 16) + at] = pl.p[pn];
	}
	// V: unit = (s, dt, lane): dim 32 dt + lane % 32, keys 16 s + 4 h + {0..3} and 16 s + 8 + 4 h + {0..3}
#pragma unroll
	for (int u = 0; u < 4; u++) {
		if (blockIdx.y != 1) break;
		const int unit = tid + PNT * u, lane = unit & 63, dt = (unit >> 6) & 7, s = unit >> 9;
		const int d = 32 * dt + (lane & 31), h = lane >> 5;
		float x[8];
#pragma unroll
		for (int sl = 0; sl < 8; sl++) {
			const int j = tile * TK + 16 * s + 8 * (sl >> 2) + 4 * h + (sl & 3);
			const float val = v[(size_t)(j < S ? j : S - 1) * ldkv + d];
			x[sl] = j < S ? val : 0.0f;
		}
		track_range<F>(rmax, x);
		const PlanesT<F> pl = split8<F>(x);
#pragma unroll
		for (int pn = 0; pn < 2; pn++) Vimg[pn * (PLANE_BYTES / 16) + unit] = pl.p[pn];
	}
	report_range<F>(rmax, range_flag);
}

__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
// acc += a . b: the three significant cross terms of two-plane operands, smallest first
__device__ __forceinline__ f32x16 mfma32_terms(const PlanesT<FmtF16x2> &a, const PlanesT<FmtF16x2> &b, f32x16 acc) {
	acc = mfma32(a.p[1], b.p[0], acc);
	acc = mfma32(a.p[0], b.p[1], acc);
	acc = mfma32(a.p[0], b.p[0], acc);
	return acc;
}
// fragment at a compile-time offset from a per-lane base: both planes
template <int OFF>
__device__ __forceinline__ PlanesT<FmtF16x2> read_wide(unsigned addr) {
	PlanesT<FmtF16x2> f;
	f.p[0] = lds_read16<f16x8, OFF>(addr);
	f.p[1] = lds_read16<f16x8, (int)PLANE_BYTES + OFF>(addr);
	return f;
}
template <int OFF>
__device__ __forceinline__ void lds_write16(unsigned addr, f32x4 v) {
	asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
// until at most N of this wave's LDS instructions are outstanding (they complete in order): names the fragment that
// must have arrived, so that the wait stays between its read and its use
template <int N>
__device__ __forceinline__ void lds_wait_but(PlanesT<FmtF16x2> &a) {
	asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a.p[0]), "+v"(a.p[1]) : "n"(N));
}
constexpr int WIDE_AHEAD = 2;  // fragments requested ahead of the one in use (3 or 4: no faster, more registers)
// The compiler inserts the wait states between a matrix instruction and a reader of its result only for readers it
// knows; an LDS store written as text is not one.  24 wait states (a 32x32x16 result needs 19 before an LDS or memory
// instruction may read it), tied to the registers so that they stay behind the matrix instructions.
__device__ __forceinline__ void mfma_result_to_asm(f32x16 &acc) { asm volatile("s_nop 15\n\ts_nop 7" : "+v"(acc)); }

// Same arguments and outputs as attn_prefill_planes_kernel<2, FmtF16x2>; plane images from attn_planes_wide_kernel.
// Wave w: head = w / 2, dims 128 (w % 2) .. + 127; lane: c = lane % 32 (query), h = lane / 32.
//
// Time line.  Per key tile a wave goes through three phases, with a workgroup barrier after each:
//   X1  its addend of the scores: 24 matrix instructions, 16 fragment reads, next to no vector work;
//   X2  the partner's addend, mask, softmax, the weights as fp16 planes: about 200 vector instructions, no matrix work;
//   Y   rescale the output (64 multiplies), then O^T += V^T P^T: 24 matrix instructions, 16 fragment reads.
// A SIMD holds wave s and wave s + 4 and overlaps one wave's matrix instructions with the other's vector instructions
// only if the two are in different phases (measured: 8 matrix instructions next to 64 multiplies take 360 clocks,
// against 256 and 280 alone), so waves 4-7 (heads 2, 3) run one step behind waves 0-3: the SIMD sees X1 | Y, X2 | X1,
// Y | X2.  A launch takes 3 ntiles + 1 steps.  Clocks between barriers, one workgroup of a long causal layer: 2,590,
// 1,870 and 1,600 for the three kinds of step (the matrix instructions alone need 1,536, 768 and 768); with all
// waves in one phase the kernel is 4 % slower.  Tried instead: the scores of tile t + 1 interleaved with the softmax
// of tile t inside a wave, two phases per tile (5,700 clocks per tile on a single workgroup instead of 6,060, no
// difference with all compute units busy); without the image copies a tile still takes 4,500 clocks.
// Images: K of tile t is image 2t, V is image 2t + 1, image i lives in buffer i % 4.  In step 3t everyone requests its
// share of K(t + 1), in step 3t + 1 of V(t + 1): the buffers they go to were last read in steps 3t - 2 and 3t, and
// the images have three and four steps to arrive.  A wave's loads complete in the order it issued them, so "at most
// n shares outstanding" is the test for the older ones.
__global__ __launch_bounds__(512) void attn_prefill_wide_kernel(float *o, const float *q, const unsigned char *planes, int S, int ldq, int ldo,
                                                                int is_sw, int window, const int4 *items, float *part_o, float *part_ml,
                                                                int *range_flag) {
	typedef FmtF16x2 F;
	typedef PlanesT<F> Planes;
	extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
	constexpr int BQ = WIDE_BQ, NW = 8, IMG_KB = (int)(WIDE_IMG / 1024), SHARE = IMG_KB / NW;  // 4 copy pieces per wave and image
	constexpr int NKS = HD / 32, NDT = HD / 64;  // k steps of a wave's score product (8), output tiles of 32 dims it owns (4)
	constexpr float EXP_SCALE = F::SSCALE * 1.44269504088896341f;  // 1/sqrt(head_dim) and log2(e) in one factor
	static_assert(F::QSCALE == 1.0f, "the scores are scaled, not q");
	unsigned rmax = 0u;

	// the wave index as a scalar: what depends on it alone (roles, LDS regions, which copies a phase issues) then lives in scalar registers
	const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int head = w >> 1, dh = w & 1, late = w >> 2, c = lane & 31, h = lane >> 5;
	int q0 = plain_query_tile(is_sw) * BQ, slot = -1;
	int4 item = int4{0, 0, 0, -1};
	if (items != nullptr) {
		item = items[blockIdx.x];
		q0 = item.x * BQ;
		slot = item.w;
	}
	int kb = (is_sw && q0 > window) ? ((q0 - window) / TK) * TK : 0;
	int ke = (q0 + BQ < S) ? q0 + BQ : S;  // exclusive
	if (items != nullptr) {
		kb = item.y * TK;
		ke = min(ke, item.z * TK);
	}
	const int ntiles = (ke - kb + TK - 1) / TK;
	const unsigned char *img0 = planes + (size_t)(kb / TK) * 2 * WIDE_IMG;
	const int nimg = 2 * ntiles;

	const int qpos = q0 + c;
	const int qrow = qpos < S ? qpos : S - 1;
	const int klo = is_sw ? qpos - window : 0;

	// Q planes: qp[ks] = dims 128 dh + 16 ks + 8 h .. + 7 of query c
	Planes qp[NKS];
	{
		const float *qsrc = q + (size_t)qrow * ldq + head * HD + 128 * dh + 8 * h;
#pragma unroll
		for (int ks = 0; ks < NKS; ks++) {
			const f32x4 x0 = *reinterpret_cast<const f32x4 *>(qsrc + 16 * ks), x1 = *reinterpret_cast<const f32x4 *>(qsrc + 16 * ks + 4);
			float x[8];
#pragma unroll
			for (int e = 0; e < 4; e++) {
				x[e] = x0[e];
				x[4 + e] = x1[e];
			}
			track_range<F>(rmax, x);
			qp[ks] = split8<F>(x);
		}
	}
	// The output is kept transposed, oacc[dt][4j + i] = O[query c][128 dh + 32 dt + 8j + 4h + i]: a lane then owns one
	// query in the scores and in the output alike, and the running maximum, the running sum and the rescaling factor
	// of that query never leave the lane.
	f32x16 oacc[NDT], mine;
#pragma unroll
	for (int e = 0; e < 16; e++) mine[e] = 0.0f;
#pragma unroll
	for (int dt = 0; dt < NDT; dt++) oacc[dt] = mine;
	float m_run = -INFINITY, l_run = 0.0f, alpha = 1.0f;  // the maximum in units of the unscaled scores
	Planes pp[2];                                          // the weights of a tile, from its X2 to its Y

	// from here on the only loads this wave has in flight are image copies, in the order it issues them
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
	copy_image_to_lds<NW, IMG_KB>(img0, smem, lane, w);
	copy_image_to_lds<NW, IMG_KB>(img0 + WIDE_IMG, smem + WIDE_IMG, lane, w);
	wait_loads_in_flight<SHARE>();
	tg_lds_barrier();  // image 0 is complete

	const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;
	const unsigned k_lane = (unsigned)(dh * NKS * 1024 + lane * 16), v_lane = (unsigned)(dh * NDT * 1024 + lane * 16);
	const unsigned my_part = lds0 + 4u * (unsigned)WIDE_IMG + (unsigned)(w * 4096 + lane * 16);
	const unsigned their_part = lds0 + 4u * (unsigned)WIDE_IMG + (unsigned)((w ^ 1) * 4096 + lane * 16);
	// end of a step: all but the youngest `shares` of this wave's copies have arrived; the barrier completes the images
	// and addends written by the other waves and releases what this step read
	auto end_step = [&](int shares) {
		if (shares == 2) {
			wait_loads_in_flight<2 * SHARE>();
		} else if (shares == 1) {
			wait_loads_in_flight<SHARE>();
		} else if (shares == 0) {
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
		}
		tg_lds_barrier();
	};
	if (late) {  // step 0 of the late waves: only their share of K(1)
		if (2 < nimg) copy_image_to_lds<NW, IMG_KB>(img0 + 2 * WIDE_IMG, smem + 2 * WIDE_IMG, lane, w);
		end_step(-1);
	}
	for (int tile = 0; tile < ntiles; tile++) {
		const bool more = tile + 1 < ntiles;  // images 2 tile + 2 and 2 tile + 3 exist
		{
			// ---- X1: this wave's addend of the scores, S^T = K Q^T over its 128 dims.  The early waves are in step 3 tile and
			// request K(tile + 1), the late ones in step 3 tile + 1 and request V(tile + 1). ----
			const int ci = 2 * tile + 2 + late;
			const unsigned char *src = img0 + (size_t)ci * WIDE_IMG;
			unsigned char *dst = smem + (size_t)(ci & 3) * WIDE_IMG;
			const unsigned kaddr = lds0 + (unsigned)((2 * tile) & 3) * (unsigned)WIDE_IMG + k_lane;
#pragma unroll
			for (int e = 0; e < 16; e++) mine[e] = 0.0f;
			Planes kf[WIDE_AHEAD];
			static_for<WIDE_AHEAD>([&](auto tc) {
				constexpr int t = decltype(tc)::value;
				kf[t] = read_wide<t * 1024>(kaddr);
			});
			static_for<NKS>([&](auto tc) {
				constexpr int t = decltype(tc)::value;
				constexpr int later = (NKS - 1 - t < WIDE_AHEAD - 1) ? NKS - 1 - t : WIDE_AHEAD - 1;  // fragments requested after this one
				lds_wait_but<2 * later>(kf[t % WIDE_AHEAD]);
				mine = mfma32_terms(kf[t % WIDE_AHEAD], qp[t], mine);
				if constexpr (t + WIDE_AHEAD < NKS) kf[t % WIDE_AHEAD] = read_wide<(t + WIDE_AHEAD) * 1024>(kaddr);
				if constexpr (t < SHARE) {
					if (more) copy_image_piece<NW>(src, dst, lane, w, t);
				}
			});
			mfma_result_to_asm(mine);
			static_for<4>([&](auto jc) {
				constexpr int j = decltype(jc)::value;
				lds_write16<j * 1024>(my_part, f32x4{mine[4 * j], mine[4 * j + 1], mine[4 * j + 2], mine[4 * j + 3]});
			});
			// late waves, step 3 tile + 1: V(tile) must be complete for the early waves' Y; K(tile + 1) and V(tile + 1) are younger
			end_step(late ? (more ? 2 : 0) : -1);
		}
		{
			// ---- X2: softmax.  The early waves (step 3 tile + 1) request V(tile + 1) here. ----
			if (!late && more) copy_image_to_lds<NW, IMG_KB>(img0 + (size_t)(2 * tile + 3) * WIDE_IMG, smem + (size_t)((2 * tile + 3) & 3) * WIDE_IMG, lane, w);
			const int t0 = kb + tile * TK;  // first key of the tile
			f32x4 th[4];
			static_for<4>([&](auto jc) {
				constexpr int j = decltype(jc)::value;
				th[j] = lds_read16<f32x4, j * 1024>(their_part);
			});
			asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(th[0]), "+v"(th[1]), "+v"(th[2]), "+v"(th[3]));
			float sv[16];  // sv[4j + i]: key t0 + 8j + 4h + i of query c; a sum of two addends is the same in either order
#pragma unroll
			for (int j = 0; j < 4; j++)
#pragma unroll
				for (int i = 0; i < 4; i++) sv[4 * j + i] = mine[4 * j + i] + th[j][i];
			// only the tiles on the diagonal and at the far end of a window hold keys that some query must not see
			if (t0 + TK - 1 > q0 || (is_sw && t0 < q0 + BQ - 1 - window)) {
#pragma unroll
				for (int j = 0; j < 4; j++)
#pragma unroll
					for (int i = 0; i < 4; i++) {
						const int key = t0 + 8 * j + 4 * h + i;
						if (key > qpos || key < klo) sv[4 * j + i] = -INFINITY;
					}
			}
			float tmax = sv[0];
#pragma unroll
			for (int e = 1; e < 16; e++) tmax = fmaxf(tmax, sv[e]);
			tmax = fmaxf(tmax, tg_red_partner<32>(tmax));
			const float m_new = fmaxf(m_run, tmax);
			const float m_ref = (m_new == -INFINITY) ? 0.0f : m_new;  // no valid key yet
			alpha = __builtin_amdgcn_exp2f((m_run - m_ref) * EXP_SCALE);
			float psum = 0.0f;
#pragma unroll
			for (int e = 0; e < 16; e++) {
				sv[e] = __builtin_amdgcn_exp2f((sv[e] - m_ref) * EXP_SCALE);
				psum += sv[e];
			}
			psum += tg_red_partner<32>(psum);
			l_run = fmaf(l_run, alpha, psum);
			m_run = m_new;
			pp[0] = split8<F>(sv);
			pp[1] = split8<F>(sv + 8);
			// early waves, step 3 tile + 1: as above; late waves, step 3 tile + 2: K(tile + 1) must be complete, V(tile + 1) is younger
			end_step(more ? (late ? 1 : 2) : 0);
		}
		{
			// ---- Y: O^T = alpha O^T + V^T P^T.  The late waves (step 3 tile + 3) request K(tile + 2) here. ----
			const int ci = 2 * tile + 4;
			const bool copy = late && ci < nimg;
			const unsigned char *src = img0 + (size_t)ci * WIDE_IMG;
			unsigned char *dst = smem + (size_t)(ci & 3) * WIDE_IMG;
			const unsigned vaddr = lds0 + (unsigned)((2 * tile + 1) & 3) * (unsigned)WIDE_IMG + v_lane;
			Planes vf[WIDE_AHEAD];
			static_for<WIDE_AHEAD>([&](auto tc) {
				constexpr int t = decltype(tc)::value;
				vf[t] = read_wide<(t / NDT) * 8192 + (t % NDT) * 1024>(vaddr);
			});
#pragma unroll
			for (int dt = 0; dt < NDT; dt++) oacc[dt] = oacc[dt] * alpha;
			static_for<2 * NDT>([&](auto sc) {
				constexpr int st = decltype(sc)::value, s = st / NDT, dt = st % NDT;
				constexpr int later = (2 * NDT - 1 - st < WIDE_AHEAD - 1) ? 2 * NDT - 1 - st : WIDE_AHEAD - 1;
				constexpr int nx = st + WIDE_AHEAD;
				lds_wait_but<2 * later>(vf[st % WIDE_AHEAD]);
				oacc[dt] = mfma32_terms(vf[st % WIDE_AHEAD], pp[s], oacc[dt]);
				if constexpr (nx < 2 * NDT) vf[st % WIDE_AHEAD] = read_wide<(nx / NDT) * 8192 + (nx % NDT) * 1024>(vaddr);
				if constexpr (st < SHARE) {
					if (copy) copy_image_piece<NW>(src, dst, lane, w, st);
				}
			});
			// early waves, step 3 tile + 2: K(tile + 1) must be complete, V(tile + 1) is younger
			end_step(late ? -1 : (more ? 1 : 0));
		}
	}
	if (!late) end_step(-1);  // the last step of the early waves

	report_range<F>(rmax, range_flag);
	if (slot >= 0) {
		float *po = part_o + (((size_t)slot * BQ + c) * NH + head) * HD + 128 * dh + 4 * h;
#pragma unroll
		for (int dt = 0; dt < NDT; dt++)
#pragma unroll
			for (int j = 0; j < 4; j++)
				*reinterpret_cast<f32x4 *>(po + 32 * dt + 8 * j) = f32x4{oacc[dt][4 * j], oacc[dt][4 * j + 1], oacc[dt][4 * j + 2], oacc[dt][4 * j + 3]};
		if (h == 0 && dh == 0) {
			float *pm = part_ml + (((size_t)slot * BQ + c) * NH + head) * 2;
			pm[0] = m_run * F::SSCALE;  // in units of the scaled scores, like the other kernels
			pm[1] = l_run;
		}
		return;
	}
	if (qpos < S) {
		const float l_inv = 1.0f / l_run;  // one division per query row, then multiplications
		float *op = o + (size_t)qpos * ldo + head * HD + 128 * dh + 4 * h;
#pragma unroll
		for (int dt = 0; dt < NDT; dt++)
#pragma unroll
			for (int j = 0; j < 4; j++)
				*reinterpret_cast<f32x4 *>(op + 32 * dt + 8 * j) = f32x4{oacc[dt][4 * j] * l_inv, oacc[dt][4 * j + 1] * l_inv, oacc[dt][4 * j + 2] * l_inv, oacc[dt][4 * j + 3] * l_inv};
	}
}

// One workgroup per query position of a split query tile; wave = head, lane = 4 consecutive dims.
// split[b] = {query tile, first slot, number of chunks}.
__global__ __launch_bounds__(PNT) void attn_prefill_merge_kernel(float *o, int S, int ldo, const int4 *split, const float *part_o,
                                                                const float *part_ml, int tq) {
	const int4 sp = split[blockIdx.x / tq];
	const int qi = blockIdx.x % tq, qpos = sp.x * tq + qi;
	if (qpos >= S) return;
	const int lane = threadIdx.x & 63, head = threadIdx.x >> 6;
	float M = -INFINITY;
	for (int ch = 0; ch < sp.z; ch++) M = fmaxf(M, part_ml[(((size_t)(sp.y + ch) * tq + qi) * NH + head) * 2]);
	float L = 0.0f;
	f32x4 acc = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
	for (int ch = 0; ch < sp.z; ch++) {
		const size_t row = ((size_t)(sp.y + ch) * tq + qi) * NH + head;
		const float wgt = expf(part_ml[row * 2] - M);
		L = fmaf(part_ml[row * 2 + 1], wgt, L);
		const f32x4 x = *reinterpret_cast<const f32x4 *>(part_o + row * HD + 4 * lane);
		acc += x * wgt;
	}
	const f32x4 res = acc * (1.0f / L);
	*reinterpret_cast<f32x4 *>(o + (size_t)qpos * ldo + head * HD + 4 * lane) = res;
}

// Attention output -> operand of the output projection in one launch: per row, the chunks of a split query tile are
// merged (as attn_prefill_merge_kernel does), the row maximum over all four heads gives the power-of-two row factor,
// and the row is written as digit planes.  Two rows per workgroup, a thread = 8 consecutive dims of a row (two waves
// per row: heads 0-1 and 2-3).  Rows of whole query tiles are read from o, where their workgroup wrote them.
__global__ __launch_bounds__(PNT) void attn_prefill_finish_kernel(const float *o, int S, int ldo, const int2 *tiles, const float *part_o,
                                                                 const float *part_ml, int tq, int8_t *apack, float *rowfac, int Mpad) {
	__shared__ float wmax[PNT / 64];
	const int tid = threadIdx.x, t = tid & 127, half = tid >> 7;
	const int row = 2 * (int)blockIdx.x + half, qrow = row < S ? row : S - 1;  // the odd last row is computed twice, written once
	const int head = t >> 5, d0 = 8 * (t & 31);
	int2 ti = int2{-1, 1};
	if (tiles != nullptr) ti = tiles[qrow / tq];
	float v[8];
	if (ti.x < 0) {
		const float *src = o + (size_t)qrow * ldo + head * HD + d0;
		const f32x4 a = *reinterpret_cast<const f32x4 *>(src), b = *reinterpret_cast<const f32x4 *>(src + 4);
#pragma unroll
		for (int e = 0; e < 4; e++) {
			v[e] = a[e];
			v[4 + e] = b[e];
		}
	} else {
		const int qi = qrow % tq;
		float M = -INFINITY;
		for (int ch = 0; ch < ti.y; ch++) M = fmaxf(M, part_ml[(((size_t)(ti.x + ch) * tq + qi) * NH + head) * 2]);
		float L = 0.0f;
		f32x4 a = f32x4{0.0f, 0.0f, 0.0f, 0.0f}, b = a;
		for (int ch = 0; ch < ti.y; ch++) {
			const size_t r = ((size_t)(ti.x + ch) * tq + qi) * NH + head;
			const float wgt = expf(part_ml[r * 2] - M);
			L = fmaf(part_ml[r * 2 + 1], wgt, L);
			a += *reinterpret_cast<const f32x4 *>(part_o + r * HD + d0) * wgt;
			b += *reinterpret_cast<const f32x4 *>(part_o + r * HD + d0 + 4) * wgt;
		}
		const float Linv = 1.0f / L;
		a = a * Linv;
		b = b * Linv;
#pragma unroll
		for (int e = 0; e < 4; e++) {
			v[e] = a[e];
			v[4 + e] = b[e];
		}
	}
	float amax = 0.0f;
#pragma unroll
	for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[e]));
	amax = tg_wave_max(amax);
	if ((tid & 63) == 0) wmax[tid >> 6] = amax;
	__syncthreads();
	amax = fmaxf(wmax[2 * half], wmax[2 * half + 1]);
	if (row >= S) return;
	float mul, inv;
	tg_row_factors(amax, mul, inv);
	if (t == 0) {
		rowfac[row] = mul;
		rowfac[Mpad + row] = inv;
	}
	uint2 pl[3];
	tg_quant8(v, mul, pl);
	const int k0 = head * HD + d0;
	uint2 *dst = reinterpret_cast<uint2 *>(tg_plane_dst(apack, row, k0 & ~15, NH * HD)) + ((k0 >> 3) & 1);
#pragma unroll
	for (int p = 0; p < 3; p++) dst[p * 128] = pl[p];  // planes are 64 pieces of 16 bytes apart
}

}  // namespace

// split-precision path: K/V split into plane images once per layer and copied straight into LDS (1: for prompts of
// TG_ATTN_PLANES_MIN_TOKENS tokens or more, where it pays: measured break-even at ~1500 tokens, -8 % prefill time at
// 2000; 2: always), or every workgroup splits what it stages (0)
int g_attn_prefill_planes = 1;
constexpr int TG_ATTN_PLANES_MIN_TOKENS = 2048;
size_t tg_attn_prefill_planes_bytes(int S) { return (size_t)((S + TK - 1) / TK) * 2 * plane_img<FmtBf16x3>(); }  // the larger format
// split path: 1 (default) = two fp16 planes, three products, on 32x32x16 matrix instructions where the plane images
// and 32-query workgroups are in use; 2 = the same planes on 16x16x32 instructions throughout; 0 = three bf16 planes,
// six products
int g_attn_prefill_f16 = 1;

int g_attn_prefill_split = 1;  // 0: fp32 matrix path; 1 (default): split-precision matrix path (two fp16 or three bf16 planes); 2: the same, always with 32-query workgroups

// Work list of a layer of S tokens, for tg_launch_attn_prefill: causal (window < 0) or local (a query sees the
// `window` keys before it and itself).  Returns false when no query tile needs splitting (then the plain launch is
// already balanced).  items: one int4 per workgroup {query tile, first key tile, end key tile, slot or -1},
// heaviest first; split: one int4 per split query tile; nslots: chunks that go through scratch.
// 32 query positions per workgroup (two waves per SIMD, a K/V tile fetched once for twice the queries) once that leaves
// a workgroup for every eighth compute unit; the work lists cut the key ranges so that the other units get items too.
// Measured crossover on 256 compute units, whole prefills: 600 tokens +1.6 %, 1000 tokens -2 %, 1536 -4.6 %, 2047 -5.5 %.
int tg_attn_prefill_query_tile(int S, int n_cu) {
	return (g_attn_prefill_split == 2 || (g_attn_prefill_split == 1 && (S + 31) / 32 >= n_cu / 8)) ? 32 : TQ;
}

bool tg_attn_prefill_plan(int S, int n_cu, int tq, int window, std::vector<int4> &items, std::vector<int4> &split, int &nslots) {
	const int nq = (S + tq - 1) / tq;
	auto first_tile = [&](int qt) { return (window >= 0 && qt * tq > window) ? (qt * tq - window) / TK : 0; };
	auto end_tile = [&](int qt) { return (std::min(qt * tq + tq, S) + TK - 1) / TK; };
	long total = 0;
	int longest = 1;
	for (int qt = 0; qt < nq; qt++) {
		total += end_tile(qt) - first_tile(qt);
		longest = std::max(longest, end_tile(qt) - first_tile(qt));
	}
	// Long prompts (causal): to begin with about 8 items per compute unit, and never chunks below 16 key tiles (512 keys);
	// the play-through below may choose another length.
	// Prompts with fewer query tiles than compute units: a workgroup's time is its chain of key tiles (one wave per
	// SIMD, nothing overlaps), so the chains are cut as short as the number of compute units allows: the smallest
	// chunk that still gives at most one item per unit.  Local layers of long prompts are balanced as they are.
	int chunk = window < 0 ? (int)std::max<long>(16, total / ((long)n_cu * 8)) : longest;
	bool one_round = false;
	for (int c = 1; c < chunk; c++) {
		long n = 0;
		for (int qt = 0; qt < nq; qt++) n += (end_tile(qt) - first_tile(qt) + c - 1) / c;
		if (n <= n_cu) {
			chunk = c;
			one_round = true;
			break;
		}
	}
	// Causal layers whose items take several rounds: the chunk length decides how many items there are and how the
	// rounds end.  With 16 key tiles a layer of 4096 tokens has 527 items for 256 compute units, and the 15 that start
	// last, when the first units have done their two, add 20 % (148-154 us measured, 151 by the model below; 17 key
	// tiles give 492 items and 124 us); at 8192 tokens and more, 8 items per unit pay the start-up of an item more
	// often than the balance needs.  Candidates: the rule above, and the shortest chunks that give at most 2, 3 and 4
	// items per unit.  Their lists are played through on the host: an item costs its key tiles plus 4 (start-up until
	// the first image is in LDS, 7 us, and storing its partial result, 5 us, against 2.95 us per key tile, all measured
	// inside the kernel), the units take the items in list order.  0.05-0.6 ms on the host for 4096-32768 tokens, once
	// per prompt length and process.
	if (window < 0 && !one_round) {
		static std::map<std::tuple<int, int, int>, int> chosen;
		const auto key = std::make_tuple(S, n_cu, tq);
		const auto hit = chosen.find(key);
		if (hit != chosen.end()) {
			chunk = hit->second;
		} else {
			auto chunks_of = [&](int nt, int c) {
				const int nc = (nt + c - 1) / c;
				return (nc > 1 && nt - (nc - 1) * c < (c + 1) / 2) ? nc - 1 : nc;
			};
			auto n_items = [&](int c) {
				long n = 0;
				for (int qt = 0; qt < nq; qt++) n += chunks_of(end_tile(qt) - first_tile(qt), c);
				return n;
			};
			std::vector<int> count((size_t)std::max(longest, chunk) + 1);  // items by length (a chunk may be longer than any key range)
			auto span = [&](int c) {
				std::fill(count.begin(), count.end(), 0);
				long n = 0;
				for (int qt = 0; qt < nq; qt++) {
					const int nt = end_tile(qt) - first_tile(qt), nc = chunks_of(nt, c);
					count[(size_t)c] += nc - 1;
					count[(size_t)(nt - (nc - 1) * c)]++;
					n += nc;
				}
				std::priority_queue<long, std::vector<long>, std::greater<long>> free_at;
				for (int i = 0; i < n_cu; i++) free_at.push(0);
				long end = 0;
				for (int l = (int)count.size() - 1; l >= 1; l--)
					for (int k = 0; k < count[(size_t)l]; k++) {
						const long t = free_at.top() + 4 + l;
						free_at.pop();
						free_at.push(t);
						end = std::max(end, t);
					}
				return end + n / 100;  // the finishing launch reads every partial result
			};
			long best = span(chunk);
			int best_c = chunk;
			for (int per_unit = 2; per_unit <= 4; per_unit++) {
				int lo = 6, hi = longest;  // the shortest chunk with at most per_unit items per unit (the count falls with the length)
				while (lo < hi) {
					const int mid = (lo + hi) / 2;
					if (n_items(mid) <= (long)per_unit * n_cu) hi = mid;
					else lo = mid + 1;
				}
				if (lo == best_c) continue;
				const long sp = span(lo);
				if (sp < best) {
					best = sp;
					best_c = lo;
				}
			}
			chunk = best_c;
			chosen[key] = chunk;
		}
	}
	items.clear();
	split.clear();
	nslots = 0;
	// Chunk boundaries are the same for every query tile (multiples of `chunk` key tiles, counted from the query tile's
	// first key tile for local layers, whose windows all start differently): the workgroups that run next to each
	// other then walk the same keys at the same time and find each other's K/V tiles in their XCD's L2.  Causal layers: a
	// last chunk of less than half a chunk is merged into the one before it.
	for (int qt = 0; qt < nq; qt++) {
		const int t0 = first_tile(qt), nt = end_tile(qt) - t0;
		int nc = (nt + chunk - 1) / chunk;
		// Local layers have at most one item per compute unit, so the longest item is the launch: a short last chunk is
		// evened out with the others instead (9 + 4 key tiles -> 7 + 6; merged into 13, such items took 45 us next to
		// 36 us for the 9-tile items of all the later query tiles).
		const bool even = window >= 0;
		if (!even && nc > 1 && nt - (nc - 1) * chunk < (chunk + 1) / 2) nc--;
		const int each = even ? (nt + nc - 1) / nc : chunk;
		if (nc == 1) {
			items.push_back(int4{qt, t0, t0 + nt, -1});
			continue;
		}
		split.push_back(int4{qt, nslots, nc, 0});
		for (int ch = 0; ch < nc; ch++) {
			const int tb = t0 + ch * each, te = ch + 1 == nc ? t0 + nt : tb + each;
			items.push_back(int4{qt, tb, te, nslots++});
		}
	}
	if (split.empty()) return false;
	// Workgroups go to the 8 XCDs round-robin in list order, and each XCD works through its share in order: sorted by
	// key range first, the 32 workgroups an XCD runs at any time share a key range (causal layers) or neighbouring
	// windows (local layers).  Longest items first (the full chunks all have one length), then by key range.
	auto by_keys = [](const int4 &a, const int4 &b) {
		if (a.z - a.y != b.z - b.y) return a.z - a.y > b.z - b.y;
		if (a.y != b.y) return a.y < b.y;
		return a.x < b.x;
	};
	std::stable_sort(items.begin(), items.end(), by_keys);
	return true;
}
size_t tg_attn_prefill_part_floats(int nslots, int tq) { return (size_t)nslots * tq * NH * HD; }
size_t tg_attn_prefill_ml_floats(int nslots, int tq) { return (size_t)nslots * tq * NH * 2; }

namespace {
// The launches of the split path in one operand format: plane images + copying kernel, or the staging kernel.
template <typename F>
void launch_split(dim3 grid, int tq, bool planes, float *o, const float *q, const float *k, const float *v, int S, int ldq, int ldkv, int ldo,
                  int is_sw, int window, const int4 *items, float *po, float *pml, void *planes_ws, int *range_flag, hipStream_t s) {
	static bool lds_set = false;
	constexpr size_t ring = 3 * plane_img<F>(), staged = split_lds_bytes<F>();
	if (!lds_set) {  // more than 64 KB of dynamic LDS needs the opt-in
		(void)hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_planes_kernel<1, F>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ring);
		(void)hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_planes_kernel<2, F>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ring);
		(void)hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_split_kernel<1, F>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)staged);
		(void)hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_split_kernel<2, F>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)staged);
		lds_set = true;
	}
	if constexpr (std::is_same<F, FmtF16x2>::value) {
		if (planes && tq == WIDE_BQ && g_attn_prefill_f16 == 1) {  // 32 queries per matrix instruction
			static bool wide_set = false;
			if (!wide_set) {
				(void)hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_wide_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)WIDE_LDS);
				wide_set = true;
			}
			unsigned char *pw = (unsigned char *)planes_ws;
			hipLaunchKernelGGL(attn_planes_wide_kernel, dim3((unsigned)((S + TK - 1) / TK), 2), dim3(PNT), 0, s, pw, k, v, S, ldkv, range_flag);
			hipLaunchKernelGGL(attn_prefill_wide_kernel, grid, dim3(512), WIDE_LDS, s, o, q, pw, S, ldq, ldo, is_sw, window, items, po, pml, range_flag);
			return;
		}
	}
	if (planes) {
		unsigned char *pw = (unsigned char *)planes_ws;
		hipLaunchKernelGGL(attn_planes_kernel<F>, dim3((unsigned)((S + TK - 1) / TK)), dim3(PNT), 0, s, pw, k, v, S, ldkv, range_flag);
		if (tq == 32)
			hipLaunchKernelGGL((attn_prefill_planes_kernel<2, F>), grid, dim3(512), ring, s, o, q, pw, S, ldq, ldo, is_sw, window, items, po, pml,
			                   range_flag);
		else
			hipLaunchKernelGGL((attn_prefill_planes_kernel<1, F>), grid, dim3(256), ring, s, o, q, pw, S, ldq, ldo, is_sw, window, items, po, pml,
			                   range_flag);
	} else if (tq == 32) {
		hipLaunchKernelGGL((attn_prefill_split_kernel<2, F>), grid, dim3(512), staged, s, o, q, k, v, S, ldq, ldkv, ldo, is_sw, window, items, po,
		                   pml, range_flag);
	} else {
		hipLaunchKernelGGL((attn_prefill_split_kernel<1, F>), grid, dim3(256), staged, s, o, q, k, v, S, ldq, ldkv, ldo, is_sw, window, items, po,
		                   pml, range_flag);
	}
}
}  // namespace

// q/k/v: rows of S tokens (q already normalised and rotated, ldq floats apart; k, v ldkv apart); o [S][ldo]
void tg_launch_attn_prefill(float *o, const float *q, const float *k, const float *v, int S, int n_head, int hd, int ldq, int ldkv,
                            int ldo, int is_sw, int window, const TgAttnPrefillPlan *plan, int n_cu, hipStream_t s,
                            bool finish_later, void *planes_ws, int *range_flag) {
	(void)n_head;
	(void)hd;
	const bool whole = plan == nullptr;  // the caller passes the work list that fits the layer kind, or none
	const int tq = tg_attn_prefill_query_tile(S, n_cu);  // a plan must have been built for this tile size
	const dim3 grid(whole ? (unsigned)((S + tq - 1) / tq) : (unsigned)plan->nitems);
	const int4 *items = whole ? nullptr : plan->items;
	float *po = whole ? nullptr : plan->part_o, *pml = whole ? nullptr : plan->part_ml;
	const bool planes = g_attn_prefill_split && planes_ws != nullptr &&
	                    (g_attn_prefill_planes == 2 || (g_attn_prefill_planes == 1 && S >= TG_ATTN_PLANES_MIN_TOKENS));
	if (!g_attn_prefill_split)
		hipLaunchKernelGGL(attn_prefill_mfma_kernel, grid, dim3(PNT), 0, s, o, q, k, v, S, ldq, ldkv, ldo, is_sw, window, items,
		                   po, pml);
	else if (g_attn_prefill_f16)
		launch_split<FmtF16x2>(grid, tq, planes, o, q, k, v, S, ldq, ldkv, ldo, is_sw, window, items, po, pml, planes_ws, range_flag, s);
	else
		launch_split<FmtBf16x3>(grid, tq, planes, o, q, k, v, S, ldq, ldkv, ldo, is_sw, window, items, po, pml, planes_ws, range_flag, s);
	if (whole || finish_later) return;
	hipLaunchKernelGGL(attn_prefill_merge_kernel, dim3((unsigned)(plan->nsplit * tq)), dim3(PNT), 0, s, o, S, ldo, plan->split,
	                   plan->part_o, plan->part_ml, tq);
}

void tg_launch_attn_prefill_finish(const float *o, int S, int ldo, const TgAttnPrefillPlan *plan, int n_cu, int8_t *apack, float *rowfac,
                                   hipStream_t s) {
	const int tq = tg_attn_prefill_query_tile(S, n_cu);
	hipLaunchKernelGGL(attn_prefill_finish_kernel, dim3((unsigned)((S + 1) / 2)), dim3(PNT), 0, s, o, S, ldo,
	                   plan ? plan->tiles : nullptr, plan ? plan->part_o : nullptr, plan ? plan->part_ml : nullptr, tq, apack, rowfac,
	                   (int)tg_gemm_mfma_rows(S));
}

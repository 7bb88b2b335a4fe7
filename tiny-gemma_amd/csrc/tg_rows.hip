// Row-wise prefill kernels (one workgroup per prompt position) and the prefill GEMM.
//
//   embed_rows : ops::embedding_prefill (ops.hpp:529-571)
//   norm_rows  : ops::rmsnorm on [S][dim] (ops.hpp:126-222), optionally preceded by the
//                "post-norm the block output, add the residual" step of modules.hpp:130-132, 199-201
//   gemm       : gemm::launch_qgemm (linalg.hpp:210-308): C = (A . W) * scales, C overwritten.
//                This version keeps the reference's arithmetic exactly — one fused multiply-add
//                chain per output element over k = 0..K-1 in fp32 (linalg.hpp:215-235) — on the
//                vector ALUs, reading the packed int8 tiles directly.

#include "tg_internal.h"

namespace {

constexpr int RNT = 256;

__device__ __forceinline__ float wsum(float v) { return tg_wave_sum(v); }

__device__ __forceinline__ float bsum(float v, float *sred) {
	v = wsum(v);
	__syncthreads();
	if ((threadIdx.x & 63) == 0) sred[threadIdx.x >> 6] = v;
	__syncthreads();
	return (sred[0] + sred[1]) + (sred[2] + sred[3]);
}

__device__ __forceinline__ float b2f(int d, int j) { return (float)(int8_t)(d >> (8 * j)); }

__device__ __forceinline__ float gelu_lut(float x, const float *lut, float gmin, float geps, int size) {
	int idx = (int)((x - gmin) / geps);
	if (idx < 0) return 0.0f;
	if (idx >= size) return x;
	return lut[idx];
}

__global__ __launch_bounds__(RNT) void embed_rows_kernel(float *x, const int *ids, const int8_t *wte, const float *scales,
                                                         int hidden, int vocab, float emb_scale) {
	const int s = blockIdx.x;
	int tok = ids[s];
	tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
	const int8_t *row = wte + (size_t)tok * hidden;
	for (int d = threadIdx.x; d < hidden; d += RNT) x[(size_t)s * hidden + d] = scales[d] * (emb_scale * (float)row[d]);
}

// One wave per row, the row held in registers (8 consecutive elements per lane and round; ROUNDS = 3 covers the
// 1152-wide rows with 24 values per lane, which keeps the kernel at four rows per SIMD), wave reductions only:
// [post-norm + residual (+ residual out)] + pre-norm.  The normalised row goes out as fp32 (out != nullptr) and/or
// straight as the int8 digit planes + row factors of the MFMA GEMM that consumes it (apack != nullptr): the same bits
// the stand-alone quantising pre-pass would produce from the fp32 row.
template <int ROUNDS, int NPARTS>
__global__ __launch_bounds__(RNT) void norm_rows_kernel(float *out, const float *in, size_t part_stride, const float *w_pre,
                                                        const float *w_post, const float *resid, float *resid_out, int S, int dim,
                                                        int8_t *apack, float *rowfac, int Mpad, float *clear_rows) {
	typedef float f32x4 __attribute__((ext_vector_type(4)));
	const int lane = threadIdx.x & 63, s = blockIdx.x * (RNT / 64) + (threadIdx.x >> 6);
	if (s >= S) return;  // uniform over the wave
	if (clear_rows != nullptr && lane == 0) clear_rows[s] = 0.0f;
	const float eps = 1e-06f;
	const int npieces = dim >> 3;
	bool act[ROUNDS];
	size_t off[ROUNDS];  // element offset of this lane's piece inside a row (clamped to piece 0 when the lane idles)
	f32x4 v[ROUNDS][2], rs[ROUNDS][2], wpo[ROUNDS][2], wpr[ROUNDS][2];
	// every load of the row is requested before the first use
#pragma unroll
	for (int r = 0; r < ROUNDS; r++) {
		const int piece = lane + 64 * r;
		act[r] = piece < npieces;
		off[r] = act[r] ? (size_t)piece * 8 : 0;
#pragma unroll
		for (int q = 0; q < 2; q++) v[r][q] = *reinterpret_cast<const f32x4 *>(in + (size_t)s * dim + off[r] + 4 * q);
	}
	if (NPARTS > 1) {  // the row arrives as NPARTS addends (a product computed in parts of K): all fetched, then added in order
		f32x4 more[NPARTS > 1 ? NPARTS - 1 : 1][ROUNDS][2];
#pragma unroll
		for (int p = 1; p < NPARTS; p++)
#pragma unroll
			for (int r = 0; r < ROUNDS; r++)
#pragma unroll
				for (int q = 0; q < 2; q++)
					more[p - 1][r][q] = *reinterpret_cast<const f32x4 *>(in + (size_t)p * part_stride + (size_t)s * dim + off[r] + 4 * q);
#pragma unroll
		for (int p = 1; p < NPARTS; p++)
#pragma unroll
			for (int r = 0; r < ROUNDS; r++)
#pragma unroll
				for (int q = 0; q < 2; q++) v[r][q] += more[p - 1][r][q];
	}
	if (resid != nullptr) {
#pragma unroll
		for (int r = 0; r < ROUNDS; r++)
#pragma unroll
			for (int q = 0; q < 2; q++) {
				rs[r][q] = *reinterpret_cast<const f32x4 *>(resid + (size_t)s * dim + off[r] + 4 * q);
				wpo[r][q] = *reinterpret_cast<const f32x4 *>(w_post + off[r] + 4 * q);
			}
	}
	if (w_pre != nullptr) {
#pragma unroll
		for (int r = 0; r < ROUNDS; r++)
#pragma unroll
			for (int q = 0; q < 2; q++) wpr[r][q] = *reinterpret_cast<const f32x4 *>(w_pre + off[r] + 4 * q);
	}
	float ss = 0.0f;
#pragma unroll
	for (int r = 0; r < ROUNDS; r++)
#pragma unroll
		for (int q = 0; q < 2; q++) {
			if (!act[r]) v[r][q] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
			for (int e = 0; e < 4; e++) ss = fmaf(v[r][q][e], v[r][q][e], ss);
		}
	ss = tg_wave_sum(ss);
	if (resid != nullptr) {
		const float irms = __builtin_amdgcn_rsqf(ss * (1.0f / (float)dim) + eps);  // v_rsq_f32, as the decode kernels
		float s2 = 0.0f;
#pragma unroll
		for (int r = 0; r < ROUNDS; r++)
#pragma unroll
			for (int q = 0; q < 2; q++) {
				f32x4 t;
#pragma unroll
				for (int e = 0; e < 4; e++) {
					t[e] = act[r] ? (v[r][q][e] * irms) * (wpo[r][q][e] + 1.0f) + rs[r][q][e] : 0.0f;
					s2 = fmaf(t[e], t[e], s2);
				}
				v[r][q] = t;
				if (act[r]) *reinterpret_cast<f32x4 *>(resid_out + (size_t)s * dim + off[r] + 4 * q) = t;
			}
		ss = tg_wave_sum(s2);
	}
	if (out == nullptr && apack == nullptr) return;
	const float irms = __builtin_amdgcn_rsqf(ss * (1.0f / (float)dim) + eps);
	float amax = 0.0f;
#pragma unroll
	for (int r = 0; r < ROUNDS; r++)
#pragma unroll
		for (int q = 0; q < 2; q++) {
			f32x4 y;
#pragma unroll
			for (int e = 0; e < 4; e++) {
				y[e] = act[r] ? (v[r][q][e] * irms) * (wpr[r][q][e] + 1.0f) : 0.0f;
				amax = fmaxf(amax, fabsf(y[e]));
			}
			v[r][q] = y;
			if (out != nullptr && act[r]) *reinterpret_cast<f32x4 *>(out + (size_t)s * dim + off[r] + 4 * q) = y;
		}
	if (apack == nullptr) return;
	amax = tg_wave_max(amax);
	float mul, inv;
	tg_row_factors(amax, mul, inv);
	if (lane == 0) {
		rowfac[s] = mul;
		rowfac[Mpad + s] = inv;
	}
#pragma unroll
	for (int r = 0; r < ROUNDS; r++) {
		if (!act[r]) continue;
		float y[8];
#pragma unroll
		for (int q = 0; q < 2; q++)
#pragma unroll
			for (int e = 0; e < 4; e++) y[4 * q + e] = v[r][q][e];
		uint2 pl[3];
		tg_quant8(y, mul, pl);
		// two neighbouring lanes share a 16-byte piece of every plane
		const int k0 = (int)off[r];
		uint2 *dst = reinterpret_cast<uint2 *>(tg_plane_dst(apack, s, k0 & ~15, dim)) + ((k0 >> 3) & 1);
#pragma unroll
		for (int p = 0; p < 3; p++) dst[p * 128] = pl[p];  // planes are 64 pieces of 16 bytes apart
	}
}

// Exact-order GEMM: every element is one fp32 fused chain over k = 0..K-1 like the reference's
// (linalg.hpp:210-308), so results are bit-identical to it.  64 rows x 128 output columns per workgroup;
// thread (ty = tid/32, tx = tid%32) owns rows ty*8..+7 and columns tx*4..+3.  Weights are read from the
// GEMV tiling (tiles of Ct columns, [K/4][Ct][4]); for the fused up|gate matrix (epi GEGLU) a tile holds
// Ct/2 up columns then the same Ct/2 gate columns and the workgroup writes gelu(gate) * up.
template <int EPI>
__global__ __launch_bounds__(RNT) void gemm_exact_kernel(float *C, const float *A, const int8_t *Wp, const float *scales, int m,
                                                         int K, int Ct, int ldc, const float *lut, float gmin, float geps,
                                                         int lut_size) {
	constexpr int NTILE = (EPI == TG_EPI_GEGLU) ? 2 : 1;
	const int tid = threadIdx.x, tx = tid & 31, ty = tid >> 5;
	const int row0 = blockIdx.y * 64 + ty * 8;
	const int kgs = K >> 2;
	const int n0 = blockIdx.x * 128 + tx * 4;  // first output column of this thread
	const int cw = (EPI == TG_EPI_GEGLU) ? Ct / 2 : Ct;
	const int tile = n0 / cw, cc = n0 % cw;
	int vcol[NTILE];  // virtual column (tile order) of the thread's first column, per operand
	vcol[0] = tile * Ct + cc;
	if (NTILE == 2) vcol[NTILE - 1] = tile * Ct + cw + cc;
	float acc[NTILE][8][4];
#pragma unroll
	for (int t = 0; t < NTILE; t++)
#pragma unroll
		for (int r = 0; r < 8; r++)
#pragma unroll
			for (int c = 0; c < 4; c++) acc[t][r][c] = 0.0f;
	const float *arow[8];
#pragma unroll
	for (int r = 0; r < 8; r++) arow[r] = A + (size_t)((row0 + r < m) ? row0 + r : m - 1) * K;
	const uint4 *wsrc[NTILE];
#pragma unroll
	for (int t = 0; t < NTILE; t++)
		wsrc[t] = reinterpret_cast<const uint4 *>(Wp + ((size_t)tile * kgs * Ct + (size_t)(vcol[t] - tile * Ct)) * 4);
	const size_t kstep = (size_t)Ct / 4;  // 16-byte pieces per k group

	for (int kg = 0; kg < kgs; kg++) {
		float4 av[8];
#pragma unroll
		for (int r = 0; r < 8; r++) av[r] = *reinterpret_cast<const float4 *>(arow[r] + 4 * kg);
#pragma unroll
		for (int t = 0; t < NTILE; t++) {
			const uint4 wv = wsrc[t][(size_t)kg * kstep];
			const int d[4] = {(int)wv.x, (int)wv.y, (int)wv.z, (int)wv.w};
#pragma unroll
			for (int c = 0; c < 4; c++) {
				const float w0 = b2f(d[c], 0), w1 = b2f(d[c], 1), w2 = b2f(d[c], 2), w3 = b2f(d[c], 3);
#pragma unroll
				for (int r = 0; r < 8; r++) {
					float a = acc[t][r][c];
					a = fmaf(av[r].x, w0, a);
					a = fmaf(av[r].y, w1, a);
					a = fmaf(av[r].z, w2, a);
					a = fmaf(av[r].w, w3, a);
					acc[t][r][c] = a;
				}
			}
		}
	}
#pragma unroll
	for (int r = 0; r < 8; r++) {
		if (row0 + r >= m) continue;
		float4 o;
		float *op = &o.x;
		if (EPI == TG_EPI_GEGLU) {
#pragma unroll
			for (int c = 0; c < 4; c++) {
				const float up = acc[0][r][c] * scales[vcol[0] + c];
				const float gate = acc[NTILE - 1][r][c] * scales[vcol[NTILE - 1] + c];
				op[c] = gelu_lut(gate, lut, gmin, geps, lut_size) * up;
			}
		} else {
#pragma unroll
			for (int c = 0; c < 4; c++) op[c] = acc[0][r][c] * scales[vcol[0] + c];
		}
		*reinterpret_cast<float4 *>(C + (size_t)(row0 + r) * ldc + n0) = o;
	}
}

// Plain streaming copy of n 16-byte pieces: the known-size kernel that hardware byte counters are
// scaled against.
__global__ __launch_bounds__(RNT) void tg_copy_kernel(uint4 *dst, const uint4 *src, size_t n) {
	for (size_t i = (size_t)blockIdx.x * RNT + threadIdx.x; i < n; i += (size_t)gridDim.x * RNT) dst[i] = src[i];
}

}  // namespace

void tg_launch_copy(void *dst, const void *src, size_t bytes, hipStream_t s) {
	hipLaunchKernelGGL(tg_copy_kernel, dim3(4096), dim3(RNT), 0, s, (uint4 *)dst, (const uint4 *)src, bytes / 16);
}

void tg_launch_embed_rows(float *x, const int *ids, int S, const int8_t *wte, const float *scales, int hidden, int vocab,
                          hipStream_t s) {
	const float emb_scale = (float)sqrt((double)hidden);  // ops.hpp:537
	hipLaunchKernelGGL(embed_rows_kernel, dim3((unsigned)S), dim3(RNT), 0, s, x, ids, wte, scales, hidden, vocab, emb_scale);
}

// in: nparts (1, 2 or 4) addends of every row, part_stride floats apart
void tg_launch_norm_rows(float *out, const float *in, int nparts, size_t part_stride, const float *w_pre, const float *w_post,
                         const float *resid, float *resid_out, int S, int dim, int8_t *apack, float *rowfac, hipStream_t s,
                         float *clear_rows) {
	const int Mpad = (int)tg_gemm_mfma_rows(S);
	const dim3 grid((unsigned)((S + RNT / 64 - 1) / (RNT / 64))), block(RNT);
	// dim is a legal row dimension: a multiple of 16, at most 1536 where a norm is applied (hidden sizes 640 and 1152)
#define TG_NORM_ROWS(R, P)                                                                                                        \
	hipLaunchKernelGGL((norm_rows_kernel<R, P>), grid, block, 0, s, out, in, part_stride, w_pre, w_post, resid, resid_out, S, dim, apack, \
	                   rowfac, Mpad, clear_rows)
	if (dim <= 1024) {
		if (nparts == 4) TG_NORM_ROWS(2, 4);
		else if (nparts == 2) TG_NORM_ROWS(2, 2);
		else TG_NORM_ROWS(2, 1);
	} else {
		if (nparts == 4) TG_NORM_ROWS(3, 4);
		else if (nparts == 2) TG_NORM_ROWS(3, 2);
		else TG_NORM_ROWS(3, 1);
	}
#undef TG_NORM_ROWS
}

// Wp/scales: GEMV tiling of the matrix (ntiles tiles of Ct columns); C gets ntiles * Ct columns, or half of that for GEGLU
void tg_launch_gemm(float *C, const float *A, const int8_t *Wp, const float *scales, int m, int K, int ntiles, int Ct, int epi,
                    const float *lut, float gmin, float geps, int lut_size, hipStream_t s) {
	dim3 block(RNT);
	const int ncols = (epi == TG_EPI_GEGLU) ? ntiles * Ct / 2 : ntiles * Ct;
	dim3 grid((unsigned)(ncols / 128), (unsigned)((m + 63) / 64));
	if (epi == TG_EPI_GEGLU) {
		hipLaunchKernelGGL(gemm_exact_kernel<TG_EPI_GEGLU>, grid, block, 0, s, C, A, Wp, scales, m, K, Ct, ncols, lut, gmin, geps, lut_size);
	} else {
		hipLaunchKernelGGL(gemm_exact_kernel<TG_EPI_STORE>, grid, block, 0, s, C, A, Wp, scales, m, K, Ct, ncols, lut, gmin, geps, lut_size);
	}
}

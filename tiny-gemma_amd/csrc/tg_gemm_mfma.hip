// Prefill int8-weight GEMM on the matrix cores (gfx950 MFMA), replacing gemm::launch_qgemm
// (csrc/include/linalg.hpp:210-308 of the reference):  C[m][n] = scales[n] * sum_k A[m][k] * float(W[k][n]).
//
// The reference accumulates every element in one fp32 fused chain.  MFMA has no fp32-input mode fast
// enough to matter (fp32 MFMA peaks at 157 TFLOP/s, fp16 at 2.5 PFLOP/s) and rounding the activations to
// one 16-bit value would cost 1e-3 of accuracy, which the model's step-function GeLU table turns into
// visible drift.  So the contraction is done at fp32-equivalent accuracy on fp16 MFMA:
//
//   * int8 weights are converted to fp16 exactly (|w| <= 127);
//   * each activation row is scaled by a power of two so that its largest magnitude lies in
//     [2^10, 2^11) (exact), then split a' = hi + lo with hi = fp16(a'), lo = fp16(a' - hi):
//     22 mantissa bits, |lo| <= 0.5, no subnormal hi for anything that matters;
//   * hi.w and lo.w are exact in fp32 (11 + 7 bits); both are accumulated into the same fp32 MFMA
//     accumulator, i.e. the kernel runs a [hi|lo] x [W;W] product: 2 MFMA per weight tile;
//   * the epilogue multiplies by the row's inverse power of two and the column scale.
//
// Data flow: a pre-pass (split_pack_rows_kernel) writes the hi/lo halves directly in MFMA A-operand
// order, so every wave fetches its A operands with fully coalesced 16-byte loads straight from global
// memory (a wave owns 32 rows: nothing to share, no LDS).  Weight tiles (128 columns, shared by the 4
// waves of a workgroup) are loaded from the packed int8 slab, converted once per workgroup and staged in
// LDS in B-operand order (double buffered, one barrier per 64 rows of K).

#include "tg_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int GNT = 256;    // threads per workgroup: 4 waves, each owns 32 rows x 128 (or 256) columns
constexpr int KSTAGE = 64;  // rows of K per LDS stage

__device__ __forceinline__ float gelu_lut(float x, const float *lut, float gmin, float geps, int size) {
	int idx = (int)((x - gmin) / geps);
	if (idx < 0) return 0.0f;
	if (idx >= size) return x;
	return lut[idx];
}

// A [M][lda] fp32 -> Apack [mtiles][K/16][2][64][8] fp16 (hi block, then lo block, each in A-operand lane
// order: lane = row % 32 + 32 * ((k % 16) / 8), 8 consecutive k per lane) and rowscale[m] = 2^-e.
// One workgroup per tile of 32 rows; rows >= M are written as zeros.
__global__ __launch_bounds__(GNT) void split_pack_rows_kernel(const float *A, int lda, int M, int K, _Float16 *Apack, float *rowscale) {
	__shared__ float smax[8][32];
	const int t = threadIdx.x, r = t & 31, kb = t >> 5;
	const int mtile = blockIdx.x, m = mtile * 32 + r;
	const bool valid = m < M;
	const float *row = A + (size_t)(valid ? m : 0) * lda;
	const int k8s = K >> 3;
	float amax = 0.0f;
	if (valid) {
		for (int kk = kb; kk < k8s; kk += 8) {
			const float4 a0 = *reinterpret_cast<const float4 *>(row + 8 * kk), a1 = *reinterpret_cast<const float4 *>(row + 8 * kk + 4);
			amax = fmaxf(amax, fmaxf(fmaxf(fabsf(a0.x), fabsf(a0.y)), fmaxf(fabsf(a0.z), fabsf(a0.w))));
			amax = fmaxf(amax, fmaxf(fmaxf(fabsf(a1.x), fabsf(a1.y)), fmaxf(fabsf(a1.z), fabsf(a1.w))));
		}
	}
	smax[kb][r] = amax;
	__syncthreads();
#pragma unroll
	for (int i = 0; i < 8; i++) amax = fmaxf(amax, smax[i][r]);
	int e = 0;
	float scale = 1.0f, inv = 1.0f;
	if (amax > 0.0f && amax < INFINITY) {
		(void)frexpf(amax, &e);          // amax = f * 2^e, f in [0.5, 1)
		scale = ldexpf(1.0f, 11 - e);    // amax * scale in [2^10, 2^11)
		inv = ldexpf(1.0f, e - 11);
	}
	if (kb == 0) rowscale[mtile * 32 + r] = inv;
	_Float16 *tilebase = Apack + (size_t)mtile * (size_t)(K >> 4) * 1024;
	for (int kk = kb; kk < k8s; kk += 8) {
		float a[8];
		if (valid) {
			const float4 a0 = *reinterpret_cast<const float4 *>(row + 8 * kk), a1 = *reinterpret_cast<const float4 *>(row + 8 * kk + 4);
			a[0] = a0.x; a[1] = a0.y; a[2] = a0.z; a[3] = a0.w; a[4] = a1.x; a[5] = a1.y; a[6] = a1.z; a[7] = a1.w;
		} else {
#pragma unroll
			for (int i = 0; i < 8; i++) a[i] = 0.0f;
		}
		half8 hi, lo;
#pragma unroll
		for (int i = 0; i < 8; i++) {
			const float s = a[i] * scale;
			const _Float16 h = (_Float16)s;
			hi[i] = h;
			lo[i] = (_Float16)(s - (float)h);
		}
		_Float16 *dst = tilebase + (size_t)(kk >> 1) * 1024 + (size_t)(r + 32 * (kk & 1)) * 8;
		*reinterpret_cast<half8 *>(dst) = hi;
		*reinterpret_cast<half8 *>(dst + 512) = lo;
	}
}

// NTB = B tiles per workgroup: 1 (plain) or 2 (the up|gate pair of one block of columns, for gelu(gate)*up)
template <int NTB>
__global__ __launch_bounds__(GNT) void gemm_mfma_kernel(float *C, const _Float16 *Apack, const float *rowscale, const int8_t *Wg,
                                                        const float *scales, int M, int K, int ldc, const float *lut, float gmin,
                                                        float geps, int lut_size) {
	// B operands of one stage: [tile][kblk (8 rows of K)][column][8 halfs], double buffered
	__shared__ __attribute__((aligned(16))) _Float16 Bs[2][NTB][KSTAGE / 8][TG_CT][8];

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
	const int tile0 = blockIdx.x * NTB;
	const int mtile = blockIdx.y * 4 + w;
	const int kgs = K >> 2, nstage = K / KSTAGE;
	const size_t slab = (size_t)K * TG_CT;

	// this thread's two 16-byte pieces of every B stage: piece p = tid and tid + 256
	// (p / 32 = kg within the stage, p % 32 = group of 4 columns)
	const i32x4 *wsrc[NTB];
#pragma unroll
	for (int tb = 0; tb < NTB; tb++) wsrc[tb] = reinterpret_cast<const i32x4 *>(Wg + (size_t)(tile0 + tb) * slab) + tid;
	const half8 *asrc = reinterpret_cast<const half8 *>(Apack + (size_t)mtile * (size_t)(K >> 4) * 1024) + lane;

	i32x4 braw[NTB][2];
	half8 acur[8], anext[8];  // [k16 step within the stage][hi, lo]
	auto load_stage = [&](int st, half8 *areg) {
#pragma unroll
		for (int tb = 0; tb < NTB; tb++) {
			braw[tb][0] = wsrc[tb][(size_t)st * (KSTAGE / 4) * 32];
			braw[tb][1] = wsrc[tb][(size_t)st * (KSTAGE / 4) * 32 + 256];
		}
#pragma unroll
		for (int s = 0; s < 4; s++) {
			areg[2 * s] = asrc[(size_t)(st * 4 + s) * 128];
			areg[2 * s + 1] = asrc[(size_t)(st * 4 + s) * 128 + 64];
		}
	};
	auto store_b = [&](int buf) {
#pragma unroll
		for (int tb = 0; tb < NTB; tb++) {
#pragma unroll
			for (int q = 0; q < 2; q++) {
				const int p = tid + 256 * q, kgl = p >> 5, cl = p & 31;
				const int d[4] = {braw[tb][q].x, braw[tb][q].y, braw[tb][q].z, braw[tb][q].w};
#pragma unroll
				for (int j = 0; j < 4; j++) {
					half4 h;
					h[0] = (_Float16)(int8_t)(d[j]);
					h[1] = (_Float16)(int8_t)(d[j] >> 8);
					h[2] = (_Float16)(int8_t)(d[j] >> 16);
					h[3] = (_Float16)(int8_t)(d[j] >> 24);
					*reinterpret_cast<half4 *>(&Bs[buf][tb][kgl >> 1][4 * cl + j][4 * (kgl & 1)]) = h;
				}
			}
		}
	};

	f32x16 acc[NTB][4];
#pragma unroll
	for (int tb = 0; tb < NTB; tb++)
#pragma unroll
		for (int j = 0; j < 4; j++)
#pragma unroll
			for (int i = 0; i < 16; i++) acc[tb][j][i] = 0.0f;

	load_stage(0, acur);
	for (int st = 0; st < nstage; st++) {
		const int buf = st & 1;
		store_b(buf);
		__syncthreads();
		if (st + 1 < nstage) load_stage(st + 1, anext);
#pragma unroll
		for (int s = 0; s < 4; s++) {
#pragma unroll
			for (int tb = 0; tb < NTB; tb++) {
#pragma unroll
				for (int j = 0; j < 4; j++) {
					const half8 b = *reinterpret_cast<const half8 *>(&Bs[buf][tb][2 * s + (lane >> 5)][32 * j + (lane & 31)][0]);
					acc[tb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(acur[2 * s], b, acc[tb][j], 0, 0, 0);
					acc[tb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(acur[2 * s + 1], b, acc[tb][j], 0, 0, 0);
				}
			}
		}
#pragma unroll
		for (int i = 0; i < 8; i++) acur[i] = anext[i];
	}

	// epilogue: accumulator element i of lane l is row 8*(i/4) + 4*(l/32) + i%4, column l%32 of the 32x32 tile
	const int mbase = mtile * 32;
#pragma unroll
	for (int j = 0; j < 4; j++) {
		const int n = 32 * j + (lane & 31);
#pragma unroll
		for (int i = 0; i < 16; i++) {
			const int m = mbase + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
			if (m < M) {
				const float rs = rowscale[m];
				if (NTB == 1) {
					C[(size_t)m * ldc + (size_t)tile0 * TG_CT + n] = (acc[0][j][i] * rs) * scales[tile0 * TG_CT + n];
				} else {
					const float up = (acc[0][j][i] * rs) * scales[tile0 * TG_CT + n];
					const float gate = (acc[NTB - 1][j][i] * rs) * scales[(tile0 + 1) * TG_CT + n];
					C[(size_t)m * ldc + (size_t)blockIdx.x * TG_CT + n] = gelu_lut(gate, lut, gmin, geps, lut_size) * up;
				}
			}
		}
	}
}

}  // namespace

size_t tg_gemm_mfma_apack_halfs(int M, int K) { return (size_t)((M + 127) / 128) * 128 * (size_t)K * 2; }

// A [M][lda] fp32 -> packed halves + row scales; apack must hold tg_gemm_mfma_apack_halfs(M, K), rowscale ceil(M/128)*128 floats
void tg_launch_split_pack(const float *A, int lda, int M, int K, _Float16 *apack, float *rowscale, hipStream_t s) {
	const int mtiles = ((M + 127) / 128) * 4;
	hipLaunchKernelGGL(split_pack_rows_kernel, dim3((unsigned)mtiles), dim3(GNT), 0, s, A, lda, M, K, apack, rowscale);
}

void tg_launch_gemm_mfma(float *C, const _Float16 *apack, const float *rowscale, const int8_t *Wg, const float *scales, int M, int K,
                         int ntiles, int epi, const float *lut, float gmin, float geps, int lut_size, hipStream_t s) {
	const unsigned mblocks = (unsigned)((M + 127) / 128);
	if (epi == TG_EPI_GEGLU) {
		hipLaunchKernelGGL(gemm_mfma_kernel<2>, dim3((unsigned)(ntiles / 2), mblocks), dim3(GNT), 0, s, C, apack, rowscale, Wg, scales, M,
		                   K, (ntiles / 2) * TG_CT, lut, gmin, geps, lut_size);
	} else {
		hipLaunchKernelGGL(gemm_mfma_kernel<1>, dim3((unsigned)ntiles, mblocks), dim3(GNT), 0, s, C, apack, rowscale, Wg, scales, M, K,
		                   ntiles * TG_CT, lut, gmin, geps, lut_size);
	}
}

// Load-time re-tiling of the reference's weight matrices on the device.
//
// The reference keeps every matrix as int8 [in][out] row-major with one fp32 scale per output column
// (tensor.hpp:144-195) and its file stores them that way (transformer.hpp:122-160).  The kernels here
// read those bytes where the upload put them and write the two layouts the compute kernels stream:
//   GEMV tiles : [tile of C columns][K/4][C][4 consecutive k]
//   MFMA tiles : [tile of 128 columns][K/16][128][16 consecutive k]
// A matrix may be assembled from several source matrices through a column map (Q|K|V side by side;
// up and gate interleaved half a tile at a time), so the fused matrices never exist in row-major form.
// Pure byte shuffling: every source byte is read once with 4-byte loads and written once with 16-byte
// stores per layout; the work is bounded by HBM traffic (2 bytes moved per weight and layout).

#include "tg_internal.h"

namespace {

constexpr int PNT = 256;
typedef unsigned int u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

// first of 4 consecutive source columns behind virtual columns vcol .. vcol + 3, and the source's row pitch
__device__ __forceinline__ const int8_t *map_cols(const TgColMap &m, int vcol, int &pitch) {
	if (m.half > 0) {  // tiles of 2*half virtual columns: half columns of source 0, then the same columns of source 1
		const int t = vcol / (2 * m.half), j = vcol - t * 2 * m.half;
		pitch = m.n[0];
		return (j < m.half) ? m.src[0] + (size_t)t * m.half + j : m.src[1] + (size_t)t * m.half + (j - m.half);
	}
	if (vcol < m.n[0]) {
		pitch = m.n[0];
		return m.src[0] + vcol;
	}
	vcol -= m.n[0];
	if (vcol < m.n[1]) {
		pitch = m.n[1];
		return m.src[1] + vcol;
	}
	pitch = m.n[2];
	return m.src[2] + (vcol - m.n[1]);
}

__device__ __forceinline__ const float *map_scale(const TgColMap &m, int vcol) {
	if (m.half > 0) {
		const int t = vcol / (2 * m.half), j = vcol - t * 2 * m.half;
		return (j < m.half) ? m.scales[0] + (size_t)t * m.half + j : m.scales[1] + (size_t)t * m.half + (j - m.half);
	}
	if (vcol < m.n[0]) return m.scales[0] + vcol;
	vcol -= m.n[0];
	if (vcol < m.n[1]) return m.scales[1] + vcol;
	return m.scales[2] + (vcol - m.n[1]);
}

// byte b of each of four dwords -> one dword (r0 in the lowest byte)
__device__ __forceinline__ u32 gather_byte(u32 r0, u32 r1, u32 r2, u32 r3, int b) {
	const int sh = 8 * b;
	return ((r0 >> sh) & 0xffu) | (((r1 >> sh) & 0xffu) << 8) | (((r2 >> sh) & 0xffu) << 16) | (((r3 >> sh) & 0xffu) << 24);
}

// thread = 4 rows of K x 4 virtual columns: a 4x4 byte transpose, one 16-byte store
__global__ __launch_bounds__(PNT) void retile_gemv_kernel(int8_t *dst, const TgColMap m, int K, int N, int C) {
	const int n4 = N >> 2, kgs = K >> 2;
	const size_t idx = (size_t)blockIdx.x * PNT + threadIdx.x;
	if (idx >= (size_t)n4 * kgs) return;
	const int g = (int)(idx % n4), kg = (int)(idx / n4), vcol = 4 * g;
	int pitch;
	const int8_t *s = map_cols(m, vcol, pitch) + (size_t)(4 * kg) * pitch;
	u32 r[4];
#pragma unroll
	for (int j = 0; j < 4; j++) r[j] = *reinterpret_cast<const u32 *>(s + (size_t)j * pitch);
	u32x4 o;
#pragma unroll
	for (int c = 0; c < 4; c++) o[c] = gather_byte(r[0], r[1], r[2], r[3], c);
	const int t = vcol / C, c0 = vcol - t * C;
	*reinterpret_cast<u32x4 *>(dst + (((size_t)t * kgs + kg) * C + c0) * 4) = o;
}

// thread = 16 rows of K x 4 virtual columns: four 16-byte stores, 64 contiguous bytes
__global__ __launch_bounds__(PNT) void retile_mfma_kernel(int8_t *dst, const TgColMap m, int K, int N) {
	const int n4 = N >> 2, k16s = K >> 4;
	const size_t idx = (size_t)blockIdx.x * PNT + threadIdx.x;
	if (idx >= (size_t)n4 * k16s) return;
	const int g = (int)(idx % n4), kb = (int)(idx / n4), vcol = 4 * g;
	int pitch;
	const int8_t *s = map_cols(m, vcol, pitch) + (size_t)(16 * kb) * pitch;
	u32 r[16];
#pragma unroll
	for (int j = 0; j < 16; j++) r[j] = *reinterpret_cast<const u32 *>(s + (size_t)j * pitch);
	const int t = vcol / TG_CT, c0 = vcol - t * TG_CT;
	u32x4 *d = reinterpret_cast<u32x4 *>(dst + (((size_t)t * k16s + kb) * TG_CT + c0) * 16);
#pragma unroll
	for (int c = 0; c < 4; c++) {
		u32x4 o;
#pragma unroll
		for (int q = 0; q < 4; q++) o[q] = gather_byte(r[4 * q], r[4 * q + 1], r[4 * q + 2], r[4 * q + 3], c);
		d[c] = o;
	}
}

__global__ __launch_bounds__(PNT) void remap_scales_kernel(float *dst, const TgColMap m, int N) {
	const int v = blockIdx.x * PNT + threadIdx.x;
	if (v < N) dst[v] = *map_scale(m, v);
}

}  // namespace

// N virtual columns described by `m` (every segment boundary a multiple of 4 columns, every source 4-byte aligned),
// K rows (a multiple of 16 for the MFMA layout, of 4 for the GEMV layout).
void tg_launch_retile_gemv(int8_t *dst, float *dst_scales, const TgColMap &m, int K, int N, int C, hipStream_t s) {
	const size_t n = (size_t)(N / 4) * (K / 4);
	hipLaunchKernelGGL(retile_gemv_kernel, dim3((unsigned)((n + PNT - 1) / PNT)), dim3(PNT), 0, s, dst, m, K, N, C);
	hipLaunchKernelGGL(remap_scales_kernel, dim3((unsigned)((N + PNT - 1) / PNT)), dim3(PNT), 0, s, dst_scales, m, N);
}

void tg_launch_retile_mfma(int8_t *dst, float *dst_scales, const TgColMap &m, int K, int N, hipStream_t s) {
	const size_t n = (size_t)(N / 4) * (K / 16);
	hipLaunchKernelGGL(retile_mfma_kernel, dim3((unsigned)((n + PNT - 1) / PNT)), dim3(PNT), 0, s, dst, m, K, N);
	hipLaunchKernelGGL(remap_scales_kernel, dim3((unsigned)((N + PNT - 1) / PNT)), dim3(PNT), 0, s, dst_scales, m, N);
}

// Prefill int8-weight GEMM on the integer matrix cores (gfx950 v_mfma_i32_32x32x32_i8), replacing
// gemm::launch_qgemm (csrc/include/linalg.hpp:210-308 of the reference):
//     C[m][n] = scales[n] * sum_k A[m][k] * float(W[k][n]).
//
// The reference accumulates every element in one fp32 fused chain.  The weights are already int8, so the
// contraction is moved to integer arithmetic altogether:
//
//   * each activation row is scaled by a power of two (exact) so that its largest magnitude lies in
//     [2^21, 2^22) and rounded to an integer xi (22 bits + sign: the row maximum keeps close to fp32
//     precision, smaller elements keep the same absolute precision);
//   * xi is written as three signed base-256 digits, xi = 65536 a2 + 256 a1 + a0, each an int8;
//   * three int8 x int8 -> int32 MFMA contractions (one per digit plane) run against the untouched int8
//     weights; |sum| <= 127 * 128 * K < 2^31 for every legal K, so the integer sums are exact;
//   * the epilogue recombines the planes in fp32 and applies the row's inverse power of two and the
//     column scale.
//
// Nothing in the inner loop converts anything: weight tiles go global -> LDS as raw bytes and are read
// back as MFMA operands, digit planes are stored in operand order by the quantising pre-pass and are
// fetched straight from global memory with 16-byte loads (a wave owns its 32 rows: nothing to share).
// The weight fragment is passed as the first MFMA operand and the activation fragment as the second (the
// two have the same register layout), which leaves C transposed in the accumulators: each lane then owns
// runs of four consecutive columns of one output row and stores them 16 bytes at a time.
//
// Layouts
//   weights (built at load time): [tile of 128 columns][K/16][128 columns][16 consecutive k]
//   activations: [tile of 32 rows][K/32][3 planes][64 lanes][16 bytes], lane = row % 32 + 32 * ((k % 32) / 16)
// The k order inside an MFMA step is irrelevant as long as both operands use the same one: lane half hb of
// both operands carries k = 16 hb .. 16 hb + 15 of the step.
//
// For the fused up|gate matrix a tile holds 64 up columns followed by the same 64 gate columns, so
// gelu(gate) * up (modules.hpp:190-195) is formed in the epilogue and the workgroup writes 64 columns.

#include "tg_internal.h"

#include <algorithm>
#include <type_traits>
#include <utility>

// n > 0: products with at least n / 2 output tiles per compute unit run on gemm_i8_lds_kernel (two workgroups per
// compute unit, both operands through an LDS ring); 0: never
int g_gemm_lds = 2;
int g_gemm_lds_cus = 256;  // compute units of the device (set by tg_init)
// launches so far of the few-row kernel, the one-workgroup-per-tile kernel and the two-workgroups-per-unit kernel
// (tests read them to make sure a product really ran on the kernel they mean to check)
long g_gemm_launches[3] = {0, 0, 0};
int g_gemm_lds_ksplit = 1;  // experiment switch: two half-K copies where the tiles would fill under 3/4 of the workgroup slots

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int GNT = 256;     // threads per workgroup: 4 waves, each owns 32 rows x 128 columns
constexpr int KSTAGE = 64;   // rows of K per LDS stage
constexpr int TG_GEMM_SKINNY_ROWS = 448;    // at most this many rows and
constexpr int TG_GEMM_SKINNY_BLOCKS = 128;  // fewer workgroups than this in the plain tiling: split K over the waves
constexpr int LUT_LDS_MAX = 4096;  // GeLU tables up to this many entries are staged in LDS (Bs holds 16 KB)

// ginv != 0: the table step is a power of two and ginv its exact reciprocal, so the product equals the quotient
__device__ __forceinline__ float gelu_lut(float x, const float *lut, float gmin, float geps, float ginv, int size) {
	int idx = (ginv != 0.0f) ? (int)((x - gmin) * ginv) : (int)((x - gmin) / geps);
	if (idx < 0) return 0.0f;
	if (idx >= size) return x;
	return lut[idx];
}

// One wave per row: mul[m] = 2^s with max|A[m][:]| * 2^s in [2^21, 2^22), inv[m] = 2^-s.
__global__ __launch_bounds__(GNT) void row_scale_kernel(const float *A, int lda, int M, int K, float *mul, float *inv, int Mpad) {
	const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
	if (m >= Mpad) return;
	float amax = 0.0f;
	if (m < M) {
		const f32x4 *row = reinterpret_cast<const f32x4 *>(A + (size_t)m * lda);
		for (int i = lane; i < (K >> 2); i += 64) {
			const f32x4 a = row[i];
			amax = fmaxf(amax, fmaxf(fmaxf(fabsf(a[0]), fabsf(a[1])), fmaxf(fabsf(a[2]), fabsf(a[3]))));
		}
	}
	amax = tg_wave_max(amax);
	if (lane == 0) {
		float s, r;
		tg_row_factors(amax, s, r);
		mul[m] = s;
		inv[m] = r;
	}
}

// A [M][lda] fp32 -> digit planes in A-operand order.  Workgroup = 32 rows x 128 k; thread = one lane's 16
// bytes of one (k step, half): row r = tid % 32, k = 128 blockIdx.y + 16 (tid / 32) .. + 15.
// FROM_MAX: `mul` holds the rows' maxima instead (left by the producer of A): the factors are formed here, and the
// workgroups of the first 128 k also store them for the product's epilogue (mul_out, inv_out).
template <bool FROM_MAX>
__global__ __launch_bounds__(GNT) void quant_pack_kernel(const float *A, int lda, int M, int K, const float *mul, int8_t *Apack,
                                                         float *mul_out, float *inv_out) {
	const int tid = threadIdx.x, r = tid & 31, kq = tid >> 5;
	const int mtile = blockIdx.x, m = mtile * 32 + r;
	const int k0 = blockIdx.y * 128 + 16 * kq;
	i32x4 pl[3] = {i32x4{0, 0, 0, 0}, i32x4{0, 0, 0, 0}, i32x4{0, 0, 0, 0}};
	float factor = 1.0f;
	if (FROM_MAX) {
		float rcp;
		tg_row_factors(m < M ? mul[m] : 0.0f, factor, rcp);  // rows of the padding were never written
		if (blockIdx.y == 0 && kq == 0) {
			mul_out[m] = factor;
			inv_out[m] = rcp;
		}
	} else if (m < M) {
		factor = mul[m];
	}
	if (m < M) {
		const f32x4 *src = reinterpret_cast<const f32x4 *>(A + (size_t)m * lda + k0);
		float v[16];
#pragma unroll
		for (int q = 0; q < 4; q++) {
			const f32x4 a = src[q];
#pragma unroll
			for (int i = 0; i < 4; i++) v[4 * q + i] = a[i];
		}
		tg_quant16(v, factor, pl);
	}
	i32x4 *dst = tg_plane_dst(Apack, m, k0, K);
#pragma unroll
	for (int p = 0; p < 3; p++) dst[p * 64] = pl[p];
}

// GEGLU: fused up|gate tile with gelu(gate) * up; LUTLDS: the GeLU table is small enough to be staged in LDS
template <bool GEGLU, bool LUTLDS>
__global__ __launch_bounds__(GNT) void gemm_i8_kernel(float *C, const int8_t *Apack, const float *rowinv, const int8_t *Wg,
                                                      const float *scales, int M, int K, int ldc, const float *lut, float gmin,
                                                      float geps, float ginv, int lut_size, float *rowmax_part, int Mpad, int ksplit,
                                                      size_t csplit) {
	// B operands of one stage: [k / 16][column][16 bytes], double buffered
	__shared__ __attribute__((aligned(16))) i32x4 Bs[2][KSTAGE / 16][TG_CT];
	__shared__ float lut_lds[(GEGLU && LUTLDS) ? LUT_LDS_MAX : 1];

	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c = lane & 31, hb = lane >> 5;
	// Workgroups are handed to the 8 XCDs (each with its own L2) round-robin in launch order.  Give every
	// XCD a contiguous share of the (row block, column tile) grid, row blocks varying fastest, so that the
	// workgroups resident on one XCD at a time share a few activation slabs and weight tiles in its L2.
	int tile, mblock;
	{
		const int ntiles = (int)gridDim.x, mblocks = (int)gridDim.y, total = ntiles * mblocks;
		const int lin = (int)blockIdx.x + ntiles * (int)blockIdx.y;
		if ((total & 7) == 0) {
			const int chunk = total >> 3, v = (lin & 7) * chunk + (lin >> 3);
			if ((mblocks & 7) == 0) {
				const int mbx = mblocks >> 3, xcd = lin & 7, i = v - xcd * chunk;
				mblock = xcd * mbx + i % mbx;
				tile = i / mbx;
			} else {
				mblock = v % mblocks;
				tile = v / mblocks;
			}
		} else {
			tile = (int)blockIdx.x;
			mblock = (int)blockIdx.y;
		}
	}
	// ksplit == 2: the grid holds every row block twice; copy z walks half z of K and writes its own partial result
	// (C + z * csplit), which the consumer adds.  Used where the plain grid would leave most compute units idle in
	// its last round (288 workgroups on 256 compute units).
	const int mreal = (int)gridDim.y / ksplit, z = mblock / mreal;
	mblock -= z * mreal;
	const int mtile = mblock * 4 + w;
	const int nstage = K / KSTAGE / ksplit;
	if (GEGLU && LUTLDS) {  // the table is read once per output element; visible after the first barrier
		for (int i = tid; i < lut_size; i += GNT) lut_lds[i] = lut[i];
	}
	C += (size_t)z * csplit;

	// a stage of B is 8 KB contiguous: 512 pieces of 16 bytes, two per thread
	const i32x4 *bsrc = reinterpret_cast<const i32x4 *>(Wg + (size_t)tile * (size_t)K * TG_CT) + tid + (size_t)z * nstage * 512;
	const i32x4 *asrc =
	    reinterpret_cast<const i32x4 *>(Apack) + (size_t)mtile * (size_t)(K >> 5) * 3 * 64 + lane + (size_t)z * nstage * 6 * 64;
	i32x4 *bdst = &Bs[0][0][0] + tid;

	// Software pipeline, all through registers (one wave per SIMD: nothing else hides latency):
	//   A of stage s is requested 3 stages before its use and lives in areg[s % 4];
	//   B of stage s is requested 4 stages ahead into breg[s % 4], written to LDS buffer s % 2 during
	//   stage s - 1 and read from there (first k step: during stage s - 1, after its barrier); one barrier per stage.
	i32x4 areg[4][6];  // [ring slot][k step within the stage * 3 + plane]
	i32x4 breg[4][2];
	auto load_b = [&](int st, i32x4 *r) {
		r[0] = bsrc[(size_t)st * 512];
		r[1] = bsrc[(size_t)st * 512 + 256];
	};
	auto store_b = [&](int buf, const i32x4 *r) {
		bdst[buf * 512] = r[0];
		bdst[buf * 512 + 256] = r[1];
	};
	auto load_a = [&](int st, i32x4 *r) {
#pragma unroll
		for (int i = 0; i < 6; i++) r[i] = asrc[(size_t)(st * 6 + i) * 64];
	};

	i32x16 acc[3][4];
#pragma unroll
	for (int p = 0; p < 3; p++)
#pragma unroll
		for (int j = 0; j < 4; j++)
#pragma unroll
			for (int i = 0; i < 16; i++) acc[p][j][i] = 0;

	// B fragments of one k step (32 rows of K): bfrag[j] = columns 32 j .. 32 j + 31
	auto read_b = [&](int buf, int ks, i32x4 *bfrag) {
#pragma unroll
		for (int j = 0; j < 4; j++) bfrag[j] = Bs[buf][2 * ks + hb][32 * j + c];
	};
	auto mfma_step = [&](const i32x4 *a, const i32x4 *bfrag) {
#pragma unroll
		for (int p = 0; p < 3; p++)
#pragma unroll
			for (int j = 0; j < 4; j++) acc[p][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bfrag[j], a[p], acc[p][j], 0, 0, 0);
	};
	i32x4 b0[4], b1[4];  // fragments of the stage's first / second k step; b0 is fetched one stage ahead

	// Every stage issues its loads unconditionally (stage indices are clamped at the end of K, the
	// surplus loads land in ring slots nobody reads again): with loads under branches the compiler can no
	// longer count how many are in flight and falls back to waiting for all of them.
	const int last = nstage - 1;
	auto clamp = [&](int st) { return st < last ? st : last; };
	auto stage = [&](int st, auto uc) {
		constexpr int u = decltype(uc)::value;
		// The scheduler may not move anything across the stage's start, its barrier or its end: free to, it spread the
		// requests over the stage (they are wanted early: 2.9 us per four stages of a 178-row product, 2.5 us pinned;
		// spreading them by hand, one in front of every third matrix instruction, gave 2.85 us).
		__builtin_amdgcn_sched_barrier(0);
		load_a(clamp(st + 3), areg[(u + 3) & 3]);
		load_b(clamp(st + 4), breg[u]);
		// LDS buffer (st+1) % 2 was last read before the previous barrier
		store_b((u + 1) & 1, breg[(u + 1) & 3]);
		// The single barrier of a stage sits between its two k steps: every LDS read is issued one MFMA
		// block before its use, and the matrix cores idle only for the skew between the waves.
		read_b(u & 1, 1, b1);
		mfma_step(areg[u], b0);
		__builtin_amdgcn_sched_barrier(0);
		tg_lds_barrier();  // all of B(st+1) is in LDS; all reads of buffer st % 2 have completed
		__builtin_amdgcn_sched_barrier(0);
		read_b((u + 1) & 1, 0, b0);
		mfma_step(areg[u] + 3, b1);
		__builtin_amdgcn_sched_barrier(0);
	};
	load_b(0, breg[0]);
	load_a(0, areg[0]);
	load_b(clamp(1), breg[1]);
	load_a(clamp(1), areg[1]);
	load_b(clamp(2), breg[2]);
	load_a(clamp(2), areg[2]);
	load_b(clamp(3), breg[3]);
	store_b(0, breg[0]);
	tg_lds_barrier();
	read_b(0, 0, b0);
	int st0 = 0;
	for (; st0 + 4 <= nstage; st0 += 4) {
		stage(st0, std::integral_constant<int, 0>{});
		stage(st0 + 1, std::integral_constant<int, 1>{});
		stage(st0 + 2, std::integral_constant<int, 2>{});
		stage(st0 + 3, std::integral_constant<int, 3>{});
	}
	if (nstage & 2) {  // nstage is even (K is a multiple of 128)
		stage(st0, std::integral_constant<int, 0>{});
		stage(st0 + 1, std::integral_constant<int, 1>{});
	}

	// epilogue.  The weight fragment is the first MFMA operand, so the accumulators hold the tile transposed:
	// element i of lane l is output column 8*(i/4) + 4*(l/32) + i%4 and output row l%32 of the 32x32 tile,
	// i.e. four consecutive floats of one row of C per group of four elements: 16-byte stores.
	const int m = mtile * 32 + c;
	const float rs = rowinv[m];  // rowinv is padded to whole row tiles
	f32x4 sc[4][4];              // column scales of [column tile j][group q]
#pragma unroll
	for (int j = 0; j < 4; j++)
#pragma unroll
		for (int q = 0; q < 4; q++) sc[j][q] = *reinterpret_cast<const f32x4 *>(scales + tile * TG_CT + 32 * j + 8 * q + 4 * hb);
	auto value = [&](int j, int i) {
		const float v = fmaf((float)acc[2][j][i], 65536.0f, fmaf((float)acc[1][j][i], 256.0f, (float)acc[0][j][i]));
		return (v * rs) * sc[j][i >> 2][i & 3];
	};
	float omax = 0.0f;  // GEGLU: largest magnitude this lane writes (its row, 32 of the tile's 64 columns)
	if (m < M) {
		float *crow = C + (size_t)m * ldc + (size_t)tile * (GEGLU ? TG_CT / 2 : TG_CT) + 4 * hb;
#pragma unroll
		for (int j = 0; j < (GEGLU ? 2 : 4); j++) {
#pragma unroll
			for (int q = 0; q < 4; q++) {
				f32x4 o;
#pragma unroll
				for (int e = 0; e < 4; e++) {
					const int i = 4 * q + e;
					if (GEGLU) {
						const float gate = value(j + 2, i);
						o[e] = (LUTLDS ? gelu_lut(gate, lut_lds, gmin, geps, ginv, lut_size) : gelu_lut(gate, lut, gmin, geps, ginv, lut_size)) *
						       value(j, i);
						omax = fmaxf(omax, fabsf(o[e]));
					} else {
						o[e] = value(j, i);
					}
				}
				*reinterpret_cast<f32x4 *>(crow + 32 * j + 8 * q) = o;
			}
		}
	}
	if (GEGLU && rowmax_part != nullptr) {
		// the consumer quantises these rows next: fold max|row| over this tile's columns into the row's maximum
		// (non-negative floats order like their bit patterns; the caller cleared the array)
		omax = fmaxf(omax, tg_red_partner<32>(omax));
		if (hb == 0 && m < M) atomicMax(reinterpret_cast<unsigned *>(rowmax_part) + m, __float_as_uint(omax));
	}
}

// ---- the same product with two workgroups per compute unit -----------------------------------------------------
// The kernels above hold one wave per SIMD (192 accumulators + a register ring of prefetched operands), so nothing
// covers a workgroup's start-up, its barriers or its epilogue (accumulators -> fp32 -> 64 KB of stores with the matrix
// cores idle: a sixth of the time at K = 1152).  Here a wave fits in 256 registers and a second workgroup shares the
// compute unit: while one converts and stores, the other issues matrix instructions.
//
//   * Nothing is prefetched into registers.  Both operands go global -> LDS directly (global_load_lds_dwordx4: no
//     registers, no conversion) into a ring of four one-k-step slots per workgroup (slot = 4 waves x 3 planes of A,
//     each wave copying and reading only its own 3 KB, + 4 KB of B shared by the four waves), three k steps ahead.
//   * One set of operand fragments (7 x 16 bytes per lane), read per k step after the barrier; the LDS latency is
//     covered by the other workgroup's wave on the same SIMD.
//   * The compiler does not see which LDS bytes a direct copy writes and would wait for ALL copies in flight before any
//     LDS read it can see; the fragment reads are therefore explicit ds_read_b128 instructions with their own waits.
//   * Of the 12 accumulator tiles, the 8 of digit planes 0 and 1 live in the accumulation registers and the 4 of plane 2
//     in ordinary vector registers, 128 + 64: with two waves per SIMD a wave has 256 registers of both kinds together.
//     The compiler allots all matrix accumulators to one kind, so the matrix instructions are written out with the
//     register class of each accumulator given.  It therefore does not know them as matrix instructions: the wait
//     between the last of them and the first ordinary read of an accumulator is explicit (s_nop).
//   * The copies of a k step are issued one at a time behind every third matrix instruction: a wave issues in order,
//     and a burst of copies or LDS reads from eight waves fills the queue it goes into and holds the matrix
//     instructions behind it back.
// Same integer sums, same epilogue arithmetic: the result equals the other kernels' bit for bit.
constexpr int LDS_NSLOT = 4, LDS_AW = 3072, LDS_BOFF = 4 * LDS_AW, LDS_SLOT = LDS_BOFF + 4096;

template <int OFF>
__device__ __forceinline__ i32x4 lds_read_frag(unsigned addr) {
	i32x4 r;
	asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
	return r;
}
struct LdsFrags {
	i32x4 a[3], b[4];
};
// names the registers, so that it stays between the reads and their use
__device__ __forceinline__ void lds_frags_wait(LdsFrags &f) {
	asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.b[3]));
}
template <int N>
__device__ __forceinline__ void wait_copies_in_flight() {  // until at most N of this wave's vector memory loads are outstanding
	asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
template <bool IN_ACC_REGS>
__device__ __forceinline__ void mfma_i8_asm(i32x16 &acc, const i32x4 &bf, const i32x4 &af) {
	if constexpr (IN_ACC_REGS) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(bf), "v"(af));
	else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "v"(bf), "v"(af));
}
template <int... I, typename F>
__device__ __forceinline__ void gemm_static_for_impl(std::integer_sequence<int, I...>, F &&f) {
	(f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void gemm_static_for(F &&f) {
	gemm_static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// Debug (tg_debug_gemm_clock): when this points at a buffer, thread 0 of every workgroup of gemm_i8_lds_kernel leaves
// the shader clocks and the ticks of the constant 100 MHz counter it lived for: their ratio is the clock the part held
// while the kernel ran (it lowers the clock under the power limit, by an amount that depends on the operand values).
__device__ unsigned long long *tg_gemm_clk = nullptr;

template <bool GEGLU, bool LUTLDS>
__global__ __launch_bounds__(GNT, 2) void gemm_i8_lds_kernel(float *C, const int8_t *Apack, const float *rowinv, const int8_t *Wg,
                                                             const float *scales, int M, int K, int ldc, const float *lut, float gmin,
                                                             float geps, float ginv, int lut_size, float *rowmax_part, int ntiles,
                                                             int mblocks, int ksplit, size_t csplit) {
	extern __shared__ __attribute__((aligned(1024))) unsigned char ring[];  // LDS_NSLOT slots; the GeLU table afterwards
	const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, hb = lane >> 5;
	const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
	unsigned long long *const clkp = tg_gemm_clk;
	unsigned long long clk_c0 = 0, clk_r0 = 0;
	if (clkp != nullptr) {
		clk_c0 = __builtin_readcyclecounter();
		clk_r0 = __builtin_amdgcn_s_memrealtime();
	}
	// (row block, column tile) of this workgroup: every XCD a contiguous share, row blocks fastest (as gemm_i8_kernel)
	int tile, mblock;
	{
		const int total = ntiles * mblocks, lin = (int)blockIdx.x;
		if ((total & 7) == 0) {
			const int chunk = total >> 3, v = (lin & 7) * chunk + (lin >> 3);
			if ((mblocks & 7) == 0) {
				const int mbx = mblocks >> 3, xcd = lin & 7, i = v - xcd * chunk;
				mblock = xcd * mbx + i % mbx;
				tile = i / mbx;
			} else {
				mblock = v % mblocks;
				tile = v / mblocks;
			}
		} else {
			tile = lin % ntiles;
			mblock = lin / ntiles;
		}
	}
	// ksplit == 2 (plain epilogue): the grid holds every row block twice; copy z walks half z of K and writes its own
	// partial result (C + z * csplit), which the consumer adds.  Taken where one workgroup per tile would leave most
	// compute units with a single workgroup and a few with two, which then set the pace.
	const int mreal = mblocks / ksplit, z = mblock / mreal;
	mblock -= z * mreal;
	const int mtile = mblock * 4 + w;
	const int nstage = (K >> 5) / ksplit, last = nstage - 1;  // one k step (32 rows of K) per stage; a multiple of 4
	const unsigned char *bsrc = reinterpret_cast<const unsigned char *>(Wg) + (size_t)tile * (size_t)K * TG_CT + (size_t)z * nstage * 4096 +
	                            (size_t)w * 1024 + 16 * lane;
	const unsigned char *asrc = reinterpret_cast<const unsigned char *>(Apack) + (size_t)mtile * (size_t)(K >> 5) * 3 * 1024 +
	                            (size_t)z * nstage * LDS_AW + 16 * lane;
	C += (size_t)z * csplit;
	// piece q of the copy of stage st into a slot: q = 0..2 the planes of this wave's 32 rows, q = 3 its quarter of B.
	// Stages past the end copy the last stage again, into slots nobody reads any more.
	auto issue = [&](int st, int slot, int q) __attribute__((always_inline)) {
		st = st < last ? st : last;
		if (q < 3)
			__builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(asrc + (size_t)st * LDS_AW + q * 1024),
			                                 (__attribute__((address_space(3))) void *)(ring + slot * LDS_SLOT + w * LDS_AW + q * 1024), 16, 0, 0);
		else
			__builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(bsrc + (size_t)st * 4096),
			                                 (__attribute__((address_space(3))) void *)(ring + slot * LDS_SLOT + LDS_BOFF + w * 1024), 16, 0, 0);
	};
#pragma unroll
	for (int st = 0; st < LDS_NSLOT - 1; st++)
#pragma unroll
		for (int q = 0; q < 4; q++) issue(st, st, q);

	i32x16 acc[3][4];
#pragma unroll
	for (int p = 0; p < 3; p++)
#pragma unroll
		for (int j = 0; j < 4; j++)
#pragma unroll
			for (int i = 0; i < 16; i++) acc[p][j][i] = 0;

	const unsigned lbase = (unsigned)(size_t)ring;
	const unsigned aaddr = lbase + w * LDS_AW + 16 * lane, baddr = lbase + LDS_BOFF + (hb * TG_CT + c) * 16;
	LdsFrags f;
	auto stage = [&](int st, auto uc) __attribute__((always_inline)) {
		constexpr int U = decltype(uc)::value, O = U * LDS_SLOT;
		wait_copies_in_flight<4 * (LDS_NSLOT - 2)>();  // this wave's copies of stage st have landed
		tg_lds_barrier();                              // everyone's have; everyone has read stage st - 1
		f.a[0] = lds_read_frag<O>(aaddr);
		f.a[1] = lds_read_frag<O + 1024>(aaddr);
		f.a[2] = lds_read_frag<O + 2048>(aaddr);
		f.b[0] = lds_read_frag<O>(baddr);
		f.b[1] = lds_read_frag<O + 512>(baddr);
		f.b[2] = lds_read_frag<O + 1024>(baddr);
		f.b[3] = lds_read_frag<O + 1536>(baddr);
		lds_frags_wait(f);
		gemm_static_for<12>([&](auto ic) {
			constexpr int i = decltype(ic)::value, p = i >> 2, j = i & 3;
			mfma_i8_asm<(p < 2)>(acc[p][j], f.b[j], f.a[p]);
			if constexpr (i % 3 == 2) issue(st + LDS_NSLOT - 1, (U + LDS_NSLOT - 1) % LDS_NSLOT, i / 3);  // into the slot of stage st - 1
		});
	};
	for (int st0 = 0; st0 < nstage; st0 += 4) {
		stage(st0, std::integral_constant<int, 0>{});
		stage(st0 + 1, std::integral_constant<int, 1>{});
		stage(st0 + 2, std::integral_constant<int, 2>{});
		stage(st0 + 3, std::integral_constant<int, 3>{});
	}
	wait_copies_in_flight<0>();  // the surplus copies too: the table below reuses the ring
	// The matrix pipeline finishes its last instruction (8 passes) before an accumulator is read by an ordinary
	// instruction.  The compiler does not know the asm statements above as matrix instructions and inserts no wait of
	// its own, so the wait names every accumulator as an operand: nothing that reads one can be scheduled above it.
	// (Bit-equality of this kernel with the compiler-scheduled gemm_i8_kernel: tests/test_gpu_kernels.py,
	// test_gemm_kernels_agree_bit_for_bit; the compiled code is walked by tests/test_isa_hazards.py.)
	asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15"
	             : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]), "+a"(acc[1][1]), "+a"(acc[1][2]),
	               "+a"(acc[1][3]), "+v"(acc[2][0]), "+v"(acc[2][1]), "+v"(acc[2][2]), "+v"(acc[2][3])
	             :
	             : "memory");
	float *lut_lds = reinterpret_cast<float *>(ring);
	if (GEGLU && LUTLDS) {
		__syncthreads();  // every wave is done with the ring
		for (int i = tid; i < lut_size; i += GNT) lut_lds[i] = lut[i];
		__syncthreads();
	}

	// epilogue, as in gemm_i8_kernel: element i of lane l is output column 8*(i/4) + 4*(l/32) + i%4, row l%32 of a 32x32 tile
	const int m = mtile * 32 + c;
	const float rs = rowinv[m];
	auto value = [&](int j, int i, float scale) {
		const float v = fmaf((float)acc[2][j][i], 65536.0f, fmaf((float)acc[1][j][i], 256.0f, (float)acc[0][j][i]));
		return (v * rs) * scale;
	};
	float omax = 0.0f;
	if (m < M) {
		float *crow = C + (size_t)m * ldc + (size_t)tile * (GEGLU ? TG_CT / 2 : TG_CT) + 4 * hb;
		const float *sc0 = scales + tile * TG_CT + 4 * hb;
#pragma unroll
		for (int j = 0; j < (GEGLU ? 2 : 4); j++) {
#pragma unroll
			for (int q = 0; q < 4; q++) {
				const f32x4 su = *reinterpret_cast<const f32x4 *>(sc0 + 32 * j + 8 * q);
				f32x4 sg = su;
				if (GEGLU) sg = *reinterpret_cast<const f32x4 *>(sc0 + 32 * (j + 2) + 8 * q);
				f32x4 o;
#pragma unroll
				for (int e = 0; e < 4; e++) {
					const int i = 4 * q + e;
					if (GEGLU) {
						const float gate = value(j + 2, i, sg[e]);
						o[e] = (LUTLDS ? gelu_lut(gate, lut_lds, gmin, geps, ginv, lut_size) : gelu_lut(gate, lut, gmin, geps, ginv, lut_size)) *
						       value(j, i, su[e]);
						omax = fmaxf(omax, fabsf(o[e]));
					} else {
						o[e] = value(j, i, su[e]);
					}
				}
				*reinterpret_cast<f32x4 *>(crow + 32 * j + 8 * q) = o;
			}
		}
	}
	if (GEGLU && rowmax_part != nullptr) {
		omax = fmaxf(omax, tg_red_partner<32>(omax));
		if (hb == 0 && m < M) atomicMax(reinterpret_cast<unsigned *>(rowmax_part) + m, __float_as_uint(omax));
	}
	if (clkp != nullptr && tid == 0) {
		clkp[2 * (size_t)blockIdx.x] = __builtin_readcyclecounter() - clk_c0;
		clkp[2 * (size_t)blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - clk_r0;
	}
}

// ---- few rows (a short prompt): the same product with the reduction split over the four waves ----------------
// With a few hundred rows (up to 448: measured crossover between 400 and 512) the kernel above has only a handful of
// workgroups (two row blocks x 9 column tiles for the down
// projection of the 1B shape) and each walks all of K alone.  Here a workgroup owns 32 rows x 128 columns and its
// four waves take the K stages round-robin (stage w, w + 4, ...), each with a private register pipeline: no LDS and
// no barrier in the main loop, weights fetched straight from global memory in operand order (32 lanes x 16 bytes =
// 512 contiguous bytes per fragment).  The integer partial sums are added through LDS at the end (exact, so the
// result equals the unsplit one bit for bit) and every wave finishes a quarter of each column block.
// gridDim.z > 1 (plain epilogue only): K is also cut into gridDim.z equal parts over workgroups; part z writes its own
// partial result C + z * part_stride and the consumer adds them (a long K with few rows and few column tiles would
// otherwise run on a few dozen compute units, each pulling megabytes of weights through its own L1).
template <bool GEGLU, bool LUTLDS>
__global__ __launch_bounds__(GNT) void gemm_i8_skinny_kernel(float *C, const int8_t *Apack, const float *rowinv, const int8_t *Wg,
                                                             const float *scales, int M, int K, int ldc, const float *lut, float gmin,
                                                             float geps, float ginv, int lut_size, float *rowmax_part, int Mpad,
                                                             size_t part_stride) {
	__shared__ __attribute__((aligned(16))) i32x4 red[4][3][4][64];  // [wave][plane][quarter of the 16 registers][lane]
	__shared__ float lut_lds[(GEGLU && LUTLDS) ? LUT_LDS_MAX : 1];
	__shared__ float pmax[4][32];
	typedef i32x4 fin_t;
	const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c = lane & 31, hb = lane >> 5;
	// Workgroups are handed to the 8 XCDs round-robin in launch order, and what one XCD's L2 holds the others must fetch
	// again from the memory side.  XCD x therefore takes a contiguous share of the (K part, column tile, row tile) grid,
	// row tiles varying fastest: the workgroups of a column tile, which read the same weights, sit on one XCD, and an
	// XCD sees one or two K parts of the activations instead of all of them.
	int tile, mtile, z;
	{
		const int ntiles = (int)gridDim.x, mtiles = (int)gridDim.y, total = ntiles * mtiles * (int)gridDim.z;
		const int lin = (int)blockIdx.x + ntiles * ((int)blockIdx.y + mtiles * (int)blockIdx.z);
		const int xcd = lin & 7, full = total >> 3, rem = total & 7;
		const int v = xcd * full + (xcd < rem ? xcd : rem) + (lin >> 3);
		mtile = v % mtiles;
		const int t = v / mtiles;
		tile = t % ntiles;
		z = t / ntiles;
	}
	const int nstage = K / KSTAGE / (int)gridDim.z, last = nstage - 1;  // stages of this workgroup's part of K
	if (GEGLU && LUTLDS) {  // visible after the barriers of the reduction
		for (int i = tid; i < lut_size; i += GNT) lut_lds[i] = lut[i];
	}
	C += (size_t)z * part_stride;
	const i32x4 *bsrc =
	    reinterpret_cast<const i32x4 *>(Wg + (size_t)tile * (size_t)K * TG_CT) + hb * TG_CT + c + (size_t)z * nstage * 4 * TG_CT;
	const i32x4 *asrc =
	    reinterpret_cast<const i32x4 *>(Apack) + (size_t)mtile * (size_t)(K >> 5) * 3 * 64 + lane + (size_t)z * nstage * 6 * 64;

	// ring of three stages: loads go to ordinary vector registers only, and 3 x 56 of them is what fits beside the
	// addresses (the 192 accumulators live in the accumulation registers)
	i32x4 areg[3][6];  // [ring slot][k step * 3 + plane]
	i32x4 breg[3][8];  // [ring slot][k step * 4 + column block]
	auto load = [&](int st, i32x4 *ar, i32x4 *br) {
		st = st < last ? st : last;  // unconditional loads: surplus ones land in ring slots nobody reads again
#pragma unroll
		for (int i = 0; i < 6; i++) ar[i] = asrc[(size_t)(st * 6 + i) * 64];
#pragma unroll
		for (int ks = 0; ks < 2; ks++)
#pragma unroll
			for (int j = 0; j < 4; j++) br[ks * 4 + j] = bsrc[(size_t)(st * 4 + 2 * ks) * TG_CT + 32 * j];
	};
	i32x16 acc[3][4];
#pragma unroll
	for (int p = 0; p < 3; p++)
#pragma unroll
		for (int j = 0; j < 4; j++)
#pragma unroll
			for (int i = 0; i < 16; i++) acc[p][j][i] = 0;

	// iteration i of wave w is stage w + 4 i; every wave runs the same number of iterations, a stage beyond K
	// contributes zeros (its activation fragments are cleared: no branch around the matrix instructions)
	auto stage = [&](int i, auto uc) {
		constexpr int u = decltype(uc)::value;
		load(w + 4 * (i + 2), areg[(u + 2) % 3], breg[(u + 2) % 3]);
		const bool valid = w + 4 * i < nstage;
#pragma unroll
		for (int ks = 0; ks < 2; ks++)
#pragma unroll
			for (int p = 0; p < 3; p++) {
				i32x4 a = areg[u][ks * 3 + p];
				if (!valid) a = i32x4{0, 0, 0, 0};
#pragma unroll
				for (int j = 0; j < 4; j++) acc[p][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(breg[u][ks * 4 + j], a, acc[p][j], 0, 0, 0);
			}
		// Where the stage's 14 loads go among its 24 matrix instructions is fixed here.  Left to itself the scheduler
		// sank the loads of two of every three unrolled stages to the end of the stage that needs their data and
		// waited there for everything in flight (vmcnt(0)): one stage in flight instead of two, 1.1 us per
		// iteration.  All loads in front of the matrix instructions: 0.76 us, but the first stage waits behind three
		// stages of requests.  One load ahead of every two matrix instructions: the same pace and the first stage 0.7 us
		// sooner (the four waves share one request path that takes a 16-byte-per-lane load every 16 clocks).
		__builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
		__builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
#pragma unroll
		for (int g = 0; g < 12; g++) {
			__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
			__builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
		}
		__builtin_amdgcn_sched_barrier(0);
	};
	load(w, areg[0], breg[0]);
	load(w + 4, areg[1], breg[1]);
	const int n_it = (nstage + 3) / 4;
	int i0 = 0;
	for (; i0 + 3 <= n_it; i0 += 3) {
		stage(i0, std::integral_constant<int, 0>{});
		stage(i0 + 1, std::integral_constant<int, 1>{});
		stage(i0 + 2, std::integral_constant<int, 2>{});
	}
	if (i0 < n_it) stage(i0, std::integral_constant<int, 0>{});
	if (i0 + 1 < n_it) stage(i0 + 1, std::integral_constant<int, 1>{});

	// reduction over the waves, one column block per round: every wave leaves its partial sums of the block in LDS and
	// adds up one quarter of it (registers 4 w .. 4 w + 3 of each plane, from all four waves).  After the four
	// rounds wave w holds, of every column block j, the four consecutive output columns 32 j + 8 w + 4 (lane / 32) ..
	fin_t fin[4][3];
#pragma unroll
	for (int j = 0; j < 4; j++) {
#pragma unroll
		for (int p = 0; p < 3; p++)
#pragma unroll
			for (int qq = 0; qq < 4; qq++)
				red[w][p][qq][lane] = i32x4{acc[p][j][4 * qq], acc[p][j][4 * qq + 1], acc[p][j][4 * qq + 2], acc[p][j][4 * qq + 3]};
		__syncthreads();
#pragma unroll
		for (int p = 0; p < 3; p++) fin[j][p] = (red[0][p][w][lane] + red[1][p][w][lane]) + (red[2][p][w][lane] + red[3][p][w][lane]);
		if (j < 3) __syncthreads();
	}

	const int m = mtile * 32 + c;
	const float rs = rowinv[m];
	auto value = [&](const fin_t *f, int e, float scale) {
		const float v = fmaf((float)f[2][e], 65536.0f, fmaf((float)f[1][e], 256.0f, (float)f[0][e]));
		return (v * rs) * scale;
	};
	float omax = 0.0f;
	const int col = 8 * w + 4 * hb;  // of a column block
	f32x4 sc[4];
#pragma unroll
	for (int j = 0; j < 4; j++) sc[j] = *reinterpret_cast<const f32x4 *>(scales + tile * TG_CT + 32 * j + col);
	if (m < M) {
		float *crow = C + (size_t)m * ldc + (size_t)tile * (GEGLU ? TG_CT / 2 : TG_CT) + col;
#pragma unroll
		for (int j = 0; j < (GEGLU ? 2 : 4); j++) {  // GEGLU: blocks 0 and 1 are up, 2 and 3 their gates
			f32x4 o;
#pragma unroll
			for (int e = 0; e < 4; e++) {
				if (GEGLU) {
					const float gate = value(fin[j + 2], e, sc[j + 2][e]);
					o[e] = (LUTLDS ? gelu_lut(gate, lut_lds, gmin, geps, ginv, lut_size) : gelu_lut(gate, lut, gmin, geps, ginv, lut_size)) *
					       value(fin[j], e, sc[j][e]);
					omax = fmaxf(omax, fabsf(o[e]));
				} else {
					o[e] = value(fin[j], e, sc[j][e]);
				}
			}
			*reinterpret_cast<f32x4 *>(crow + 32 * j) = o;
		}
	}
	if (GEGLU && rowmax_part != nullptr) {
		omax = fmaxf(omax, tg_red_partner<32>(omax));
		if (hb == 0) pmax[w][c] = omax;
		__syncthreads();
		if (w == 0 && hb == 0 && m < M)
			atomicMax(reinterpret_cast<unsigned *>(rowmax_part) + m,
			          __float_as_uint(fmaxf(fmaxf(pmax[0][c], pmax[1][c]), fmaxf(pmax[2][c], pmax[3][c]))));
	}
}

}  // namespace

// scratch sizes for M rows of K: digit planes (bytes) and row factors (floats, two arrays of this length)
size_t tg_gemm_mfma_apack_bytes(int M, int K) { return (size_t)((M + 127) / 128) * 128 * (size_t)K * 3; }
size_t tg_gemm_mfma_rows(int M) { return (size_t)((M + 127) / 128) * 128; }

// A [M][lda] fp32 -> digit planes + row factors; rowfac holds 2 * tg_gemm_mfma_rows(M) floats (multipliers, then inverses).
// rowmax != nullptr: [tg_gemm_mfma_rows(M)] row maxima left by the producer of A (no pass over A for them).
void tg_launch_quant_pack(const float *A, int lda, int M, int K, int8_t *apack, float *rowfac, const float *rowmax, hipStream_t s) {
	const int Mpad = (int)tg_gemm_mfma_rows(M);
	const dim3 grid((unsigned)(Mpad / 32), (unsigned)(K / 128));
	if (rowmax != nullptr) {
		hipLaunchKernelGGL(quant_pack_kernel<true>, grid, dim3(GNT), 0, s, A, lda, M, K, rowmax, apack, rowfac, rowfac + Mpad);
		return;
	}
	hipLaunchKernelGGL(row_scale_kernel, dim3((unsigned)(Mpad / 4)), dim3(GNT), 0, s, A, lda, M, K, rowfac, rowfac + Mpad, Mpad);
	hipLaunchKernelGGL(quant_pack_kernel<false>, grid, dim3(GNT), 0, s, A, lda, M, K, rowfac, apack, (float *)nullptr, (float *)nullptr);
}

// whether a product of M rows, K deep, ntiles column tiles runs on gemm_i8_lds_kernel (K in whole groups of four k steps)
static bool tg_gemm_lds_taken(int M, int K, int ntiles) {
	const int tiles = ntiles * ((M + 127) / 128);
	if (M <= TG_GEMM_SKINNY_ROWS && tiles < TG_GEMM_SKINNY_BLOCKS) return false;  // the few-row kernel's case
	return g_gemm_lds > 0 && (K & 127) == 0 && 2 * tiles >= g_gemm_lds * g_gemm_lds_cus;
}

// ntiles tiles of 128 (virtual) columns; epi GEGLU: every tile is 64 up | 64 gate columns and C has ntiles * 64 columns;
// rowmax_part (GEGLU only, may be null): [tg_gemm_mfma_rows(M)] floats cleared by the caller; max|C[m][:]| is folded into it
void tg_launch_gemm_mfma(float *C, const int8_t *apack, const float *rowfac, const int8_t *Wg, const float *scales, int M, int K,
                         int ntiles, int epi, const float *lut, float gmin, float geps, int lut_size, float *rowmax_part,
                         int kparts, size_t part_stride, hipStream_t s) {
	const unsigned mblocks = (unsigned)((M + 127) / 128);
	const int Mpad = (int)tg_gemm_mfma_rows(M);
	const float *rowinv = rowfac + Mpad;
	int e = 0;
	const float ginv = (epi == TG_EPI_GEGLU && geps > 0.0f && frexpf(geps, &e) == 0.5f && e > -100 && e < 100) ? 1.0f / geps : 0.0f;
	const bool geglu = epi == TG_EPI_GEGLU, lutlds = geglu && lut_size <= LUT_LDS_MAX;
	const int ldc = geglu ? ntiles * (TG_CT / 2) : ntiles * TG_CT;
	float *rmp = geglu ? rowmax_part : nullptr;
	// few rows and few column tiles: split K over the waves instead of leaving most compute units idle
	if (M <= TG_GEMM_SKINNY_ROWS && (int)mblocks * ntiles < TG_GEMM_SKINNY_BLOCKS) {
		g_gemm_launches[0]++;
		const dim3 grid((unsigned)ntiles, (unsigned)((M + 31) / 32), (unsigned)(geglu ? 1 : kparts)), block(GNT);
		if (geglu && lutlds)
			hipLaunchKernelGGL((gemm_i8_skinny_kernel<true, true>), grid, block, 0, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin, geps,
			                   ginv, lut_size, rmp, Mpad, (size_t)0);
		else if (geglu)
			hipLaunchKernelGGL((gemm_i8_skinny_kernel<true, false>), grid, block, 0, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin, geps,
			                   ginv, lut_size, rmp, Mpad, (size_t)0);
		else
			hipLaunchKernelGGL((gemm_i8_skinny_kernel<false, false>), grid, block, 0, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin,
			                   geps, ginv, lut_size, rmp, Mpad, part_stride);
		return;
	}
	// kparts == 2 (STORE only; see tg_gemm_mfma_k_parts): two half-K copies of the grid, the second writes C + part_stride
	const int ksplit = (kparts == 2 && !geglu) ? 2 : 1;
	const size_t csplit = ksplit == 2 ? part_stride : 0;
	if (tg_gemm_lds_taken(M, K, ntiles) && (K >> 5) % (4 * ksplit) == 0) {
		g_gemm_launches[2]++;
		static bool lds_set = false;
		constexpr int ring_bytes = LDS_NSLOT * LDS_SLOT;
		if (!lds_set) {  // 64 KB of dynamic LDS
			(void)hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_i8_lds_kernel<true, true>), hipFuncAttributeMaxDynamicSharedMemorySize, ring_bytes);
			(void)hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_i8_lds_kernel<true, false>), hipFuncAttributeMaxDynamicSharedMemorySize, ring_bytes);
			(void)hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_i8_lds_kernel<false, false>), hipFuncAttributeMaxDynamicSharedMemorySize, ring_bytes);
			lds_set = true;
		}
		const int mb = (int)mblocks * ksplit;
		const dim3 grid((unsigned)(ntiles * mb)), block(GNT);
		if (geglu && lutlds)
			hipLaunchKernelGGL((gemm_i8_lds_kernel<true, true>), grid, block, ring_bytes, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin, geps,
			                   ginv, lut_size, rmp, ntiles, mb, 1, (size_t)0);
		else if (geglu)
			hipLaunchKernelGGL((gemm_i8_lds_kernel<true, false>), grid, block, ring_bytes, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin, geps,
			                   ginv, lut_size, rmp, ntiles, mb, 1, (size_t)0);
		else
			hipLaunchKernelGGL((gemm_i8_lds_kernel<false, false>), grid, block, ring_bytes, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin,
			                   geps, ginv, lut_size, rmp, ntiles, mb, ksplit, csplit);
		return;
	}
	g_gemm_launches[1]++;
	const dim3 grid((unsigned)ntiles, mblocks * (unsigned)ksplit), block(GNT);
	if (geglu && lutlds)
		hipLaunchKernelGGL((gemm_i8_kernel<true, true>), grid, block, 0, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin, geps, ginv,
		                   lut_size, rmp, Mpad, 1, (size_t)0);
	else if (geglu)
		hipLaunchKernelGGL((gemm_i8_kernel<true, false>), grid, block, 0, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin, geps, ginv,
		                   lut_size, rmp, Mpad, 1, (size_t)0);
	else
		hipLaunchKernelGGL((gemm_i8_kernel<false, false>), grid, block, 0, s, C, apack, rowinv, Wg, scales, M, K, ldc, lut, gmin, geps, ginv,
		                   lut_size, rmp, Mpad, ksplit, csplit);
}

// In how many parts of K (1, 2 or 4) a STORE product of M rows, K deep, ntiles column tiles should run; the parts
// write separate partial results which the consumer adds.
//   * the few-row kernel: as many parts as leave each at least 8 stages (the down projection of a 178-token prompt:
//     54 workgroups walking 6912 rows of K become 216 walking 1728);
//   * the tiled kernel: 2 when that fills the last round of workgroups noticeably better (whole pairs of stages per half).
int tg_gemm_mfma_k_parts(int M, int K, int ntiles, int n_cu) {
	const int nstage = K / KSTAGE;
	if (M <= TG_GEMM_SKINNY_ROWS && ((M + 127) / 128) * ntiles < TG_GEMM_SKINNY_BLOCKS) {
		if (nstage % 4 == 0 && nstage / 4 >= 8) return 4;
		if (nstage % 2 == 0 && nstage / 2 >= 8) return 2;
		return 1;
	}
	if (M <= TG_GEMM_SKINNY_ROWS || nstage % 4 != 0) return 1;
	if (tg_gemm_lds_taken(M, K, ntiles)) {
		// Two workgroups per compute unit.  With more tiles than compute units but well under two per unit, most units
		// would hold one workgroup and a few two, and those few set the pace: two half-K copies fill both slots of
		// every unit (halves of whole groups of four k steps).  Only for a long K: each copy has its own start-up and
		// writes its own partial result, which at K = 1024 costs more than the idle slots (output projection at 4096
		// rows: 26.5 us unsplit, 32.7 us as two copies; down projection, K = 6912: 123 -> 108 us).
		const long tiles = (long)((M + 127) / 128) * ntiles;
		const int ksteps = K >> 5;
		return (g_gemm_lds_ksplit && 4 * tiles <= 3 * 2 * (long)n_cu && ksteps % 8 == 0 && ksteps / 2 >= 32) ? 2 : 1;
	}
	const long wgs = (long)((M + 127) / 128) * ntiles;
	auto eff = [&](long n) { return (double)n / (double)(((n + n_cu - 1) / n_cu) * n_cu); };
	// measured: worth it only when the last round is nearly empty (288 workgroups on 256 compute units: -2 % prefill time);
	// at 0.75 or better the second prologue/epilogue and the extra partial result cost more than the idle units
	return (eff(wgs) < 0.6 && eff(2 * wgs) > eff(wgs) + 0.1) ? 2 : 1;
}


// tg_debug_gemm_clock: the buffer gemm_i8_lds_kernel leaves its clock readings in (n workgroups at most), and their
// evaluation: sum of shader clocks / sum of 100 MHz ticks over the workgroups that ran.
int tg_gemm_clk_begin(unsigned long long **buf, int n, hipStream_t s) {
	TG_HIP(hipMalloc((void **)buf, sizeof(unsigned long long) * 2 * (size_t)n));
	TG_HIP(hipMemsetAsync(*buf, 0, sizeof(unsigned long long) * 2 * (size_t)n, s));
	TG_HIP(hipStreamSynchronize(s));
	TG_HIP(hipMemcpyToSymbol(HIP_SYMBOL(tg_gemm_clk), buf, sizeof(*buf)));
	return TG_OK;
}
int tg_gemm_clk_end(unsigned long long *buf, int n, double *clock_mhz, double *workgroup_us, int *workgroups) {
	unsigned long long *null_ptr = nullptr;
	const hipError_t e0 = hipMemcpyToSymbol(HIP_SYMBOL(tg_gemm_clk), &null_ptr, sizeof(null_ptr));
	std::vector<unsigned long long> h(2 * (size_t)n);
	const hipError_t e1 = hipMemcpy(h.data(), buf, sizeof(unsigned long long) * h.size(), hipMemcpyDeviceToHost);
	(void)hipFree(buf);
	if (e0 != hipSuccess || e1 != hipSuccess) return tg_fail(TG_ERR_HIP, "reading the clock samples failed");
	double c = 0.0, r = 0.0;
	int k = 0;
	for (int i = 0; i < n; i++)
		if (h[2 * (size_t)i + 1] != 0) {
			c += (double)h[2 * (size_t)i];
			r += (double)h[2 * (size_t)i + 1];
			k++;
		}
	if (k == 0) return tg_fail(TG_ERR_STATE, "the product did not run on the kernel with two workgroups per compute unit (too few rows or tiles)");
	*clock_mhz = 100.0 * c / r;
	*workgroup_us = r / k / 100.0;
	*workgroups = k;
	return TG_OK;
}

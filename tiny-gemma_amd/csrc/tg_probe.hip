// Timing probes of the machine facts the design rests on.
//
// tg_debug_launch_chain, tg_debug_grid_barrier: what a dependent kernel launch costs on this part, and what a
// device-wide barrier inside one kernel costs.  A decode step is a chain of ~130 small dependent launches; the
// alternative, one resident kernel per step with a barrier wherever a launch boundary is now, only pays if the
// barrier is the cheaper of the two.
//
// tg_debug_mfma_clock: the rate the integer matrix cores really sustain.  The instruction rate is fixed (one
// v_mfma_i32_32x32x32_i8 per 32 clocks and SIMD), the clock is not: with every compute unit issuing matrix
// instructions the part runs into its power limit and lowers the shader clock, by an amount that depends on the
// operand VALUES (how many bits toggle).  The probe runs nothing but matrix instructions on operands held in
// registers (no memory traffic at all) and reports clocks per instruction and the clock itself, for operands that
// are all zero, small, or uniformly random int8: the ceiling the prefill GEMM can be measured against.
//
// tg_debug_l1_fill: the rate at which a compute unit takes data that its L1 does not hold (from its XCD's L2, or from
// memory): the bound of the prefill products on short prompts, whose workgroups pull their operands straight through
// the L1 with one wave per SIMD.
//
// Every wait in here is bounded: a workgroup that does not see the others arrive within max_spins polls gives up,
// sets a flag and goes on, so the kernel always drains.

#include "tg_internal.h"
#include <algorithm>

extern hipStream_t tg_probe_stream();  // the library's stream (tg_api.hip)
extern int tg_probe_n_cu();             // compute units of the device the library runs on

namespace {

constexpr int PNT = 256;

// One link of a dependent chain: reads what the previous launch wrote, writes what the next one reads.
__global__ __launch_bounds__(PNT) void chain_kernel(const float *in, float *out, int n) {
	const int i = blockIdx.x * PNT + threadIdx.x;
	if (i < n) out[i] = in[i] + 1.0f;
}

// rounds x (publish 64 B per workgroup, device-wide barrier, read a neighbour's 64 B).
//   FENCED = true : plain stores/loads for the data, made visible with device-scope fences (release before the
//                   arrival, acquire after the wait): what a kernel needs whose data is written by ordinary stores
//   FENCED = false: the data itself goes through device-scope atomic stores/loads (write-through, cache-bypassing),
//                   ordered before the arrival by waiting for the stores: no cache write-back/invalidate at all
template <bool FENCED>
__global__ __launch_bounds__(PNT) void grid_barrier_kernel(unsigned *counter, float *xchg, float *sink, int rounds, int max_spins,
                                                           int *timed_out) {
	const unsigned nwg = gridDim.x;
	const int tid = threadIdx.x;
	float acc = 0.0f;
	for (int r = 0; r < rounds; r++) {
		float *slot = xchg + (size_t)(r & 1) * nwg * 16;
		if (tid < 16) {
			const float v = (float)(r + (int)blockIdx.x);
			if (FENCED) slot[blockIdx.x * 16 + tid] = v;
			else __hip_atomic_store(&slot[blockIdx.x * 16 + tid], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		}
		if (!FENCED) __builtin_amdgcn_s_waitcnt(0);  // the write-through stores have left the wave's queues
		__syncthreads();
		if (tid == 0) {
			if (FENCED) __threadfence();
			__hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			const unsigned target = (unsigned)(r + 1) * nwg;
			int spins = 0;
			while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
				if (++spins >= max_spins) {  // bounded wait: give up, flag it, go on
					__hip_atomic_store(timed_out, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					break;
				}
				__builtin_amdgcn_s_sleep(1);
			}
			if (FENCED) __threadfence();
		}
		__syncthreads();
		if (tid < 16) {
			const float *src = &slot[((blockIdx.x + 1) % nwg) * 16 + tid];  // the next workgroup sits on another XCD
			acc += FENCED ? *src : __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		}
	}
	if (tid < 16) sink[blockIdx.x * 16 + tid] = acc;
}

// ---- sharded hand-over between the workgroups of one resident kernel ----------------------------------------------
// What the single-counter barrier above measures is mostly serialisation: every workgroup adds to one address and
// then every workgroup polls that same address.  handover_kernel asks what the hand-over costs when arrivals and
// polls are spread over the machine the way it is built: 8 XCDs with an L2 each, a memory side they all share.
// Barrier (BAR):
//   0  one counter, everyone polls it (the figure above, with the data volume and the check of this kernel)
//   1  an arrival counter per XCD (its own 128-byte line), the last arriver of an XCD adds to one 8-way counter, the
//      last of those writes a release flag per XCD; a workgroup polls its XCD's flag line with device-scope loads
//   2  the same tree, but a workgroup polls its XCD's flag with a returning read-modify-write (which the L2 executes;
//      a device-scope load is sent past the L2) and the XCD's last arriver polls the 8-way counter and sets the flag
//   3  no tree: an arrival counter per XCD, added to without waiting for the old value; every workgroup polls all 8
//      counters (8 lanes, one load instruction per poll)
//   4  no atomics: every workgroup stores the round number into its own word of a flag array (8 lines for 256
//      workgroups); one wave per workgroup polls the whole array, 16 bytes per lane
// Data (DATA): workgroup b publishes words_per_wg floats per round with device-scope (write-through) stores; after the
// hand-over every workgroup reads ALL nwg * words_per_wg of them
//   0  with device-scope loads (sent past the L2), from one of two alternating slots
//   1  with ordinary loads, from a slot that is used for this round only (a ring as long as the launch): a line that
//      has never been read cannot be stale in any cache, so nothing is invalidated; the 32 workgroups of an XCD
//      share one fetch through their L2
//   2  with ordinary loads from two alternating slots: the XCD's last arriver invalidates the L2 (device-scope
//      acquire) before it releases its XCD, every workgroup invalidates its L1 (BAR 2 only)
//   3  no barrier at all: every datum is an 8-byte (value, round) pair written and polled with device-scope atomics
//   4  no barrier and no tag: a slot is used for one round only and starts out filled with a NaN pattern no result
//      can have; a consumer polls the floats themselves (16-byte device-scope loads) until none of them is the pattern
// The reads of a round are all issued before the first is used (unrolled, clamped indices), as a real consumer would.
// and checks their sum against the closed form, so a stale or early read is counted, not just timed.  Which XCD a
// workgroup runs on is read from the hardware register; the number of workgroups per XCD is counted by a
// registration round (single counter) at kernel start.
constexpr int BL = 32;  // words per 128-byte line
constexpr int HO_MAX_TOTAL = 7168;            // floats published per round, upper bound (28 per thread)
constexpr unsigned HO_SENTINEL = 0xffffffffu;  // a NaN no arithmetic produces
typedef float ho_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned ho_u32x4 __attribute__((ext_vector_type(4)));
enum { HS_TOP = 0, HS_SINGLE = 1, HS_MEMBERS = 2, HS_REG = 3, HS_ARRIVE = 4, HS_FLAG = 12, HS_LINES = 20 };

#define TG_AG_ADD(p, v) __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define TG_AG_LD(p) __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define TG_AG_ST(p, v) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

__device__ __forceinline__ unsigned probe_xcc_id() {
	unsigned v;
	asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(v));
	return v & 7u;
}
// the current value of *p through a returning atomic OR of 0 (written out: the compiler turns an atomic that cannot
// change memory into a load, which an L1 may serve)
__device__ __forceinline__ unsigned probe_rmw_read(unsigned *p) {
	unsigned v;
	const unsigned zero = 0u;
	asm volatile("global_atomic_or %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p), "v"(zero) : "memory");
	return v;
}
__device__ __forceinline__ float handover_value(int r, int i) { return (float)((r * 131 + i * 7) & 255); }

// Bounded wait of one thread: false (and *flag set, `dead` latched: later waits return at once) after max_spins polls.
template <class F>
__device__ __forceinline__ bool probe_wait(F ready, int max_spins, bool &dead, int *flag) {
	if (dead) return false;
	int spins = 0;
	while (!ready()) {
		if (++spins >= max_spins) {
			dead = true;
			TG_AG_ST(flag, 1);
			return false;
		}
		__builtin_amdgcn_s_sleep(1);
	}
	return true;
}

template <int BAR, int DATA>
__global__ __launch_bounds__(PNT) void handover_kernel(unsigned *st, float *xchg, unsigned long long *xchg2, int rounds, int wpw, int max_spins,
                                                       int *flags /* [0] timed out, [1] wrong sums */, int *xcd_of_wg) {
	__shared__ unsigned s_x, s_members, s_nx;
	__shared__ unsigned s_target[8];
	const int nwg = (int)gridDim.x, tid = threadIdx.x, b = blockIdx.x, total = nwg * wpw;
	bool dead = false;
	if (tid == 0) {
		const unsigned x = probe_xcc_id();
		TG_AG_ADD(&st[HS_MEMBERS * BL + x], 1u);
		__builtin_amdgcn_s_waitcnt(0);
		TG_AG_ADD(&st[HS_REG * BL], 1u);
		probe_wait([&] { return TG_AG_LD(&st[HS_REG * BL]) >= (unsigned)nwg; }, max_spins, dead, &flags[0]);
		unsigned nx = 0;
		for (int k = 0; k < 8; k++) {
			const unsigned mk = TG_AG_LD(&st[HS_MEMBERS * BL + k]);
			s_target[k] = mk;
			nx += mk != 0u;
		}
		s_x = x;
		s_members = s_target[x];
		s_nx = nx;
		xcd_of_wg[b] = (int)x;
	}
	__syncthreads();
	const unsigned x = s_x, members = s_members, nx = s_nx;
	const unsigned my_target = s_target[tid & 7];
	int wrong = 0;
	for (int r = 0; r < rounds; r++) {
		const unsigned e = (unsigned)r + 1u;
		float *slot = xchg + (size_t)((DATA == 1 || DATA == 4) ? r : (r & 1)) * total;
		unsigned long long *slot2 = xchg2 + (size_t)(r & 1) * total;
		for (int j = tid; j < wpw; j += PNT) {
			const int i = b * wpw + j;
			const float v = handover_value(r, i);
			if (DATA == 3) __hip_atomic_store(&slot2[i], ((unsigned long long)e << 32) | __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			else TG_AG_ST(&slot[i], v);
		}
		if (DATA != 3 && DATA != 4) {
			__builtin_amdgcn_s_waitcnt(0);  // the write-through stores have been acknowledged
			__syncthreads();
			if (BAR == 3) {
				if (tid == 0) __hip_atomic_fetch_add(&st[(HS_ARRIVE + x) * BL], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				if (tid < 64) {  // lanes 0..7 poll one counter each; the wave leaves when all 8 are there
					probe_wait([&] { return __all(tid >= 8 || TG_AG_LD(&st[(HS_ARRIVE + (tid & 7)) * BL]) >= e * my_target); }, max_spins, dead, &flags[0]);
				}
			} else if (BAR == 4) {
				if (tid == 0) TG_AG_ST(&st[HS_LINES * BL + b], e);
				if (tid < 64) {
					const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(&st[HS_LINES * BL], 0, nwg * 4, 0x00020000);
					probe_wait(
					    [&] {
						    bool ok = true;
						    for (int i0 = 0; i0 < nwg; i0 += 256) {  // words past the array read as 0: counted as arrived below
							    const ho_u32x4 f = __builtin_bit_cast(ho_u32x4, __builtin_amdgcn_raw_buffer_load_b128(rf, (unsigned)(i0 + 4 * tid) * 4u, 0, 16));
#pragma unroll
							    for (int c = 0; c < 4; c++) ok = ok && (i0 + 4 * tid + c >= nwg || f[c] >= e);
						    }
						    return (bool)__all(ok);
					    },
					    max_spins, dead, &flags[0]);
				}
			} else if (tid == 0) {
				if (BAR == 0) {
					TG_AG_ADD(&st[HS_SINGLE * BL], 1u);
					probe_wait([&] { return TG_AG_LD(&st[HS_SINGLE * BL]) >= e * (unsigned)nwg; }, max_spins, dead, &flags[0]);
				} else if (BAR == 1) {
					if (TG_AG_ADD(&st[(HS_ARRIVE + x) * BL], 1u) + 1u == e * members) {
						if (TG_AG_ADD(&st[HS_TOP * BL], 1u) + 1u == e * nx)
							for (int k = 0; k < 8; k++) TG_AG_ST(&st[(HS_FLAG + k) * BL], e);
					}
					probe_wait([&] { return TG_AG_LD(&st[(HS_FLAG + x) * BL]) >= e; }, max_spins, dead, &flags[0]);
				} else {
					if (TG_AG_ADD(&st[(HS_ARRIVE + x) * BL], 1u) + 1u == e * members) {
						TG_AG_ADD(&st[HS_TOP * BL], 1u);
						probe_wait([&] { return TG_AG_LD(&st[HS_TOP * BL]) >= e * nx; }, max_spins, dead, &flags[0]);
						if (DATA == 2) asm volatile("buffer_inv sc1\n\ts_waitcnt vmcnt(0)" ::: "memory");
						__hip_atomic_fetch_max(&st[(HS_FLAG + x) * BL], e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					} else {
						probe_wait([&] { return probe_rmw_read(&st[(HS_FLAG + x) * BL]) >= e; }, max_spins, dead, &flags[0]);
					}
				}
			}
			__syncthreads();
		}
		// read everything every workgroup published this round
		float sum = 0.0f, want = 0.0f;
		constexpr int MAXV = HO_MAX_TOTAL / PNT / 4;  // 16-byte pieces per thread
		const int nvec = total >> 2;
		if (DATA == 3) {
			bool ok = false;
			probe_wait(
			    [&] {
				    ok = true;
				    sum = 0.0f;
				    for (int i = tid; i < total; i += PNT) {
					    const unsigned long long p = __hip_atomic_load(&slot2[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					    ok = ok && (unsigned)(p >> 32) == e;
					    sum += __uint_as_float((unsigned)p);
				    }
				    return ok;
			    },
			    max_spins, dead, &flags[0]);
		} else if (DATA == 0 || DATA == 4) {
			// 16-byte loads with the device-scope bit (aux bit 4 = sc1) through a buffer descriptor
			const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(slot, 0, (int)(total * 4), 0x00020000);
			auto pass = [&] {
				ho_f32x4 v[MAXV];
#pragma unroll
				for (int k = 0; k < MAXV; k++) {
					const int i = tid + k * PNT;
					v[k] = __builtin_bit_cast(ho_f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, (unsigned)(i < nvec ? i : 0) * 16u, 0, 16));
				}
				bool ok = true;
				sum = 0.0f;
#pragma unroll
				for (int k = 0; k < MAXV; k++) {
					if (tid + k * PNT < nvec) {
#pragma unroll
						for (int c = 0; c < 4; c++) {
							ok = ok && __float_as_uint(v[k][c]) != HO_SENTINEL;
							sum += v[k][c];
						}
					}
				}
				return ok;
			};
			if (DATA == 0) (void)pass();
			else probe_wait(pass, max_spins, dead, &flags[0]);
		} else {
			if (DATA == 2) asm volatile("buffer_inv sc0" ::: "memory");  // this compute unit's L1 may hold the slot's lines of two rounds ago
			else asm volatile("" ::: "memory");
			ho_f32x4 v[MAXV];
#pragma unroll
			for (int k = 0; k < MAXV; k++) {
				const int i = tid + k * PNT;
				v[k] = reinterpret_cast<const ho_f32x4 *>(slot)[i < nvec ? i : 0];
			}
#pragma unroll
			for (int k = 0; k < MAXV; k++)
				if (tid + k * PNT < nvec) sum += (v[k][0] + v[k][1]) + (v[k][2] + v[k][3]);
		}
		if (DATA == 3) {
			for (int i = tid; i < total; i += PNT) want += handover_value(r, i);
		} else {  // the 16-byte pieces tid, tid + PNT, ...
			for (int i = tid; i < nvec; i += PNT)
				for (int c = 0; c < 4; c++) want += handover_value(r, 4 * i + c);
		}
		if (sum != want) wrong++;
	}
	if (wrong) atomicAdd(&flags[1], wrong);
}

// Back-to-back matrix instructions on register operands: 12 independent accumulators (3 x 4, as in the GEMM's inner
// step), 3 A and 4 B fragments per wave filled from a hash of (workgroup, thread, fragment).  operands: 0 = zero,
// 1 = uniformly random bytes, 2 = bytes in [-6, 6].  out[2 b] = shader clocks, out[2 b + 1] = ticks of the constant
// 100 MHz counter, both around the loop of workgroup b's first thread.
__device__ __forceinline__ unsigned probe_hash(unsigned x) {
	x ^= x >> 16;
	x *= 0x7feb352du;
	x ^= x >> 15;
	x *= 0x846ca68bu;
	x ^= x >> 16;
	return x;
}
__global__ __launch_bounds__(PNT) void mfma_clock_kernel(long long *out, int *sink, int iters, int operands) {
	typedef int i32x4 __attribute__((ext_vector_type(4)));
	typedef int i32x16 __attribute__((ext_vector_type(16)));
	i32x4 frag[7];
#pragma unroll
	for (int f = 0; f < 7; f++)
#pragma unroll
		for (int e = 0; e < 4; e++) {
			const unsigned h = probe_hash((((unsigned)blockIdx.x * PNT + threadIdx.x) * 7 + f) * 4 + e + 1u);
			unsigned v = 0;
			if (operands == 1) v = h;
			if (operands == 2)
				for (int b = 0; b < 4; b++) v |= (unsigned)(((int)((h >> (8 * b)) & 0xff) % 13 - 6) & 0xff) << (8 * b);
			frag[f][e] = (int)v;
		}
	i32x16 acc[12];
#pragma unroll
	for (int i = 0; i < 12; i++)
#pragma unroll
		for (int e = 0; e < 16; e++) acc[i][e] = 0;
	__syncthreads();
	const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
	for (int it = 0; it < iters; it++) {
#pragma unroll
		for (int i = 0; i < 12; i++) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[3 + (i & 3)], frag[i >> 2], acc[i], 0, 0, 0);
	}
	const long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
	int x = 0;
#pragma unroll
	for (int i = 0; i < 12; i++)
#pragma unroll
		for (int e = 0; e < 16; e++) x ^= acc[i][e];
	if (x == 0x5a5a5a5a && iters < 0) sink[threadIdx.x] = x;  // keeps the loop alive; never taken
	if (threadIdx.x == 0) {
		out[2 * blockIdx.x] = c1 - c0;
		out[2 * blockIdx.x + 1] = r1 - r0;
	}
}

// What one compute unit can pull through its vector L1: every workgroup walks `buf` (a power of two of 16-byte
// pieces, cyclically, from a start of its own) with 16-byte loads, N x 4 KiB per step, the next step's loads issued
// before this step's are consumed.  A buffer of a megabyte stays in every XCD's L2 and never in a 32 KB L1.
template <int N>
__global__ __launch_bounds__(PNT) void l1_fill_kernel(const int4 *buf, unsigned mask, unsigned start_stride, int steps, long long *out, int *sink) {
	const unsigned tid = threadIdx.x;
	unsigned pos = blockIdx.x * start_stride + tid;
	int4 a[N], b[N];
	int x = 0;
	auto load = [&](int4 *r) {
#pragma unroll
		for (int i = 0; i < N; i++) r[i] = buf[(pos + i * PNT) & mask];
		pos += N * PNT;
	};
	auto eat = [&](const int4 *r) {
#pragma unroll
		for (int i = 0; i < N; i++) x ^= r[i].x ^ r[i].y ^ r[i].z ^ r[i].w;
	};
	__syncthreads();
	const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
	load(a);
	for (int st = 0; st < steps; st += 2) {
		load(b);
		eat(a);
		load(a);
		eat(b);
	}
	eat(a);
	const long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
	if (x == 0x5a5a5a5a && steps < 0) sink[tid] = x;  // keeps the loads alive; never taken
	if (tid == 0) {
		out[3 * blockIdx.x] = c1 - c0;
		out[3 * blockIdx.x + 1] = r0;
		out[3 * blockIdx.x + 2] = r1;
	}
}

// Which XCD every workgroup of a launch ran on (for tg_debug_xcd_deal).
__global__ __launch_bounds__(PNT) void xcd_deal_kernel(int *out) {
	if (threadIdx.x == 0) out[blockIdx.x] = (int)probe_xcc_id();
}

struct Timer {
	hipEvent_t e0 = nullptr, e1 = nullptr;
	int begin(hipStream_t s) {
		TG_HIP(hipEventCreate(&e0));
		TG_HIP(hipEventCreate(&e1));
		TG_HIP(hipEventRecord(e0, s));
		return TG_OK;
	}
	int end(hipStream_t s, double *us) {
		TG_HIP(hipEventRecord(e1, s));
		TG_HIP(hipEventSynchronize(e1));
		float ms = 0.0f;
		TG_HIP(hipEventElapsedTime(&ms, e0, e1));
		*us = 1e3 * (double)ms;
		return TG_OK;
	}
	~Timer() {
		if (e0) (void)hipEventDestroy(e0);
		if (e1) (void)hipEventDestroy(e1);
	}
};

}  // namespace

extern "C" {

int tg_debug_launch_chain(int n_launches, int workgroups, double *us_per_launch) {
	if (n_launches < 1 || workgroups < 1 || workgroups > 65536 || !us_per_launch) return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	hipStream_t s = tg_probe_stream();
	if (!s) return tg_fail(TG_ERR_STATE, "tg_init has not run");
	const int n = workgroups * PNT;
	float *buf = nullptr;
	TG_HIP(hipMalloc((void **)&buf, sizeof(float) * 2 * (size_t)n));
	int rc = TG_OK;
	auto run = [&](int launches) {
		for (int i = 0; i < launches; i++)
			hipLaunchKernelGGL(chain_kernel, dim3((unsigned)workgroups), dim3(PNT), 0, s, buf + (size_t)(i & 1) * n, buf + (size_t)((i + 1) & 1) * n, n);
	};
	if (hipMemsetAsync(buf, 0, sizeof(float) * 2 * (size_t)n, s) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemsetAsync failed");
	if (rc == TG_OK) {
		run(16);  // warm-up
		Timer t;
		rc = t.begin(s);
		if (rc == TG_OK) {
			run(n_launches);
			double us = 0.0;
			rc = t.end(s, &us);
			*us_per_launch = us / n_launches;
		}
	}
	(void)hipStreamSynchronize(s);
	if (rc == TG_OK && hipGetLastError() != hipSuccess) rc = tg_fail(TG_ERR_HIP, "launch failed");
	(void)hipFree(buf);
	return rc;
}

int tg_debug_grid_barrier(int rounds, int workgroups, int fenced, int max_spins, double *us_per_barrier, int *timed_out) {
	// the workgroups must all be resident at once (they are small: several fit a compute unit) and the kernel must end
	// in bounded time whatever happens
	if (rounds < 1 || rounds > 100000 || workgroups < 2 || workgroups > 2 * tg_probe_n_cu() || max_spins < 1 || max_spins > (1 << 22) || !us_per_barrier ||
	    !timed_out)
		return tg_fail(TG_ERR_BAD_ARG, "bad argument (workgroups <= 2 per compute unit, max_spins <= 2^22)");
	hipStream_t s = tg_probe_stream();
	if (!s) return tg_fail(TG_ERR_STATE, "tg_init has not run");
	const size_t xf = (size_t)2 * workgroups * 16, words = 2 + xf + (size_t)workgroups * 16;
	unsigned *buf = nullptr;
	TG_HIP(hipMalloc((void **)&buf, sizeof(float) * words));
	unsigned *counter = buf;
	int *flag = (int *)(buf + 1);
	float *xchg = (float *)(buf + 2), *sink = xchg + xf;
	int rc = TG_OK;
	auto run = [&](int n) {
		if (fenced) hipLaunchKernelGGL(grid_barrier_kernel<true>, dim3((unsigned)workgroups), dim3(PNT), 0, s, counter, xchg, sink, n, max_spins, flag);
		else hipLaunchKernelGGL(grid_barrier_kernel<false>, dim3((unsigned)workgroups), dim3(PNT), 0, s, counter, xchg, sink, n, max_spins, flag);
	};
	double us_few = 0.0, us_many = 0.0;
	// two launches that differ only in the number of rounds: their difference is the cost of the rounds alone
	for (int pass = 0; pass < 3 && rc == TG_OK; pass++) {  // pass 0: warm-up
		const int n = pass == 2 ? rounds + 8 : 8;
		if (hipMemsetAsync(buf, 0, sizeof(float) * words, s) != hipSuccess) {
			rc = tg_fail(TG_ERR_HIP, "hipMemsetAsync failed");
			break;
		}
		Timer t;
		rc = t.begin(s);
		if (rc != TG_OK) break;
		run(n);
		rc = t.end(s, pass == 2 ? &us_many : &us_few);
	}
	int h_flag = 0;
	if (rc == TG_OK && hipMemcpy(&h_flag, flag, sizeof(int), hipMemcpyDeviceToHost) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemcpy failed");
	(void)hipStreamSynchronize(s);
	(void)hipFree(buf);
	if (rc != TG_OK) return rc;
	*timed_out = h_flag;
	*us_per_barrier = (us_many - us_few) / rounds;
	return TG_OK;
}

int tg_debug_handover(int rounds, int workgroups, int barrier, int data, int words_per_wg, int max_spins, double *us_per_round,
                      int *timed_out, int *wrong_sums, int *xcd_of_wg) {
	if (rounds < 1 || rounds > 4096 || workgroups < 2 || workgroups > 2 * tg_probe_n_cu() || barrier < 0 || barrier > 4 || data < 0 || data > 4 || (size_t)workgroups * words_per_wg > HO_MAX_TOTAL || ((workgroups * words_per_wg) & 3) ||
	    (data == 2 && barrier != 2) || words_per_wg < 1 || words_per_wg > 64 || max_spins < 1 || max_spins > (1 << 22) || !us_per_round || !timed_out ||
	    !wrong_sums)
		return tg_fail(TG_ERR_BAD_ARG, "bad argument (rounds <= 4096, workgroups <= 2 per compute unit, workgroups * words_per_wg <= 7168 and a multiple of 4, max_spins <= 2^22, data 2 needs barrier 2)");
	hipStream_t s = tg_probe_stream();
	if (!s) return tg_fail(TG_ERR_STATE, "tg_init has not run");
	const size_t total = (size_t)workgroups * words_per_wg, nslots = (data == 1 || data == 4) ? (size_t)rounds + 8 : 2;
	const size_t head = sizeof(unsigned) * (HS_LINES * BL + 512) + 128, map_bytes = (sizeof(int) * (size_t)workgroups + 127) / 128 * 128;
	const size_t bytes = head + map_bytes + sizeof(unsigned long long) * 2 * total + sizeof(float) * nslots * total;
	unsigned char *buf = nullptr;
	TG_HIP(hipMalloc((void **)&buf, bytes));
	unsigned *st = (unsigned *)buf;
	int *flags = (int *)(st + HS_LINES * BL + 512);
	int *map = (int *)(buf + head);
	unsigned long long *xchg2 = (unsigned long long *)(buf + head + map_bytes);
	float *xchg = (float *)(xchg2 + 2 * total);
	int rc = TG_OK;
	auto run = [&](int n) {
#define TG_HO(B, D) \
	if (barrier == B && data == D) hipLaunchKernelGGL((handover_kernel<B, D>), dim3((unsigned)workgroups), dim3(PNT), 0, s, st, xchg, xchg2, n, words_per_wg, max_spins, flags, map)
		TG_HO(0, 0); TG_HO(0, 1); TG_HO(0, 3);
		TG_HO(1, 0); TG_HO(1, 1); TG_HO(1, 3);
		TG_HO(2, 0); TG_HO(2, 1); TG_HO(2, 2); TG_HO(2, 3);
		TG_HO(3, 0); TG_HO(3, 1); TG_HO(3, 3);
		TG_HO(4, 0); TG_HO(4, 1); TG_HO(0, 4);
#undef TG_HO
	};
	double us_few = 0.0, us_many = 0.0;
	int h_flags[2] = {0, 0};
	// two launches that differ only in the number of rounds: their difference is the cost of the rounds alone
	for (int pass = 0; pass < 3 && rc == TG_OK; pass++) {  // pass 0: warm-up
		const int n = pass == 2 ? rounds + 8 : 8;
		// flags are kept across the passes; the counters and the exchange buffers start from zero each time
		if (hipMemsetAsync(buf, 0, pass == 0 ? bytes : sizeof(unsigned) * (HS_LINES * BL + 512), s) != hipSuccess ||
		    hipMemsetAsync(xchg2, 0, sizeof(unsigned long long) * 2 * total, s) != hipSuccess ||
		    (data == 4 && hipMemsetAsync(xchg, 0xff, sizeof(float) * nslots * total, s) != hipSuccess)) {
			rc = tg_fail(TG_ERR_HIP, "hipMemsetAsync failed");
			break;
		}
		Timer t;
		rc = t.begin(s);
		if (rc != TG_OK) break;
		run(n);
		rc = t.end(s, pass == 2 ? &us_many : &us_few);
		if (rc == TG_OK && hipMemcpy(h_flags, flags, sizeof(h_flags), hipMemcpyDeviceToHost) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemcpy failed");
		if (h_flags[0]) break;  // a wait timed out: the workgroups may not be co-resident; do not start the long launch
	}
	if (rc == TG_OK && xcd_of_wg && hipMemcpy(xcd_of_wg, map, sizeof(int) * (size_t)workgroups, hipMemcpyDeviceToHost) != hipSuccess)
		rc = tg_fail(TG_ERR_HIP, "hipMemcpy failed");
	(void)hipStreamSynchronize(s);
	(void)hipFree(buf);
	if (rc != TG_OK) return rc;
	*timed_out = h_flags[0];
	*wrong_sums = h_flags[1];
	*us_per_round = h_flags[0] ? 0.0 : (us_many - us_few) / rounds;
	return TG_OK;
}

int tg_debug_mfma_clock(int workgroups, int iters, int operands, double *clocks_per_mfma, double *clock_mhz) {
	if (workgroups < 1 || workgroups > 4096 || iters < 1 || iters > (1 << 20) || operands < 0 || operands > 2 || !clocks_per_mfma || !clock_mhz)
		return tg_fail(TG_ERR_BAD_ARG, "bad argument");
	hipStream_t s = tg_probe_stream();
	if (!s) return tg_fail(TG_ERR_STATE, "tg_init has not run");
	long long *buf = nullptr;
	TG_HIP(hipMalloc((void **)&buf, sizeof(long long) * 2 * (size_t)workgroups + sizeof(int) * PNT));
	int *sink = (int *)(buf + 2 * (size_t)workgroups);
	int rc = TG_OK;
	// the clock settles over some hundred microseconds of load: the figures come from the last of three launches
	for (int pass = 0; pass < 3; pass++) hipLaunchKernelGGL(mfma_clock_kernel, dim3((unsigned)workgroups), dim3(PNT), 0, s, buf, sink, iters, operands);
	if (hipStreamSynchronize(s) != hipSuccess || hipGetLastError() != hipSuccess) rc = tg_fail(TG_ERR_HIP, "launch failed");
	if (rc == TG_OK) {
		std::vector<long long> h(2 * (size_t)workgroups);
		if (hipMemcpy(h.data(), buf, sizeof(long long) * h.size(), hipMemcpyDeviceToHost) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemcpy failed");
		double c = 0.0, r = 0.0;
		for (int i = 0; i < workgroups; i++) {
			c += (double)h[2 * (size_t)i];
			r += (double)h[2 * (size_t)i + 1];
		}
		if (rc == TG_OK && r <= 0.0) rc = tg_fail(TG_ERR_STATE, "the constant-rate counter did not advance");
		if (rc == TG_OK) {
			*clocks_per_mfma = c / workgroups / ((double)iters * 12.0);
			*clock_mhz = 100.0 * c / r;
		}
	}
	(void)hipFree(buf);
	return rc;
}

int tg_debug_l1_fill(int workgroups, int loads_per_step, int steps, int buf_kib, int disjoint, double *gbps_per_workgroup, double *gbps_total,
                     double *clock_mhz) {
	if (workgroups < 1 || workgroups > 4096 || (loads_per_step != 4 && loads_per_step != 8 && loads_per_step != 16) || steps < 2 || steps > (1 << 16) ||
	    (steps & 1) || buf_kib < 64 || buf_kib > (1 << 20) || (buf_kib & (buf_kib - 1)) || !gbps_per_workgroup || !gbps_total || !clock_mhz)
		return tg_fail(TG_ERR_BAD_ARG, "bad argument (loads_per_step 4, 8 or 16; steps even; buf_kib a power of two from 64 to 2^20)");
	// a launch that ends in seconds at any rate the machine reaches: at most 16 GiB read in all
	if ((unsigned long long)workgroups * (unsigned long long)(steps + 1) * (unsigned long long)loads_per_step * 4096ull > (16ull << 30))
		return tg_fail(TG_ERR_BAD_ARG, "workgroups x steps x loads_per_step x 4 KiB exceeds 16 GiB");
	hipStream_t s = tg_probe_stream();
	if (!s) return tg_fail(TG_ERR_STATE, "tg_init has not run");
	const size_t bytes = (size_t)buf_kib << 10, pieces = bytes / 16;
	char *mem = nullptr;
	TG_HIP(hipMalloc((void **)&mem, bytes + sizeof(long long) * 3 * (size_t)workgroups + sizeof(int) * PNT));
	long long *out = (long long *)(mem + bytes);
	int *sink = (int *)(out + 3 * (size_t)workgroups);
	int rc = TG_OK;
	if (hipMemsetAsync(mem, 1, bytes, s) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemsetAsync failed");
	// disjoint: every workgroup starts in a share of its own (a large buffer streamed once from memory); otherwise the
	// starts are 4 KiB x an odd number apart, so that workgroups of one compute unit never walk in step
	const unsigned stride = disjoint ? (unsigned)(pieces / (size_t)workgroups) : 37u * PNT;
	for (int pass = 0; pass < 2 && rc == TG_OK; pass++) {
		const dim3 grid((unsigned)workgroups), block(PNT);
		if (loads_per_step == 4) hipLaunchKernelGGL(l1_fill_kernel<4>, grid, block, 0, s, (const int4 *)mem, (unsigned)(pieces - 1), stride, steps, out, sink);
		if (loads_per_step == 8) hipLaunchKernelGGL(l1_fill_kernel<8>, grid, block, 0, s, (const int4 *)mem, (unsigned)(pieces - 1), stride, steps, out, sink);
		if (loads_per_step == 16) hipLaunchKernelGGL(l1_fill_kernel<16>, grid, block, 0, s, (const int4 *)mem, (unsigned)(pieces - 1), stride, steps, out, sink);
	}
	if (rc == TG_OK && (hipStreamSynchronize(s) != hipSuccess || hipGetLastError() != hipSuccess)) rc = tg_fail(TG_ERR_HIP, "launch failed");
	if (rc == TG_OK) {
		std::vector<long long> h(3 * (size_t)workgroups);
		if (hipMemcpy(h.data(), out, sizeof(long long) * h.size(), hipMemcpyDeviceToHost) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemcpy failed");
		if (rc == TG_OK) {
			const double wg_bytes = (double)(steps + 1) * loads_per_step * PNT * 16.0;
			std::vector<double> ticks((size_t)workgroups);
			long long first = h[1], last = h[2];
			double c = 0.0, r = 0.0;
			for (int i = 0; i < workgroups; i++) {
				ticks[(size_t)i] = (double)(h[3 * (size_t)i + 2] - h[3 * (size_t)i + 1]);
				first = std::min(first, h[3 * (size_t)i + 1]);
				last = std::max(last, h[3 * (size_t)i + 2]);
				c += (double)h[3 * (size_t)i];
				r += ticks[(size_t)i];
			}
			std::sort(ticks.begin(), ticks.end());
			const double med = ticks[(size_t)workgroups / 2];
			if (med <= 0.0 || last <= first) rc = tg_fail(TG_ERR_STATE, "the constant-rate counter did not advance");
			else {
				*gbps_per_workgroup = wg_bytes / (med * 10.0);  // a tick is 10 ns
				*gbps_total = wg_bytes * workgroups / ((double)(last - first) * 10.0);
				*clock_mhz = 100.0 * c / r;
			}
		}
	}
	(void)hipFree(mem);
	return rc;
}

int tg_debug_xcd_deal(int n_launches, const int *workgroups, int *first_xcd, int *out_of_order) {
	if (n_launches < 1 || n_launches > 64 || !workgroups || !first_xcd || !out_of_order) return tg_fail(TG_ERR_BAD_ARG, "bad argument (1 to 64 launches)");
	size_t total = 0;
	for (int i = 0; i < n_launches; i++) {
		if (workgroups[i] < 1 || workgroups[i] > 65536) return tg_fail(TG_ERR_BAD_ARG, "1 to 65536 workgroups per launch");
		total += (size_t)workgroups[i];
	}
	hipStream_t s = tg_probe_stream();
	if (!s) return tg_fail(TG_ERR_STATE, "tg_init has not run");
	int *buf = nullptr;
	TG_HIP(hipMalloc((void **)&buf, sizeof(int) * total));
	size_t at = 0;
	for (int i = 0; i < n_launches; i++) {  // back to back, nothing else on the stream in between
		hipLaunchKernelGGL(xcd_deal_kernel, dim3((unsigned)workgroups[i]), dim3(PNT), 0, s, buf + at);
		at += (size_t)workgroups[i];
	}
	int rc = TG_OK;
	if (hipStreamSynchronize(s) != hipSuccess || hipGetLastError() != hipSuccess) rc = tg_fail(TG_ERR_HIP, "launch failed");
	std::vector<int> h(total);
	if (rc == TG_OK && hipMemcpy(h.data(), buf, sizeof(int) * total, hipMemcpyDeviceToHost) != hipSuccess) rc = tg_fail(TG_ERR_HIP, "hipMemcpy failed");
	(void)hipFree(buf);
	if (rc != TG_OK) return rc;
	at = 0;
	for (int i = 0; i < n_launches; i++) {
		first_xcd[i] = h[at];
		int bad = 0;
		for (int b = 0; b < workgroups[i]; b++) bad += h[at + (size_t)b] != ((h[at] + b) & 7);
		out_of_order[i] = bad;
		at += (size_t)workgroups[i];
	}
	return TG_OK;
}

}  // extern "C"

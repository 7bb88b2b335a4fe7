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
// Every wait in here is bounded: a workgroup that does not see the others arrive within max_spins polls gives up,
// sets a flag and goes on, so the kernel always drains.

#include "tg_internal.h"

extern hipStream_t tg_probe_stream();  // the library's stream (tg_api.hip)

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
					*timed_out = 1;
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
	if (rounds < 1 || workgroups < 2 || workgroups > 1024 || max_spins < 1 || !us_per_barrier || !timed_out)
		return tg_fail(TG_ERR_BAD_ARG, "bad argument");
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

}  // extern "C"

/*
 * tinygemma_hip_debug — the part of libtinygemma_hip.so's C ABI that has no counterpart in the reference: process-wide
 * tuning knobs (tg_set_*), timing probes of the machine and of single kernels (tg_debug_*, tg_decode_profile), and the
 * host-side planning helpers (tg_plan_*).  Tests, the benchmark and experiments use them; a caller of the reference's
 * interface needs none of them.  Same conventions as tinygemma_hip.h (status codes, one caller thread at a time).
 */
#ifndef TINYGEMMA_HIP_DEBUG_H
#define TINYGEMMA_HIP_DEBUG_H

#include "tinygemma_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* device-to-device streaming copy kernel (bytes % 16 == 0), asynchronous: the known-size kernel
 * that hardware byte counters are calibrated against */
int tg_dev_copy(void *dst_dev, const void *src_dev, size_t bytes);
/* How tg_decode_enqueue issues greedy decode steps.  -1 (default): the library chooses, 2 for a model whose step
 * streams under 5 MB of weights per launch (the 270m shape: the device would otherwise wait for the host's launches), 0
 * for larger ones, and always 0 under a profiler.  0: plain stream launches.  1: replay of a captured step
 * whose kernels read the position from device memory and launch the largest grids their geometry can need.  2: replay
 * of a captured step of the stream path's own launches; the nodes that depend on the position (attention, its merge
 * launch, the output projection) get new parameters before every replay: 2-3 node updates per layer and step and one
 * graph launch per four steps on the host instead of 5-6 kernel launches per layer and step.  Other values: TG_ERR_BAD_ARG.
 * 1 and 2 are refused with TG_ERR_STATE while a profiler's tool library is loaded (rocprofv3's environment): a kernel trace of
 * replayed graphs ended the process.  Captured graphs are dropped whenever a tuning knob changes. */
int tg_set_graphs(int enable);
/* 1 (default): inside one tg_decode_enqueue call the first launch of a step also finishes the previous step's greedy
 * pick (second stage of the argmax, token log, counters), which saves one launch per token; 0: every step ends with
 * its own finishing launch.  Same picks either way. */
int tg_set_chain_picks(int enable);
/* every tg_set_* knob back to its default (a test that fails between a set and its restore must not leak its
 * setting into the tests after it) */
int tg_reset_knobs(void);
/* prefill GEMM: 1 (default) = int8 matrix cores on three int8 digit planes of the row-scaled activations
 * (exact integer accumulation, fp32-rounding-level accuracy),
 * 0 = the reference's exact per-element order on the vector ALUs (bit-exact with gemm::launch_qgemm, slower) */
int tg_set_gemm_mode(int mfma);
/* prefill, int8 matrix path: 1 (default) = the output and down projections run in 2 or 4 parts of K with separate
 * partial results where that keeps more compute units busy (a badly filled last round of workgroups at a few thousand
 * tokens; the long-K products of a short prompt); the following norm adds the parts.  0 = never */
int tg_set_gemm_split(int enable);
/* n > 0 (default 2): prefill products of more than 448 rows with at least n / 2 output tiles per compute unit run two workgroups per compute
 * unit with both operands staged through LDS (same bits as the other kernels); 0: one workgroup per compute unit always.
 * n + 64: the same without the two half-K copies that products filling under 3/4 of the workgroup slots otherwise run as */
int tg_set_gemm_lds(int half_tiles_per_cu);
/* launches of the int8-matrix GEMM so far, by kernel: the few-row kernel, one workgroup per tile, two workgroups per
 * compute unit (tests read them to make sure a product ran on the kernel they mean to check) */
int tg_debug_gemm_launches(long long *few_rows, long long *one_per_tile, long long *two_per_unit);
/* prefill attention: 1 (default) = 16-bit matrix cores on two fp16 or three bf16 planes of every fp32 operand (cross
 * terms summed in fp32: fp32-level accuracy at several times the fp32 matrix rate), workgroups of 32 query positions
 * once there is a 32-query tile for every eighth compute unit (about 1000 tokens on 256 compute units), else of 16; 2 = the same with 32 at any length;
 * 3 = the same with 16 at any length; 0 = fp32 matrix cores, workgroups of 16 */
int tg_set_attn_prefill_mode(int mode);
/* prefill attention, modes 1-3: the operand format of the matrix products.  1 (default) = every fp32 operand as two fp16
 * planes (x = h + l, 22 significant bits), three products per fp32 product; 0 = three bf16 planes, six products
 * (24 bits).  The fp16 form runs half the matrix instructions; its operands must lie within +-65504 (q and k are
 * RMS-normalised, p is a probability, v a projection of a normalised vector): a value outside makes the forward
 * return TG_ERR_STATE instead of a wrong result, and the bf16 form, which has fp32's range, is the way out.
 * With 1, launches that use the K/V plane images and 32-query workgroups run on 32x32x16 matrix instructions (two
 * waves per head, each with half the head dimension); 2 = two fp16 planes on the 16x16x32 kernels only.  Other values: TG_ERR_BAD_ARG. */
int tg_set_attn_prefill_format(int f16);
/* prefill attention, modes 1-3: where the planes of K and V come from.  1 (default) = for prompts of 2048
 * tokens or more a pre-pass splits the K and V rows of a layer once and stores every 32-key tile as the image of the
 * attention kernel's LDS arrays, which the attention workgroups copy straight into LDS (shorter prompts: as 0);
 * 2 = the same at any length; 0 = every workgroup splits the tiles it stages itself.  Same arithmetic, same bits. */
int tg_set_attn_prefill_planes(int mode);
/* tuning knob: a GEMV launch uses at most n workgroups, which then loop over column tiles (0: one per tile) */
int tg_set_gemv_max_blocks(int n);
/* tuning knob: extra workgroups per decode launch that pull the NEXT launch's weights out of HBM into
 * the caches while the current launch is latency bound (multiple of 8; 0 = off).  A hint only. */
int tg_set_prefetch_blocks(int n);
/* tuning knob: which launch carries which prefetch.  0 (default): the q|k|v launch touches the o matrix, attention
 * the up|gate matrix, o the down matrix, up|gate the next layer's q|k|v.  1: an alternative kept for measurement
 * (q|k|v touches o and up|gate, attention touches down). */
int tg_set_prefetch_plan(int plan);
/* tuning knob: decode attention gives a workgroup at most this many keys (multiple of 16 in 32..256, default 64) while 16
 * workgroups cover the context; longer contexts use up to 1024 workgroups of 32 keys and one extra merge launch. */
int tg_set_attn_merge_chunk(int keys);
/* Kernel classes of one decode step, in launch order per layer; the head runs once per step. */
enum { TG_KC_QKV = 0, TG_KC_ATTN, TG_KC_OPROJ, TG_KC_UPGATE, TG_KC_DOWN, TG_KC_LMHEAD, TG_KC_ARGMAX, TG_KC_COUNT };
/* Runs n_steps decode steps like tg_decode_enqueue, with a HIP event recorded on tg_stream()
 * before every launch: ms_sum[k] / launches[k] is the average event-to-event time of class k. */
int tg_decode_profile(tg_session *s, int n_steps, double *ms_sum, int *launches);
/* Re-launches the kernel of class k (layer `layer`; the head ignores it) of the NEXT decode step `repeat`
 * times on the session's current buffers, back to back, without advancing the session: for timing one
 * kernel in isolation with events on tg_stream().  The kernels are idempotent on their inputs. */
int tg_debug_repeat_kernel(tg_session *s, int kernel_class, int layer, int repeat);
/* Timing probes of the machine facts the decode design rests on; no counterpart in the reference.
 * tg_debug_launch_chain: n_launches dependent launches of a trivial kernel of `workgroups` x 256 threads (each reads what
 * the previous one wrote) on tg_stream(): *us_per_launch = what one link of such a chain costs.
 * tg_debug_grid_barrier: one resident kernel of `workgroups` workgroups (at most one per compute unit is meaningful)
 * that runs `rounds` rounds of: publish 64 bytes, device-wide barrier, read a neighbour's 64 bytes.  fenced = 1:
 * ordinary stores/loads made visible by device-scope fences; 0: the data itself moves through device-scope atomic
 * accesses and no cache is written back or invalidated.  Every wait gives up after max_spins polls (*timed_out = 1:
 * the figure is meaningless), so the kernel always ends.  max_spins <= 2^22, workgroups <= 2 per compute unit. */
int tg_debug_launch_chain(int n_launches, int workgroups, double *us_per_launch);
/* tg_debug_handover: what a hand-over between the workgroups of one resident kernel costs when arrivals and polls are
 * spread over the 8 XCDs.  Per round every workgroup publishes words_per_wg floats with write-through stores, all hand
 * over, and every workgroup reads all workgroups * words_per_wg floats and checks their sum (*wrong_sums counts
 * failures: a stale or early read).  barrier: 0 = one counter; 1 = counter per XCD -> 8-way counter -> release flag per
 * XCD; 2 = the same, flags polled with read-modify-write atomics; 3 = counter per XCD, every workgroup polls all 8 and
 * sums them; 4 = a flag word per workgroup.  data: 0 = read with device-scope loads; 1 = ordinary loads from a buffer
 * used for that round only; 2 = ordinary loads after an L2 invalidate by one workgroup per XCD (barrier 2 only; reads
 * stale data on this part, kept as a negative result); 3 = no barrier, (value, round) pairs polled in place; 4 = no
 * barrier, the floats themselves polled against a NaN pattern the buffer starts out with.  xcd_of_wg (may be NULL):
 * [workgroups], the XCD each workgroup ran on.  Limits: rounds <= 4096, workgroups <= 2 per compute unit, workgroups *
 * words_per_wg <= 7168 and a multiple of 4, max_spins <= 2^22; every wait gives up after max_spins polls. */
int tg_debug_handover(int rounds, int workgroups, int barrier, int data, int words_per_wg, int max_spins, double *us_per_round,
                      int *timed_out, int *wrong_sums, int *xcd_of_wg);
/* enable = 1: tg_decode_enqueue / tg_forward_decode run all layers of a decode step as ONE launch of resident workgroups
 * that hand over through device memory (the LM head stays a launch of its own) instead of five launches per layer.
 * Bit-identical results; off by default because it is slower on this machine (a hand-over through memory costs more
 * than a launch boundary).  gemv_workgroups: 0 = one per compute unit less the 16 attention workgroups; max_spins: polls
 * before a wait between workgroups gives up (0 = 2^20, at most 2^22).  When a wait gives up the next read-back returns
 * TG_ERR_STATE, the decode steps since the previous read-back are invalid, and the session stays on the launch path.
 * Used up to 4096 cached keys; longer contexts take the launch path by themselves. */
int tg_set_fused_decode(int enable, int gemv_workgroups, int max_spins);
/* One decode step of the session on the one-kernel path with timestamps of the 100 MHz counter: out[n_layers][24];
 * entries 0..15 of a layer: GEMV workgroup 0 at layer start, after the norms, after its Q|K|V tiles, after arriving, after
 * the wait for the attention, after the merge, after its O tiles, after arriving, after the wait, after the norms, after
 * its up|gate tiles, after arriving, after the wait, after its down tiles, after arriving, after the wait; 16..18:
 * attention workgroup 0 when it has seen Q|K|V, after its chunk, after arriving.  tg_set_fused_decode(1, ..) must be on. */
int tg_debug_fused_timestamps(tg_session *s, unsigned long long *out, int n_layers);
int tg_debug_grid_barrier(int rounds, int workgroups, int fenced, int max_spins, double *us_per_barrier, int *timed_out);

/* The rate the integer matrix cores sustain on this machine (no counterpart in the reference: measurement aid).
 * `workgroups` x 4 waves issue nothing but v_mfma_i32_32x32x32_i8 on register operands for `iters` x 12 instructions
 * each; operands: 0 = all zero, 1 = uniformly random int8, 2 = int8 in [-6, 6].  Returns the average shader clocks
 * per instruction (32 when nothing stalls) and the average shader clock in MHz during the loop, which the part
 * lowers under load depending on the operand values.  workgroups <= 4096, iters <= 2^20. */
int tg_debug_mfma_clock(int workgroups, int iters, int operands, double *clocks_per_mfma, double *clock_mhz);
/* What a compute unit can pull through its vector L1 (no counterpart in the reference: measurement aid).  `workgroups`
 * x 256 threads walk a buffer of buf_kib KiB (a power of two, 64 .. 2^20) cyclically with 16-byte loads,
 * loads_per_step (4, 8 or 16) x 4 KiB per step and workgroup, the next step requested before this one is consumed,
 * `steps` (even, <= 2^16) steps.  disjoint = 0: all walk the same buffer from different starts (1 MiB stays in every
 * XCD's L2 and never in an L1); 1: every workgroup starts in a share of its own (a large buffer: streamed from
 * memory).  Returns GB/s of the median workgroup, GB/s of the whole launch (first start to last end) and the shader
 * clock.  workgroups <= 4096, and workgroups x (steps + 1) x loads_per_step x 4 KiB <= 16 GiB (the launch ends in seconds). */
/* How the dispatcher deals workgroups to the 8 XCDs (measurement aid, no counterpart in the reference): n_launches
 * (<= 64) launches of workgroups[i] x 256 threads back to back on tg_stream().  first_xcd[i] = the XCD workgroup 0 of
 * launch i ran on, out_of_order[i] = how many of its workgroups b did not run on XCD (first_xcd[i] + b) mod 8. */
int tg_debug_xcd_deal(int n_launches, const int *workgroups, int *first_xcd, int *out_of_order);
int tg_debug_l1_fill(int workgroups, int loads_per_step, int steps, int buf_kib, int disjoint, double *gbps_per_workgroup, double *gbps_total,
                     double *clock_mhz);
/* tg_qgemm_dev (same arguments), five times back to back, with the matrix kernel that runs two workgroups per compute unit
 * reporting its own clocks (the figures are those of the last launch):
 * *clock_mhz = shader clocks / ticks of the constant 100 MHz counter, summed over the workgroups (the clock the part held
 * while the product ran: it lowers it under the power limit, more so the more operand bits toggle), *workgroup_us = the
 * average lifetime of a workgroup, *workgroups = how many reported.  TG_ERR_STATE when the product is too small for that
 * kernel. */
int tg_debug_gemm_clock(float *C_dev, const float *A_dev, const tg_qweight *w, int m, double *clock_mhz, double *workgroup_us, int *workgroups);
/* Host-side planning of a prefill, for inspection and tests; no counterpart in the reference, no GPU call.
 * tg_plan_attention_prefill: the work list of one attention layer of n_tokens on n_cu compute units, causal (window < 0)
 * or local (a query sees `window` keys before it and itself): *query_tile = query positions per workgroup; items =
 * 4 ints per workgroup {query tile, first key tile, end key tile, scratch slot or -1} (key tiles of 32 keys), heaviest
 * first, at most max_items of them written; *n_items = their number (0: the layer runs one workgroup per query tile over
 * its whole key range); *n_split = query tiles whose key range is cut and merged afterwards.
 * tg_plan_gemm_k_parts: in how many parts of K (1, 2, 4) a projection of m rows, in_dim -> out_dim, runs when the
 * consumer can add partial results (output and down projection). */
int tg_plan_attention_prefill(int n_tokens, int n_cu, int window, int *query_tile, int32_t *items, int max_items, int *n_items,
                              int *n_split);
int tg_plan_gemm_k_parts(int m, int in_dim, int out_dim, int n_cu);
/* the form tg_decode_enqueue's greedy steps take for a model of this configuration under the current tg_set_graphs
 * setting and environment: 0 stream launches, 1 or 2 the graph replays described there; -1: bad argument */
int tg_plan_decode_launch_mode(const tg_config *cfg);



#ifdef __cplusplus
}
#endif
#endif

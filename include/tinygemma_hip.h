/*
 * tinygemma_hip — C ABI of the MI355X (gfx950) implementation of tiny-gemma's int8 weight-only
 * matrix-product path and of the single-GPU forward built around it.
 *
 * Plain pointers and sizes only; no C++ or torch types.  Every entry point returns TG_OK (0) or a
 * negative TG_ERR_* code; tg_last_error() gives the message of the calling thread's last failure.
 * The reference reports the same conditions by `assert` abort or std::runtime_error; the C++
 * mirror in tiny-gemma_amd/host/ turns the codes back into those exceptions.
 *
 * This header is the contract a caller binds to.  Tuning knobs, timing probes and planning helpers (nothing a caller of
 * the reference's interface needs) are declared in tinygemma_hip_debug.h.
 *
 * Threading contract (the reference is single-threaded with no globals, transformer.hpp:167-258): the library is
 * NOT thread safe.  One caller thread at a time for the whole library: the stream, the tuning knobs (tg_set_*)
 * and the scratch of the stand-alone GEMM entry points are process-wide and unsynchronised; only the error
 * message of tg_last_error() is per thread.  One HIP stream (tg_stream()); the library owns all device memory
 * of models and sessions.  A model outlives its sessions: tg_model_load_weights* returns TG_ERR_STATE while a
 * session of the model exists, and after tg_model_destroy every call on a surviving session returns
 * TG_ERR_STATE (no kernel is launched on freed weights).  Citations are file:line in the reference checkout.
 */
#ifndef TINYGEMMA_HIP_H
#define TINYGEMMA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
	TG_OK = 0,
	TG_ERR_UNSUPPORTED_SHAPE = -1, /* static_switch.hpp:28,56: "Unsupported ROW/COL dimension" */
	TG_ERR_FILE_OPEN = -2,         /* transformer.hpp:163: "Could not open file." */
	TG_ERR_FILE_SHORT = -3,        /* the reference ignores short reads (transformer.hpp:120-160); this library does not */
	TG_ERR_BAD_ARG = -4,           /* the reference's assert()s on bs/seq/ndim (ops.hpp:622-646, decode.hpp:78-79) */
	TG_ERR_HIP = -5,               /* a HIP runtime call failed */
	TG_ERR_NO_DEVICE = -6,
	TG_ERR_STATE = -7              /* e.g. a second prefill on a used session (decode.hpp:78-79), context overflow */
};

typedef struct tg_model tg_model;
typedef struct tg_session tg_session;

/* config::Config, config.hpp:7-44 */
typedef struct {
	int hidden_size;
	int intermediate_size;
	int n_layers;
	int n_vocab;
	int n_pos;
	int n_pos_local;
	int head_dim;
	int n_head;
	int n_kv;
	float rope_theta;
	float rope_theta_local;
	int window_pattern;
} tg_config;

/* ---- library ---- */
int tg_init(int device);              /* selects the device, creates the stream; idempotent */
const char *tg_last_error(void);
const char *tg_status_string(int code);
void *tg_stream(void);                /* the hipStream_t every kernel of this library is launched on */
int tg_synchronize(void);
const char *tg_device_name(void);

/* CONFIG_MAP.at(name), config.hpp:46-48: "270m" or "1B" */
int tg_config_named(const char *name, tg_config *out);

/* ---- kernel level: host pointers in the reference's layout -------------------------------- */
/* gemv::launch_qgemv (linalg.hpp:176): C[outDim] must be zero on entry — like the reference it
 * holds C += A.B, then C *= scales.  B is [inDim][outDim] row-major int8, scales [outDim].
 * inDim/outDim outside ROW_SWITCH/COL_SWITCH (static_switch.hpp:7-58) -> TG_ERR_UNSUPPORTED_SHAPE. */
int tg_qgemv(float *C, const float *A, const int8_t *B, const float *scales, int inDim, int outDim);
/* gemv::launch_qgemv_logits (linalg.hpp:197) */
int tg_qgemv_logits(float *C, const float *A, const int8_t *B, const float *scales, int inDim, int outDim);
/* gemm::launch_qgemm (linalg.hpp:298): C[m][outDim] is overwritten. */
int tg_qgemm(float *C, const float *A, const int8_t *B, const float *scales, int m, int inDim, int outDim);
/* ops::attention_prefill (ops.hpp:377-526), host pointers in the reference's layouts: q and o [4][S][256]
 * (heads outermost, as activation [1,4,S,256]), k and v [S][256].  q is taken as it reaches the reference's
 * op: normalised and rotated, not yet scaled by 1/sqrt(256).  is_sw: keys qs - sw_context .. qs
 * (ops.hpp:437-443), else causal. */
int tg_attention_prefill(float *o, const float *q, const float *k, const float *v, int S, int is_sw, int sw_context);

/* ---- kernel level: device-resident operands (what the forward uses; for timing) ----------- */
typedef struct tg_qweight tg_qweight;
/* uploads a reference-layout matrix once (re-tiled for the GPU, values unchanged) */
int tg_qweight_create(const int8_t *B, const float *scales, int inDim, int outDim, tg_qweight **out);
void tg_qweight_destroy(tg_qweight *w);
int tg_dev_alloc(void **p, size_t bytes);
int tg_dev_free(void *p);
int tg_copy_h2d(void *dst_dev, const void *src_host, size_t bytes);
int tg_copy_d2h(void *dst_host, const void *src_dev, size_t bytes);
/* y_dev[outDim] = scales * (x_dev . W); asynchronous on tg_stream(); overwrites y_dev */
int tg_qgemv_dev(float *y_dev, const float *x_dev, const tg_qweight *w, int logits_variant);
/* C_dev[m][outDim] = scales * (A_dev[m][inDim] . W); asynchronous */
int tg_qgemm_dev(float *C_dev, const float *A_dev, const tg_qweight *w, int m);
/* No counterpart in the reference.  tg_qgemm_dev for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same kernels and the same bits, but the scratch of
 * the int8 matrix path (three int8 digit planes of the activations + row factors) is a fixed array inside the
 * library's device image instead of a buffer grown on demand.  It calls no hipMalloc / hipFree and sets nothing up:
 * tg_init must have run.  Limit: (m rounded up to a multiple of 128) * inDim <= TG_QGEMM_STATIC_MAX_ELEMS, else
 * TG_ERR_BAD_ARG.  All calls on a GPU share that one array: calls that overlap would race (the library's single
 * stream orders them); every GPU the library runs on holds the array (about 6.1 MiB) until the process ends. */
#define TG_QGEMM_STATIC_MAX_ELEMS (2 * 1024 * 1024)
int tg_qgemm_dev_static(float *C_dev, const float *A_dev, const tg_qweight *w, int m);

/* ---- model level --------------------------------------------------------------------------- */
/* gemma::Transformer(Config), transformer.hpp:33 */
int tg_model_create(const tg_config *cfg, tg_model **out);
/* gemma::read_weights, transformer.hpp:99-165: flat little-endian file, no header */
int tg_model_load_weights(tg_model *m, const char *path);
/* same bytes from memory (n must equal tg_weight_file_bytes) */
int tg_model_load_weights_mem(tg_model *m, const void *image, size_t n);
size_t tg_weight_file_bytes(const tg_config *cfg);
void tg_model_destroy(tg_model *m);

/* What gemma::generate builds before the first forward (transformer.hpp:193-202): both RoPE
 * tables, the GeLU table, the DecodeState (KV caches + counters) and the logits buffer.
 * Like the reference's forward_* the tables are parameters: pass host arrays to use the caller's
 * own (rope_*: [n_pos][head_dim] as decode::RoPE holds them, decode.hpp:107-127; gelu_table:
 * [gelu_size], ops.hpp:22-39) or NULL to have the library compute them. */
int tg_session_create(tg_model *m, const float *rope_cos, const float *rope_sin, const float *rope_sw_cos,
                      const float *rope_sw_sin, const float *gelu_table, float gelu_min, float gelu_max, int gelu_size,
                      tg_session **out);
int tg_session_reset(tg_session *s); /* empty KV caches, position 0 */
void tg_session_destroy(tg_session *s);
int tg_session_position(const tg_session *s);
/* tg_forward_prefill keeps its scratch (the reference's PrefillState, decode.hpp:281-351: a few hundred MB for a
 * 4096-token prompt) in the session for the next prefill; this frees it.  Decode needs none of it. */
int tg_session_release_workspace(tg_session *s);

/* gemma::forward_prefill (transformer.hpp:49) + ops::argmax_logits (ops.hpp:744).
 * logits (host, [n_vocab]) and argmax may each be NULL.  Needs an empty session. */
int tg_forward_prefill(tg_session *s, const int32_t *ids, int n, float *logits, int32_t *argmax);
/* gemma::forward_decode (transformer.hpp:75) + argmax */
int tg_forward_decode(tg_session *s, int32_t id, float *logits, int32_t *argmax);
/* greedy branch of gemma::generate (transformer.hpp:204-250) without tokenizer/EOS stop:
 * out_ids gets n_decode+1 ids (the first from the prefill logits); seconds are wall clock around
 * forward_prefill+argmax and around the decode loop (the tok/s definitions of gemma.cpp:53-58). */
int tg_generate_greedy(tg_session *s, const int32_t *prompt, int n_prompt, int n_decode, int32_t *out_ids,
                       double *s_prefill, double *s_decode);
/* Enqueues n_steps decode steps without host synchronisation (each step feeds the device-side
 * argmax of the previous one).  Ids are read back with tg_session_read_ids after tg_synchronize. */
int tg_decode_enqueue(tg_session *s, int n_steps);
/* ops::minp_logits (ops.hpp:762-859) on host pointers: temperature, softmax, min-p renormalisation of the
 * denominator and inverse-transform sampling with the caller's uniform number randf in [0, 1).  Like the
 * reference, tokens below the min-p cut are removed from the denominator only and can still be drawn.
 * `logits` is not modified (the reference overwrites it with the probabilities).  n_vocab must be a multiple
 * of 1024 (the reference is fixed to 262144); temp > 0. */
int tg_minp_logits(const float *logits, int n_vocab, float minp, float temp, float randf, int32_t *token_out);
/* The sampling branch of the decode loop of gemma::generate (transformer.hpp:229-235): like tg_decode_enqueue,
 * but step i draws its token with minp_logits and randf[i] (the reference takes them from std::mt19937 +
 * uniform_real_distribution<float>, transformer.hpp:170-172).  minp >= 1 selects the argmax branch, as there. */
int tg_decode_enqueue_sampled(tg_session *s, int n_steps, float minp, float temp, const float *randf);
/* Both branches of gemma::generate on token ids (transformer.hpp:166-256): prefill, first token, n_decode steps.
 * randf[n_decode + 1] (first entry: the token after the prompt) is only read when minp < 1. */
int tg_generate(tg_session *s, const int32_t *prompt, int n_prompt, int n_decode, float minp, float temp, const float *randf,
                int32_t *out_ids, double *s_prefill, double *s_decode);
/* Debug taps of tg_forward_prefill (a copy of the residual stream after every block: every row of prompts of up
 * to 1024 tokens, the last row of longer ones; read back with tg_session_tap): off by default, they cost one
 * device copy per block. */
int tg_set_taps(int enable);
int tg_session_read_ids(tg_session *s, int32_t *ids, int max_ids, int *n_out);

/* ---- block level: one modules::attention / mlp / lm_head call at a time (parity checks) ---------------------
 * The reference's unit tests drive these blocks one by one (tests/csrc/test_bench_modules.cpp:13-512) and hold
 * them to a norm-relative 1e-3.  Host pointers; x is the residual stream [rows][hidden], replaced by the block's
 * output (post-norm + residual included).  rows > 1 runs the kernels of tg_forward_prefill, rows == 1 the kernels
 * of a decode step.  The layer's weights are those of the session's model.  The position counter of a session is
 * shared by all layers, so a session driven through these entry points should be reset before a forward.
 * They invalidate the prefill taps.
 *
 * modules::attention (modules.hpp:89-169).  rows > 1: needs an empty session; afterwards the layer's cache and the
 * session's counters are those after a prefill of `rows` tokens.  rows == 1: attends to the layer's cache at the
 * session's position and advances the counters like KVCache::update_single (decode.hpp:49-70). */
int tg_block_attention(tg_session *s, int layer, float *x, int rows);
/* modules::mlp (modules.hpp:171-220) */
int tg_block_mlp(tg_session *s, int layer, float *x, int rows);
/* modules::lm_head (modules.hpp:222-247): final norm + LM head on the last row; logits (host) [n_vocab] */
int tg_block_lm_head(tg_session *s, const float *x, int rows, float *logits);
/* KVCache::update_prefill (decode.hpp:72-105) on one layer of an empty session: keys/values (host) [rows][head_dim];
 * a local layer keeps the last n_pos_local rows in slots 0..; counters as after a prefill of `rows` tokens */
int tg_session_kv_prefill(tg_session *s, int layer, const float *keys, const float *values, int rows);

/* Debug taps: the residual stream of the most recent forward after block b
 * (b = 0: embedding; 2l+1: after attention of layer l; 2l+2: after the MLP of layer l).
 * After a prefill `rows` = prompt length (1 for a prompt of more than 1024 tokens: only the last row is kept),
 * after a decode 1. out is [rows][hidden]. */
int tg_session_tap(tg_session *s, int b, float *out, int rows);
/* layer's KV cache as the reference holds it (decode.hpp:14-24): keys/values [max_pos][head_dim] */
int tg_session_kv(tg_session *s, int layer, float *keys, float *values, int *position_ptr, int *buffer_ptr, int *max_pos);

#ifdef __cplusplus
}
#endif
#endif

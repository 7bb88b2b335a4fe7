/* TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement (plain scalar C, own code) of tiny-gemma's int8 weight-only forward path.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library;
 * the HIP product path never calls it.
 *
 * File:line citations are relative to the reference checkout (csrc/include/... and py/...).
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   - tgo_qgemv / tgo_qgemv_logits / tgo_qgemm: bit-exact against the compiled reference
 *     (oracle/_ref) on seeded inputs; bit-exact against an integer closed form for
 *     integer-valued x and power-of-two scales; brute-force float64 on tiny shapes.
 *   - tgo_quantize: closed-form invariants (max|q| == 127 per column, |w - q*s| <= s/2,
 *     s == fp32(max|w|/127), ties to even) and a numpy restatement of the three-line rule.
 *   - everything else: against the compiled reference op by op and end to end, plus
 *     textbook float64 forms (softmax attention with explicit key sets, rotate-half RoPE, RMSNorm).
 *   The reference is built with -ffast-math, which lets gcc use rsqrtss/rcpps + one Newton step
 *   for 1/sqrt and vector divisions; this restatement uses correctly rounded IEEE operations
 *   there, so those ops agree with the compiled reference to a few ULP, not bit for bit.
 */
#ifndef TG_ORACLE_H
#define TG_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
	int hidden;       /* config.hpp:8  hidden_size */
	int ffn;          /* intermediate_size */
	int n_layers;
	int vocab;
	int n_pos;        /* global KV slots / RoPE table rows (32768) */
	int n_pos_local;  /* ring KV slots and sliding-window width (512) */
	int head_dim;
	int n_head;
	int n_kv;
	float theta;       /* global-layer RoPE base */
	float theta_local; /* local-layer RoPE base */
	int pattern;       /* layer l is local iff l % pattern != pattern-1 */
} tgo_config;

/* config.hpp:46-48 ("270m", "1B"); returns 0 on success */
int tgo_config_named(const char *name, tgo_config *out);

/* ---- kernels (linalg.hpp) ---- */
/* gemv::launch_qgemv, linalg.hpp:176: y must be zero on entry; row tile 8 iff out == 6912 */
int tgo_qgemv(float *y, const float *x, const int8_t *W, const float *s, int in, int out);
/* gemv::launch_qgemv_logits, linalg.hpp:197: row tile 4 */
int tgo_qgemv_logits(float *y, const float *x, const int8_t *W, const float *s, int in, int out);
/* gemm::launch_qgemm, linalg.hpp:298: overwrites C */
int tgo_qgemm(float *C, const float *A, const int8_t *B, const float *s, int m, int in, int out);
/* 1 iff d is in ROW_SWITCH / COL_SWITCH (static_switch.hpp:7-58) */
int tgo_legal_in(int d);
int tgo_legal_out(int d);

/* ---- ops (ops.hpp, decode.hpp) ---- */
void tgo_rmsnorm(float *x, const float *w, int rows, int dim);                                      /* ops.hpp:126-222 */
void tgo_rope_tables(float theta, int n_pos, int dhead, float *cos_out, float *sin_out);            /* decode.hpp:176-201 */
void tgo_rope_apply(float *x, int heads, int seq, int dhead, const float *cos_t, const float *sin_t, int offset); /* decode.hpp:136-174 */
void tgo_gelu_table(float gmin, float gmax, int size, float *table);                                /* ops.hpp:16-39 */
void tgo_gelu(float *x, size_t n, const float *table, float gmin, float gmax, int size);            /* ops.hpp:41-75 */
void tgo_embedding(float *out, const int32_t *ids, int n, const int8_t *wte, const float *scales, int hidden); /* ops.hpp:529-616 */
void tgo_attention_prefill(float *o, const float *q, const float *k, const float *v, int heads, int S, int dim, int is_sw, int sw_context); /* ops.hpp:377-526 */
void tgo_attention_decode(float *o, const float *q, const float *kc, const float *vc, int heads, int dim, int valid); /* ops.hpp:224-370 */
int tgo_argmax(const float *logits, int n);                                                         /* ops.hpp:744-760 */
/* Overwrites logits[n] (n a multiple of 32) with the probabilities the reference leaves there; returns the drawn index. */
int tgo_minp_logits(float *logits, int n, float minp, float temp, float randf);                     /* ops.hpp:762-859 */

/* ---- quantizer and weight-file producer (py/weight_handlers.py:10-20, py/gemma.py:27-77) ---- */
/* w is [rows][cols] fp32; q [rows][cols] int8; scales [cols]. Returns -1 if a column is all zero. */
int tgo_quantize(const float *w, size_t rows, size_t cols, int8_t *q, float *scales);
/* i-th draw of the seeded N(0, std) stream of tensor `tensor_id` (counter based, order independent) */
float tgo_normal(uint64_t seed, uint64_t tensor_id, uint64_t i, float std);
/* bytes of the flat weight file for cfg (transformer.hpp:99-165) */
size_t tgo_weight_file_bytes(const tgo_config *cfg);
/* Random-init N(0, 0.02) matrices (norm weights N(0, 0.1)), lm_head tied to wte^T, quantized by
 * tgo_quantize, written in the reference's file order. buf must hold tgo_weight_file_bytes(cfg). */
int tgo_generate_weights_mem(const tgo_config *cfg, uint64_t seed, void *buf);
int tgo_generate_weights_file(const tgo_config *cfg, uint64_t seed, const char *path);

/* ---- model (transformer.hpp, modules.hpp) ---- */
typedef struct tgo_model tgo_model;
typedef struct tgo_session tgo_session;

tgo_model *tgo_model_create(const tgo_config *cfg);
int tgo_model_load_file(tgo_model *m, const char *path); /* -1: cannot open; -2: short file */
int tgo_model_load_mem(tgo_model *m, const void *buf, size_t n);
void tgo_model_destroy(tgo_model *m);

/* RoPE tables, GeLU table, KV caches, position counters (transformer.hpp:193-202) */
tgo_session *tgo_session_create(tgo_model *m, float gmin, float gmax, int gsize);
void tgo_session_destroy(tgo_session *s);
/* taps (optional): residual stream after each block, [(2*l + {0 attn, 1 mlp})][S][hidden] */
int tgo_prefill(tgo_session *s, const int32_t *ids, int n, float *logits_out, int32_t *argmax_out, float *taps);
int tgo_decode(tgo_session *s, int32_t id, float *logits_out, int32_t *argmax_out, float *taps);
int tgo_kv_read(tgo_session *s, int layer, float *keys, float *values, int *position_ptr, int *buffer_ptr, int *max_pos);

#ifdef __cplusplus
}
#endif
#endif

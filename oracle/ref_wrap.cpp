// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// C-ABI wrapper around the *real* reference implementation.  This file contains no
// reference source: it #includes the reference's headers from where they lie
// (-I /root/reference/csrc/include, see oracle/Makefile) and exposes their free
// functions behind plain-C entry points so that Python tests (ctypes) can
//   1. pin oracle/tg_oracle.c against the reference on seeded inputs, and
//   2. write the golden fixtures in tests/golden/, and
//   3. time the reference's single-threaded AVX2 path as the CPU baseline.
// The output (oracle/_ref/libtg_ref.so) is git-ignored; it only exists where
// /root/reference was present at build time.
//
// Every entry point names the reference function it forwards to.

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "transformer.hpp"  // pulls in linalg/tensor/ops/decode/modules/config/tokenizer

namespace {

// The reference uses 32-byte aligned vector loads on every buffer it is handed.
template <typename T>
struct Aligned {
	T *p = nullptr;
	bool owned = false;
	size_t n = 0;
	T *src = nullptr;
	Aligned(T *in, size_t n, bool copy_in) : n(n), src(in) {
		if ((reinterpret_cast<uintptr_t>(in) & 31u) == 0) {
			p = in;
		} else {
			p = static_cast<T *>(std::aligned_alloc(32, ((n * sizeof(T) + 31) / 32) * 32));
			owned = true;
			if (copy_in) std::memcpy(p, in, n * sizeof(T));
		}
	}
	void copy_back() {
		if (owned) std::memcpy(src, p, n * sizeof(T));
	}
	~Aligned() {
		if (owned) std::free(p);
	}
};

struct RefModel {
	config::Config cfg;
	gemma::Transformer t;
	explicit RefModel(config::Config c) : cfg(c), t(c) {}
};

struct RefSession {
	RefModel *m;
	decode::RoPE rope;
	decode::RoPE rope_sw;
	lut::GeLUTable table;
	decode::DecodeState d;
	tensor::activation o;
	RefSession(RefModel *m, float gmin, float gmax, int gsize)
	    : m(m), rope(&m->cfg, false), rope_sw(&m->cfg, true), table(gmin, gmax, (size_t)gsize), d(1, &m->cfg), o(1, 1, m->cfg.n_vocab) {}
};

}  // namespace

extern "C" {

// gemv::launch_qgemv (csrc/include/linalg.hpp:176). C must be zero on entry (it accumulates).
int ref_qgemv(float *C, float *A, int8_t *B, float *scales, int inDim, int outDim) {
	try {
		Aligned<float> c(C, outDim, true), a(A, inDim, true), s(scales, outDim, true);
		Aligned<int8_t> b(B, (size_t)inDim * outDim, true);
		gemv::launch_qgemv(c.p, a.p, b.p, s.p, inDim, outDim);
		c.copy_back();
		return 0;
	} catch (const std::runtime_error &) {
		return -1;
	}
}

// gemv::launch_qgemv_logits (linalg.hpp:197)
int ref_qgemv_logits(float *C, float *A, int8_t *B, float *scales, int inDim, int outDim) {
	try {
		Aligned<float> c(C, outDim, true), a(A, inDim, true), s(scales, outDim, true);
		Aligned<int8_t> b(B, (size_t)inDim * outDim, true);
		gemv::launch_qgemv_logits(c.p, a.p, b.p, s.p, inDim, outDim);
		c.copy_back();
		return 0;
	} catch (const std::runtime_error &) {
		return -1;
	}
}

// gemm::launch_qgemm (linalg.hpp:298). Overwrites C. Its pack buffers live on the stack
// (linalg.hpp:258-259): callers with inDim=6912 must run with an unlimited stack.
int ref_qgemm(float *C, float *A, int8_t *B, float *scales, int m, int inDim, int outDim) {
	try {
		Aligned<float> c(C, (size_t)m * outDim, false), a(A, (size_t)m * inDim, true), s(scales, outDim, true);
		Aligned<int8_t> b(B, (size_t)inDim * outDim, true);
		gemm::launch_qgemm(c.p, a.p, b.p, s.p, m, inDim, outDim);
		c.copy_back();
		return 0;
	} catch (const std::runtime_error &) {
		return -1;
	}
}

// ops::rmsnorm on a [1, rows, dim] activation (ops.hpp:182)
void ref_rmsnorm(float *x, float *w, int rows, int dim) {
	tensor::activation a(1, rows, dim);
	std::memcpy(a.data.get(), x, sizeof(float) * rows * dim);
	tensor::weight<float> wt(dim);
	std::memcpy(wt.data.get(), w, sizeof(float) * dim);
	ops::rmsnorm(&a, &wt);
	std::memcpy(x, a.data.get(), sizeof(float) * rows * dim);
}

// decode::RoPE tables (decode.hpp:176-201). cos/sin are [n_pos][dhead].
void ref_rope_tables(float theta, int n_pos, int dhead, float *cos_out, float *sin_out) {
	config::Config cfg(640, 2048, 1, 262144, n_pos, 512, dhead, 4, 1, theta, theta, 6);
	decode::RoPE r(&cfg, false);
	std::memcpy(cos_out, r.freqs_cos.data.get(), sizeof(float) * n_pos * dhead);
	std::memcpy(sin_out, r.freqs_sin.data.get(), sizeof(float) * n_pos * dhead);
}

// decode::RoPE::apply_rotary_emb on a [1, heads, seq, dhead] activation (decode.hpp:136)
void ref_rope_apply(float *x, int heads, int seq, int dhead, float theta, int n_pos, int offset) {
	config::Config cfg(640, 2048, 1, 262144, n_pos, 512, dhead, 4, 1, theta, theta, 6);
	decode::RoPE r(&cfg, false);
	tensor::activation a(1, heads, seq, dhead);
	std::memcpy(a.data.get(), x, sizeof(float) * heads * seq * dhead);
	r.apply_rotary_emb(&a, offset, seq);
	std::memcpy(x, a.data.get(), sizeof(float) * heads * seq * dhead);
}

// lut::GeLUTable (ops.hpp:22-52)
void ref_gelu_table(float gmin, float gmax, int size, float *table_out) {
	lut::GeLUTable t(gmin, gmax, (size_t)size);
	std::memcpy(table_out, t.table.get(), sizeof(float) * size);
}

// ops::gelu (ops.hpp:62); n must be a multiple of 8
void ref_gelu(float *x, int n, float gmin, float gmax, int size) {
	lut::GeLUTable t(gmin, gmax, (size_t)size);
	tensor::activation a(1, 1, n);
	std::memcpy(a.data.get(), x, sizeof(float) * n);
	ops::gelu(&a, &t);
	std::memcpy(x, a.data.get(), sizeof(float) * n);
}

// ops::embedding_prefill (ops.hpp:529). wte is [n_rows][hidden]; ids index its rows.
void ref_embedding(float *out, const int *ids, int n, int8_t *wte, float *scales, int n_rows, int hidden) {
	tensor::weight<int8_t> w(n_rows, hidden, true);
	std::memcpy(w.data.get(), wte, (size_t)n_rows * hidden);
	std::memcpy(w.scales.get(), scales, sizeof(float) * hidden);
	tensor::tokens t(1, n);
	std::memcpy(t.data.get(), ids, sizeof(int) * n);
	tensor::activation o(1, n, hidden);
	ops::embedding_prefill(&o, &t, &w);
	std::memcpy(out, o.data.get(), sizeof(float) * n * hidden);
}

// ops::attention_prefill (ops.hpp:377). q,o are [heads][S][dim]; k,v are [S][dim].
void ref_attention_prefill(float *o, float *q, float *k, float *v, int heads, int S, int dim, int is_sw, int sw_context) {
	tensor::activation ao(1, heads, S, dim), aq(1, heads, S, dim), ak(1, 1, S, dim), av(1, 1, S, dim);
	std::memcpy(aq.data.get(), q, sizeof(float) * heads * S * dim);
	std::memcpy(ak.data.get(), k, sizeof(float) * S * dim);
	std::memcpy(av.data.get(), v, sizeof(float) * S * dim);
	ops::attention_prefill(&ao, &aq, &ak, &av, is_sw != 0, sw_context);
	std::memcpy(o, ao.data.get(), sizeof(float) * heads * S * dim);
}

// ops::attention_decode (ops.hpp:224) over the first `valid` slots of a cache of `max_pos` slots.
// q,o are [heads][dim]; kc, vc are [max_pos][dim].
void ref_attention_decode(float *o, float *q, float *kc, float *vc, int heads, int dim, int max_pos, int valid) {
	config::Config cfg(640, 2048, 1, 262144, max_pos, max_pos, dim, heads, 1, 1e6f, 1e4f, 6);
	decode::KVCache kv(1, &cfg, false);
	std::memcpy(kv.keys.data.get(), kc, sizeof(float) * max_pos * dim);
	std::memcpy(kv.values.data.get(), vc, sizeof(float) * max_pos * dim);
	kv.position_ptr = valid;
	kv.buffer_ptr = valid;
	tensor::activation ao(1, heads, 1, dim), aq(1, heads, 1, dim);
	std::memcpy(aq.data.get(), q, sizeof(float) * heads * dim);
	ops::attention_decode(&ao, &aq, &kv);
	std::memcpy(o, ao.data.get(), sizeof(float) * heads * dim);
}

// ops::argmax_logits (ops.hpp:744); logits has constants::vocab entries.
int ref_argmax(float *logits) {
	tensor::activation o(1, 1, constants::vocab);
	std::memcpy(o.data.get(), logits, sizeof(float) * constants::vocab);
	tensor::tokens t(1, 1);
	ops::argmax_logits(&t, &o);
	return t.data[0];
}

// ops::minp_logits (ops.hpp:762); logits has constants::vocab entries and is overwritten with the
// probabilities the reference leaves in it.
int ref_minp_logits(float *logits, float minp, float temp, float randf) {
	tensor::activation o(1, 1, constants::vocab);
	std::memcpy(o.data.get(), logits, sizeof(float) * constants::vocab);
	tensor::tokens t(1, 1);
	ops::minp_logits(&t, &o, minp, temp, randf);
	std::memcpy(logits, o.data.get(), sizeof(float) * constants::vocab);
	return t.data[0];
}

// gemma::Transformer(Config) (transformer.hpp:33)
void *ref_model_create(int hidden, int ffn, int layers, int vocab, int n_pos, int n_pos_local, int head_dim, int n_head,
                       int n_kv, float theta, float theta_local, int pattern) {
	config::Config cfg(hidden, ffn, layers, vocab, n_pos, n_pos_local, head_dim, n_head, n_kv, theta, theta_local, pattern);
	return new RefModel(cfg);
}

// gemma::read_weights (transformer.hpp:99)
int ref_model_load(void *model, const char *path) {
	try {
		gemma::read_weights(&static_cast<RefModel *>(model)->t, path);
		return 0;
	} catch (const std::runtime_error &) {
		return -1;
	}
}

void ref_model_destroy(void *model) { delete static_cast<RefModel *>(model); }

// What gemma::generate sets up before the first forward (transformer.hpp:193-202):
// both RoPE tables, the GeLU table, the DecodeState and the logits buffer.
void *ref_session_create(void *model, float gmin, float gmax, int gsize) {
	return new RefSession(static_cast<RefModel *>(model), gmin, gmax, gsize);
}

void ref_session_destroy(void *s) { delete static_cast<RefSession *>(s); }

// gemma::forward_prefill (transformer.hpp:49) + ops::argmax_logits.
// With taps != NULL the layer loop is driven from here through the same
// modules::attention / modules::mlp / modules::lm_head calls, copying the residual
// stream [S][hidden] after every block into taps[(2*l + {0: attention, 1: mlp})][S][hidden].
int ref_prefill(void *sp, const int *ids, int n, float *logits_out, int *argmax_out, float *taps) {
	RefSession *s = static_cast<RefSession *>(sp);
	gemma::Transformer *t = &s->m->t;
	tensor::tokens toks(1, n);
	std::memcpy(toks.data.get(), ids, sizeof(int) * n);
	if (taps == nullptr) {
		gemma::forward_prefill(&s->o, &toks, t, &s->d, &s->rope, &s->rope_sw, &s->table);
	} else {
		const int hidden = t->cfg.hidden_size;
		decode::PrefillState pf(1, n, &(t->cfg));
		ops::embedding_prefill(&(pf.xact), &toks, &(t->wte));
		for (int l = 0; l < t->cfg.n_layers; l++) {
			decode::RoPE *r = t->layers[l].attn.is_sw ? &s->rope_sw : &s->rope;
			modules::attention(&(pf.xact), &(t->layers)[l].attn, &s->d, &(s->d.kvcache[l]), &pf, r);
			std::memcpy(taps + (size_t)(2 * l) * n * hidden, pf.xact.data.get(), sizeof(float) * n * hidden);
			modules::mlp(&(pf.xact), &(t->layers)[l].mlp, &s->d, &pf, &s->table);
			std::memcpy(taps + (size_t)(2 * l + 1) * n * hidden, pf.xact.data.get(), sizeof(float) * n * hidden);
		}
		modules::lm_head(&s->o, &(pf.xact), &(t->lm_head), &(t->RMSw));
	}
	if (logits_out) std::memcpy(logits_out, s->o.data.get(), sizeof(float) * t->cfg.n_vocab);
	if (argmax_out) {
		tensor::tokens a(1, 1);
		ops::argmax_logits(&a, &s->o);
		*argmax_out = a.data[0];
	}
	return 0;
}

// gemma::forward_decode (transformer.hpp:75) + ops::argmax_logits; taps as above with S = 1.
int ref_decode(void *sp, int id, float *logits_out, int *argmax_out, float *taps) {
	RefSession *s = static_cast<RefSession *>(sp);
	gemma::Transformer *t = &s->m->t;
	tensor::tokens toks(1, 1);
	toks.data[0] = id;
	if (taps == nullptr) {
		gemma::forward_decode(&s->o, &toks, t, &s->d, &s->rope, &s->rope_sw, 0, &s->table);
	} else {
		const int hidden = t->cfg.hidden_size;
		decode::DecodeState *d = &s->d;
		ops::embedding_decode(&(d->xact), &toks, &(t->wte), 0);
		for (int l = 0; l < t->cfg.n_layers; l++) {
			decode::RoPE *r = t->layers[l].attn.is_sw ? &s->rope_sw : &s->rope;
			modules::attention(&(d->xact), &(t->layers)[l].attn, d, &(d->kvcache[l]), nullptr, r);
			std::memcpy(taps + (size_t)(2 * l) * hidden, d->xact.data.get(), sizeof(float) * hidden);
			modules::mlp(&(d->xact), &(t->layers)[l].mlp, d, nullptr, &s->table);
			std::memcpy(taps + (size_t)(2 * l + 1) * hidden, d->xact.data.get(), sizeof(float) * hidden);
		}
		modules::lm_head(&s->o, &(d->xact), &(t->lm_head), &(t->RMSw));
	}
	if (logits_out) std::memcpy(logits_out, s->o.data.get(), sizeof(float) * t->cfg.n_vocab);
	if (argmax_out) {
		tensor::tokens a(1, 1);
		ops::argmax_logits(&a, &s->o);
		*argmax_out = a.data[0];
	}
	return 0;
}

// Copies layer l's KV cache (decode.hpp:14-24) out: keys/values [max_pos][head_dim], and its two counters.
int ref_kv_read(void *sp, int layer, float *keys, float *values, int *position_ptr, int *buffer_ptr, int *max_pos) {
	RefSession *s = static_cast<RefSession *>(sp);
	decode::KVCache *kv = &s->d.kvcache[layer];
	size_t n = (size_t)kv->max_pos * kv->head_dim;
	if (keys) std::memcpy(keys, kv->keys.data.get(), sizeof(float) * n);
	if (values) std::memcpy(values, kv->values.data.get(), sizeof(float) * n);
	if (position_ptr) *position_ptr = kv->position_ptr;
	if (buffer_ptr) *buffer_ptr = kv->buffer_ptr;
	if (max_pos) *max_pos = kv->max_pos;
	return 0;
}

// ---- one block at a time, the way the reference's own unit tests drive them (tests/csrc/test_bench_modules.cpp) ----
// modules::attention (modules.hpp:89-169) of layer `layer` on the residual stream x [rows][hidden], in place.
// rows > 1: prefill branch (fills the layer's cache from position 0); rows == 1: decode branch at the cache's position.
int ref_block_attention(void *sp, int layer, float *x, int rows) {
	RefSession *s = static_cast<RefSession *>(sp);
	gemma::Transformer *t = &s->m->t;
	const int hidden = t->cfg.hidden_size;
	tensor::activation act(1, rows, hidden);
	std::memcpy(act.data.get(), x, sizeof(float) * rows * hidden);
	decode::RoPE *r = t->layers[layer].attn.is_sw ? &s->rope_sw : &s->rope;
	if (rows > 1) {
		decode::PrefillState pf(1, rows, &(t->cfg));
		modules::attention(&act, &(t->layers)[layer].attn, &s->d, &(s->d.kvcache[layer]), &pf, r);
	} else {
		modules::attention(&act, &(t->layers)[layer].attn, &s->d, &(s->d.kvcache[layer]), nullptr, r);
	}
	std::memcpy(x, act.data.get(), sizeof(float) * rows * hidden);
	return 0;
}

// modules::mlp (modules.hpp:171-220) of layer `layer` on x [rows][hidden], in place
int ref_block_mlp(void *sp, int layer, float *x, int rows) {
	RefSession *s = static_cast<RefSession *>(sp);
	gemma::Transformer *t = &s->m->t;
	const int hidden = t->cfg.hidden_size;
	tensor::activation act(1, rows, hidden);
	std::memcpy(act.data.get(), x, sizeof(float) * rows * hidden);
	if (rows > 1) {
		decode::PrefillState pf(1, rows, &(t->cfg));
		modules::mlp(&act, &(t->layers)[layer].mlp, &s->d, &pf, &s->table);
	} else {
		modules::mlp(&act, &(t->layers)[layer].mlp, &s->d, nullptr, &s->table);
	}
	std::memcpy(x, act.data.get(), sizeof(float) * rows * hidden);
	return 0;
}

// modules::lm_head (modules.hpp:222-247) on x [rows][hidden]: logits [n_vocab] of the last row
int ref_block_lm_head(void *sp, const float *x, int rows, float *logits) {
	RefSession *s = static_cast<RefSession *>(sp);
	gemma::Transformer *t = &s->m->t;
	const int hidden = t->cfg.hidden_size;
	tensor::activation act(1, rows, hidden);
	std::memcpy(act.data.get(), x, sizeof(float) * rows * hidden);
	modules::lm_head(&s->o, &act, &(t->lm_head), &(t->RMSw));
	std::memcpy(logits, s->o.data.get(), sizeof(float) * t->cfg.n_vocab);
	return 0;
}

// KVCache::update_prefill (decode.hpp:72-105) on one layer's empty cache: keys/values [rows][head_dim]
int ref_kv_prefill(void *sp, int layer, const float *keys, const float *values, int rows) {
	RefSession *s = static_cast<RefSession *>(sp);
	const int hd = s->m->t.cfg.head_dim;
	tensor::activation k(1, 1, rows, hd), v(1, 1, rows, hd);
	std::memcpy(k.data.get(), keys, sizeof(float) * rows * hd);
	std::memcpy(v.data.get(), values, sizeof(float) * rows * hd);
	s->d.kvcache[layer].update_prefill(&k, &v);
	return 0;
}

// ---- sentencepiece::Tokenizer (tokenizer.hpp:14-239) ----
void *ref_tok_create(const char *path, int bos_id, int eos_id, int vocab_size, int chat_format) {
	try {
		return new sentencepiece::Tokenizer(path, bos_id, eos_id, vocab_size, chat_format != 0);
	} catch (const std::exception &) {
		return nullptr;
	}
}
void ref_tok_destroy(void *tp) { delete static_cast<sentencepiece::Tokenizer *>(tp); }
// Tokenizer::encode (tokenizer.hpp:113-201); text is n bytes (may hold any byte but is passed on as a std::string).
// Returns the number of ids; writes at most cap of them.
int ref_tok_encode(void *tp, const char *text, int n, int *ids, int cap) {
	std::vector<int> v = static_cast<sentencepiece::Tokenizer *>(tp)->encode(std::string(text, (size_t)n));
	for (int i = 0; i < (int)v.size() && i < cap; i++) ids[i] = v[i];
	return (int)v.size();
}
// Tokenizer::decode(token, prev_token) (tokenizer.hpp:203-218).  Returns the piece length; writes at most cap bytes.
// -2: the reference threw std::invalid_argument, -3: another exception.
int ref_tok_decode_piece(void *tp, int token, int prev_token, char *out, int cap) {
	try {
		std::string piece = static_cast<sentencepiece::Tokenizer *>(tp)->decode(token, prev_token);
		std::memcpy(out, piece.data(), std::min((size_t)cap, piece.size()));
		return (int)piece.size();
	} catch (const std::invalid_argument &) {
		return -2;
	} catch (const std::exception &) {
		return -3;
	}
}
// Tokenizer::decode(tokens) (tokenizer.hpp:220-233)
int ref_tok_decode(void *tp, const int *ids, int n, char *out, int cap) {
	try {
		std::string text = static_cast<sentencepiece::Tokenizer *>(tp)->decode(std::vector<int>(ids, ids + n));
		std::memcpy(out, text.data(), std::min((size_t)cap, text.size()));
		return (int)text.size();
	} catch (const std::invalid_argument &) {
		return -2;
	} catch (const std::exception &) {
		return -3;
	}
}

}  // extern "C"

// C++20 host-side mirror of the reference's interface for the int8 path, over the C ABI of
// include/tinygemma_hip.h.  Same namespaces, function names, argument order and meaning, ownership
// and error behaviour as the reference's headers, so that a call site written against
// csrc/include/{linalg,ops,decode,transformer}.hpp compiles against this header and runs on the GPU:
//
//   gemv::launch_qgemv / launch_qgemv_logits      linalg.hpp:176, 197
//   gemm::launch_qgemm                            linalg.hpp:298
//   config::Config, CONFIG_MAP                    config.hpp:7-48
//   tensor::activation, tensor::tokens            tensor.hpp:57-142   (host buffers, caller owned)
//   lut::GeLUTable                                ops.hpp:22-52       (a parameter of forward_*)
//   decode::RoPE, decode::DecodeState             decode.hpp:107-276
//   gemma::Transformer, read_weights,
//   gemma::forward_prefill, forward_decode        transformer.hpp:22-165
//   ops::argmax_logits, ops::minp_logits          ops.hpp:744, 762
//   gemma::generate_greedy, gemma::generate_ids   transformer.hpp:167-258 on token ids (argmax / min-p branch)
//   gemma::generate                               transformer.hpp:167-258 on text, streaming (with tokenizer.hpp)
//   sentencepiece::Tokenizer                      tokenizer.hpp:14-239 (in host/tokenizer.hpp)
//
// Errors: the reference throws std::runtime_error for an unknown dimension ("Unsupported ROW/COL
// dimension: N") and an unopenable weight file ("Could not open file."), and assert()s on shape
// mistakes; here every failing C-ABI status becomes a std::runtime_error with the library's message.
// Single caller thread, like the reference.
#pragma once

#include <cmath>
#include <cstdint>
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <memory>
#include <random>
#include <stdexcept>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "../../include/tinygemma_hip.h"
#include "tokenizer.hpp"

namespace tinygemma {

inline void check(int rc) {
	if (rc != TG_OK) throw std::runtime_error(tg_last_error());
}

namespace constants {
static constexpr size_t vocab{262144};
static constexpr int bos_id{2};
static constexpr int eos_id{1};
}  // namespace constants

namespace config {
struct Config {
	int hidden_size, intermediate_size, n_layers, n_vocab, n_pos, n_pos_local, head_dim, n_head, n_kv;
	float rope_theta, rope_theta_local;
	int window_pattern;
	Config(int hidden_size, int intermediate_size, int n_layers, int n_vocab, int n_pos, int n_pos_local, int head_dim, int n_head,
	       int n_kv, float theta, float theta_local, int window_pattern)
	    : hidden_size(hidden_size), intermediate_size(intermediate_size), n_layers(n_layers), n_vocab(n_vocab), n_pos(n_pos),
	      n_pos_local(n_pos_local), head_dim(head_dim), n_head(n_head), n_kv(n_kv), rope_theta(theta), rope_theta_local(theta_local),
	      window_pattern(window_pattern) {}
	tg_config c_struct() const {
		return tg_config{hidden_size, intermediate_size, n_layers, n_vocab, n_pos, n_pos_local, head_dim, n_head, n_kv,
		                 rope_theta, rope_theta_local, window_pattern};
	}
};
inline const std::unordered_map<std::string, Config> CONFIG_MAP = {
    {"270m", Config(640, 2048, 18, 262144, 32768, 512, 256, 4, 1, 1000000, 10000, 6)},
    {"1B", Config(1152, 6912, 26, 262144, 32768, 512, 256, 4, 1, 1000000, 10000, 6)}};
}  // namespace config

namespace gemv {
// C must be zero on entry: C += A.B, then C *= scales.  B is [inDim][outDim] row-major.
inline void launch_qgemv(float *C, float *A, int8_t *B, float *scales, int inDim, int outDim) {
	check(tg_qgemv(C, A, B, scales, inDim, outDim));
}
inline void launch_qgemv_logits(float *C, float *A, int8_t *B, float *scales, int inDim, int outDim) {
	check(tg_qgemv_logits(C, A, B, scales, inDim, outDim));
}
}  // namespace gemv

namespace gemm {
// C[m][outDim] is overwritten.
inline void launch_qgemm(float *C, float *A, int8_t *B, float *scales, int m, int inDim, int outDim) {
	check(tg_qgemm(C, A, B, scales, m, inDim, outDim));
}
}  // namespace gemm

namespace tensor {
struct activation {  // 3-D host activation [x][y][z]
	std::vector<float> data;
	size_t x = 0, y = 0, z = 0, ndim = 3;
	activation() = default;
	activation(size_t x, size_t y, size_t z) : data(x * y * z, 0.0f), x(x), y(y), z(z) {}
	size_t numel() const { return x * y * z; }
	void zero() { std::fill(data.begin(), data.end(), 0.0f); }
};
struct tokens {  // [BS][SEQ]
	std::vector<int> data;
	size_t x = 0, y = 0;
	tokens() = default;
	tokens(size_t x, size_t y) : data(x * y, 0), x(x), y(y) {}
	size_t numel() const { return x * y; }
};
}  // namespace tensor

namespace lut {
struct GeLUTable {
	float min, max;
	size_t table_size;
	std::vector<float> table;
	float eps;
	GeLUTable(float min, float max, size_t table_size) : min(min), max(max), table_size(table_size), table(table_size) {
		eps = (float)(max - min) / float(table_size);
		const float c0 = 0.7978845608f, c1 = 0.044715f;
		for (size_t i = 0; i < table_size; i++) {
			const double a = (double)(min + (float)i * eps);
			table[i] = (float)((0.5 * a) * (1.0 + std::tanh((double)c0 * (a + (double)c1 * (a * a * a)))));
		}
	}
};
}  // namespace lut

namespace decode {
struct RoPE {  // cos/sin [max_pos][dhead], both halves equal
	std::vector<float> freqs_cos, freqs_sin;
	int dhead, max_pos;
	float theta;
	RoPE(config::Config *cfg, bool is_sw) : dhead(cfg->head_dim), max_pos(cfg->n_pos), theta(is_sw ? cfg->rope_theta_local : cfg->rope_theta) {
		freqs_cos.resize((size_t)max_pos * dhead);
		freqs_sin.resize((size_t)max_pos * dhead);
		const int dhalf = dhead / 2;
		std::vector<float> freqs((size_t)dhalf);
		for (int i = 0; i < dhalf; i++) freqs[(size_t)i] = 1.0f / std::pow(theta, float(2 * i) / float(dhead));
		for (int p = 0; p < max_pos; p++)
			for (int d = 0; d < dhalf; d++) {
				const float outer = (float)p * freqs[(size_t)d];
				const size_t i = (size_t)p * dhead + d;
				freqs_cos[i] = freqs_cos[i + dhalf] = std::cos(outer);
				freqs_sin[i] = freqs_sin[i + dhalf] = std::sin(outer);
			}
	}
};

// KV caches and counters live on the GPU inside a tg_session; it is created at the first forward,
// when the tables it should use are known (the reference passes them to every forward_* call).
struct DecodeState {
	int batch;
	config::Config cfg;
	tg_session *session = nullptr;
	const RoPE *bound_r = nullptr, *bound_r_sw = nullptr;
	const lut::GeLUTable *bound_table = nullptr;
	DecodeState(int batch, config::Config *cfg) : batch(batch), cfg(*cfg) {
		if (batch != 1) throw std::runtime_error("batch must be 1");
	}
	DecodeState(const DecodeState &) = delete;
	DecodeState &operator=(const DecodeState &) = delete;
	~DecodeState() { tg_session_destroy(session); }
	int position() const { return session ? tg_session_position(session) : 0; }
};
}  // namespace decode

namespace gemma {
struct Transformer {
	config::Config cfg;
	tg_model *model = nullptr;
	explicit Transformer(config::Config cfg) : cfg(cfg) {
		tg_config c = cfg.c_struct();
		check(tg_model_create(&c, &model));
	}
	Transformer(const Transformer &) = delete;
	Transformer &operator=(const Transformer &) = delete;
	~Transformer() { tg_model_destroy(model); }
};

inline void read_weights(Transformer *t, const char *file) { check(tg_model_load_weights(t->model, file)); }

inline void bind_session(Transformer *t, decode::DecodeState *d, decode::RoPE *r, decode::RoPE *r_sw, lut::GeLUTable *table) {
	if (d->session) {
		if (d->bound_r != r || d->bound_r_sw != r_sw || d->bound_table != table)
			throw std::runtime_error("a DecodeState keeps the tables of its first forward");
		return;
	}
	check(tg_session_create(t->model, r->freqs_cos.data(), r->freqs_sin.data(), r_sw->freqs_cos.data(), r_sw->freqs_sin.data(),
	                        table->table.data(), table->min, table->max, (int)table->table_size, &d->session));
	d->bound_r = r;
	d->bound_r_sw = r_sw;
	d->bound_table = table;
}

// o: [1][1][n_vocab] logits of the last position; toks: [1][S]
inline void forward_prefill(tensor::activation *o, tensor::tokens *toks, Transformer *t, decode::DecodeState *d, decode::RoPE *r,
                            decode::RoPE *r_sw, lut::GeLUTable *table) {
	if (o->ndim != 3 || toks->x != 1 || o->numel() != (size_t)t->cfg.n_vocab) throw std::runtime_error("forward_prefill: bad shapes");
	bind_session(t, d, r, r_sw, table);
	check(tg_forward_prefill(d->session, toks->data.data(), (int)toks->y, o->data.data(), nullptr));
}

// pos_offset is accepted and ignored, as in the reference (ops.hpp:574)
inline void forward_decode(tensor::activation *o, tensor::tokens *toks, Transformer *t, decode::DecodeState *d, decode::RoPE *r,
                           decode::RoPE *r_sw, size_t pos_offset, lut::GeLUTable *table) {
	(void)pos_offset;
	if (o->ndim != 3 || toks->x != 1 || toks->y != 1 || o->numel() != (size_t)t->cfg.n_vocab)
		throw std::runtime_error("forward_decode: bad shapes");
	bind_session(t, d, r, r_sw, table);
	check(tg_forward_decode(d->session, toks->data[0], o->data.data(), nullptr));
}

// {n_generated, ids (n_generated + 1, the first from the prefill logits), s_prefill, s_decode}
inline std::tuple<int, std::vector<int>, float, float> generate_greedy(const std::vector<int> &prompt, int n_decode, Transformer *t) {
	decode::RoPE rope(&t->cfg, false), rope_sw(&t->cfg, true);
	lut::GeLUTable table{-4.0, 4.0, 1024};  // transformer.hpp:197
	decode::DecodeState d(1, &t->cfg);
	bind_session(t, &d, &rope, &rope_sw, &table);
	std::vector<int> ids((size_t)n_decode + 1);
	double sp = 0, sd = 0;
	check(tg_generate_greedy(d.session, prompt.data(), (int)prompt.size(), n_decode, ids.data(), &sp, &sd));
	return {n_decode, ids, (float)sp, (float)sd};
}

// Both branches of gemma::generate on token ids: minp < 1 draws every token with ops::minp_logits and uniform
// numbers from `gen` in the reference's order (one per produced token, transformer.hpp:170-172, 208-211, 232-235);
// the reference seeds its std::mt19937 from std::random_device, here the caller owns the generator.
inline std::tuple<int, std::vector<int>, float, float> generate_ids(const std::vector<int> &prompt, int n_decode, Transformer *t,
                                                                    const float minp, const float temp, std::mt19937 &gen) {
	if (!(minp < 1)) return generate_greedy(prompt, n_decode, t);
	std::uniform_real_distribution<float> unif(0.0, 1.0);
	std::vector<float> randf((size_t)n_decode + 1);
	for (float &r : randf) r = unif(gen);
	decode::RoPE rope(&t->cfg, false), rope_sw(&t->cfg, true);
	lut::GeLUTable table{-4.0, 4.0, 1024};  // transformer.hpp:197
	decode::DecodeState d(1, &t->cfg);
	bind_session(t, &d, &rope, &rope_sw, &table);
	std::vector<int> ids((size_t)n_decode + 1);
	double sp = 0, sd = 0;
	check(tg_generate(d.session, prompt.data(), (int)prompt.size(), n_decode, minp, temp, randf.data(), ids.data(), &sp, &sd));
	return {n_decode, ids, (float)sp, (float)sd};
}

// gemma::generate (transformer.hpp:167-258): tokenize, print the prompt, prefill, then up to n_decode steps, every
// token printed as it is produced; returns {decode steps completed, generated text, prefill seconds, decode seconds}
// with the reference's timing boundaries (tokenizing and the first token belong to the prefill time).  minp >= 1 is
// greedy, else every token is drawn with ops::minp_logits and a uniform number from a std::mt19937 seeded from
// std::random_device, as in the reference.  The decode loop runs on the device in bursts of `burst` tokens (the ids
// come back once per burst, so text appears burst by burst; 1 = token by token); with terminate_on_end the text
// stops before the first <end_of_turn> and the count is that of the steps before it, as in the reference.
// Where the reference's tokenizer throws on a byte token (see tokenizer.hpp) the byte itself is printed.
inline std::tuple<int, std::string, float, float> generate(std::string prompt, int n_decode, sentencepiece::Tokenizer *tokenizer,
                                                           Transformer *t, const float minp, const float temp,
                                                           const bool terminate_on_end, int burst = 16) {
	using clk = std::chrono::high_resolution_clock;
	auto t_prefill_s = clk::now();
	std::random_device rd;
	std::mt19937 gen(rd());
	std::uniform_real_distribution<float> unif(0.0, 1.0);
	const bool sampling = minp < 1;

	std::vector<int> ids = tokenizer->encode(prompt);
	const size_t prompt_len = ids.size();
	std::string decoded;
	decoded.reserve((size_t)std::max(n_decode, 0));
	printf("Prompt length: %lu\n", (unsigned long)prompt_len);
	std::cout << tokenizer->decode(ids);

	auto piece_of = [&](int token, int prev) -> std::string {
		try {
			return tokenizer->decode(token, prev);
		} catch (const std::invalid_argument &) {
			const int b = tokenizer->byte_of(token);
			return b >= 0 ? std::string(1, (char)b) : std::string();
		}
	};

	decode::RoPE rope(&t->cfg, false), rope_sw(&t->cfg, true);
	lut::GeLUTable table{-4.0, 4.0, 1024};  // transformer.hpp:197
	decode::DecodeState d(1, &t->cfg);
	bind_session(t, &d, &rope, &rope_sw, &table);

	std::vector<float> randf((size_t)std::max(n_decode, 0) + 1, 0.0f);
	if (sampling)
		for (float &r : randf) r = unif(gen);
	std::vector<int> out((size_t)std::max(n_decode, 0) + 1);
	// prefill and the first token (from the prefill logits)
	check(tg_generate(d.session, ids.data(), (int)prompt_len, 0, minp, temp, randf.data(), out.data(), nullptr, nullptr));
	int prev_token = ids[ids.size() - 1];
	std::cout << piece_of(out[0], prev_token) << std::flush;
	prev_token = out[0];
	auto t_prefill_e = clk::now();

	auto t_decode_s = clk::now();
	int done = 0;
	bool stop = false;
	if (burst < 1) burst = 1;
	while (done < n_decode && !stop) {
		const int n = std::min(burst, n_decode - done);
		if (sampling) check(tg_decode_enqueue_sampled(d.session, n, minp, temp, randf.data() + 1 + done));
		else check(tg_decode_enqueue(d.session, n));
		int got = 0;
		check(tg_session_read_ids(d.session, out.data(), done + 1 + n, &got));
		if (got != done + 1 + n) throw std::runtime_error("token log incomplete");
		for (int i = 0; i < n; i++) {
			const int tok = out[(size_t)done + 1];
			if (terminate_on_end && tok == tokenizer->get_eot_id()) {
				stop = true;
				break;
			}
			const std::string piece = piece_of(tok, prev_token);
			decoded.append(piece);
			std::cout << piece << std::flush;
			prev_token = tok;
			done++;
		}
	}
	auto t_decode_e = clk::now();
	const double s_prefill = std::chrono::duration<double>(t_prefill_e - t_prefill_s).count();
	const double s_decode = std::chrono::duration<double>(t_decode_e - t_decode_s).count();
	return {done, decoded, (float)s_prefill, (float)s_decode};
}
}  // namespace gemma

namespace ops {
// strict '>' scan from index 0: the lowest index wins ties
inline void argmax_logits(tensor::tokens *toks, tensor::activation *o) {
	float best = -INFINITY;
	int arg = -1;
	for (size_t i = 0; i < constants::vocab && i < o->data.size(); i++)
		if (o->data[i] > best) {
			arg = (int)i;
			best = o->data[i];
		}
	toks->data[0] = arg;
}

// ops.hpp:762: the logits buffer is left as it is (the reference overwrites it with the probabilities)
inline void minp_logits(tensor::tokens *toks, tensor::activation *o, float minp, float temp, float randf) {
	int32_t tok = 0;
	check(tg_minp_logits(o->data.data(), (int)o->data.size(), minp, temp, randf, &tok));
	toks->data[0] = tok;
}
}  // namespace ops

}  // namespace tinygemma

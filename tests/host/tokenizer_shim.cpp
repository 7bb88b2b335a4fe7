// Test harness: plain-C entry points around tiny-gemma_amd/host/tokenizer.hpp so that the Python tests can
// drive it next to the reference's tokenizer (oracle/ref_wrap.cpp: ref_tok_*), same signatures; and around the
// prompt builder of the pass key run (tiny-gemma_amd/host/passkey.hpp).
#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

#include "../../tiny-gemma_amd/host/passkey.hpp"
#include "../../tiny-gemma_amd/host/tokenizer.hpp"

using tinygemma::sentencepiece::Tokenizer;

extern "C" {

void *tok_create(const char *path, int bos_id, int eos_id, int vocab_size, int chat_format) {
	try {
		return new Tokenizer(path, bos_id, eos_id, vocab_size, chat_format != 0);
	} catch (const std::exception &) {
		return nullptr;
	}
}
void tok_destroy(void *tp) { delete static_cast<Tokenizer *>(tp); }
int tok_encode(void *tp, const char *text, int n, int *ids, int cap) {
	std::vector<int> v = static_cast<Tokenizer *>(tp)->encode(std::string(text, (size_t)n));
	for (int i = 0; i < (int)v.size() && i < cap; i++) ids[i] = v[i];
	return (int)v.size();
}
// -2: std::invalid_argument, -3: another exception
int tok_decode_piece(void *tp, int token, int prev_token, char *out, int cap) {
	try {
		std::string piece = static_cast<Tokenizer *>(tp)->decode(token, prev_token);
		std::memcpy(out, piece.data(), std::min((size_t)cap, piece.size()));
		return (int)piece.size();
	} catch (const std::invalid_argument &) {
		return -2;
	} catch (const std::exception &) {
		return -3;
	}
}
int tok_decode(void *tp, const int *ids, int n, char *out, int cap) {
	try {
		std::string text = static_cast<Tokenizer *>(tp)->decode(std::vector<int>(ids, ids + n));
		std::memcpy(out, text.data(), std::min((size_t)cap, text.size()));
		return (int)text.size();
	} catch (const std::invalid_argument &) {
		return -2;
	} catch (const std::exception &) {
		return -3;
	}
}
int tok_byte_of(void *tp, int token) { return static_cast<Tokenizer *>(tp)->byte_of(token); }

int passkey_prompt(int n_garbage, int n_garbage_prefix, int key, char *out, int cap) {
	const std::string p = tinygemma::passkey::build_prompt(n_garbage, n_garbage_prefix, key);
	std::memcpy(out, p.data(), std::min((size_t)cap, p.size()));
	return (int)p.size();
}
void passkey_draw(unsigned seed, int n_garbage, int *n_garbage_prefix, int *key) {
	std::mt19937 gen(seed);
	auto d = tinygemma::passkey::draw(n_garbage, gen);
	*n_garbage_prefix = d.first;
	*key = d.second;
}

}  // extern "C"

// Host-side tokenizer with the interface and the results of the reference's sentencepiece::Tokenizer
// (csrc/include/tokenizer.hpp:14-239): same constructor, encode / decode signatures and getters, so a
// reference call site (gemma.cpp:45, transformer.hpp:174-250) compiles unchanged against it.
//
// File format (written by py/convert.py:83-113): u32 max_token_length, then per token
// { f32 score, u32 nbytes, bytes }.
//
// What the reference computes, and what is kept:
//   encode  (tokenizer.hpp:113-201): BOS (+ <start_of_turn> user \n in chat format); the text is cut into
//           UTF-8 code points (a lead byte plus up to three continuation bytes), each looked up whole, else
//           emitted byte by byte as ids byte + 3; then the adjacent pair whose concatenation is the
//           best-scored vocabulary entry is merged, leftmost first among equal scores (strict >), until no
//           pair merges; chat format appends <end_of_turn> \n <start_of_turn> model \n.
//   decode  (tokenizer.hpp:203-233): the piece of the id; a leading space is dropped when the previous
//           token is id 1.  A piece of the form <0xHH> (a byte token) makes the reference throw
//           std::invalid_argument: it hands "xHH" to std::stoi (tokenizer.hpp:213-214, the substring starts
//           one character early; checked against the compiled reference).  decode() throws the same
//           exception; byte_of() tells a caller which byte such a piece stands for.
// What differs: lookups go through a hash map instead of a sorted array, and merge candidates are cached
// per position and refreshed only next to a merge (the reference rebuilds and looks up every pair string
// in every round); both change the cost, not the result.  Were two vocabulary entries the same string,
// the lowest id wins here (the reference's unstable sort leaves that unspecified).

#pragma once

#include <cstdint>
#include <fstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace tinygemma {
namespace sentencepiece {

class Tokenizer {
	int bos_id;
	int eos_id;
	int vocab_size;
	int max_token_length = 0;
	bool chat_format;

	// Gemma chat template ids (tokenizer.hpp:33-39)
	int sot_id = 105;  // <start_of_turn>
	int eot_id = 106;  // <end_of_turn>
	int newline_id = 107;
	int user_id = 2364;
	int model_id = 4368;

	std::vector<std::string> vocab;
	std::vector<float> vocab_scores;
	std::unordered_map<std::string, int> lookup;

	int str_lookup(const std::string &x) const {
		auto it = lookup.find(x);
		return it == lookup.end() ? -1 : it->second;
	}

	struct Merge {
		int id = -1;
		float score = 0.0f;
	};
	Merge merge_of(int left, int right) const {
		Merge m;
		m.id = str_lookup(vocab[(size_t)left] + vocab[(size_t)right]);
		if (m.id != -1) m.score = vocab_scores[(size_t)m.id];
		return m;
	}

	// <0x + two or three hex digits + > (the reference's regex, tokenizer.hpp:211); returns the value or -1
	static int byte_piece_value(const std::string &p) {
		if (p.size() < 6 || p.size() > 7 || p[0] != '<' || p[1] != '0' || p[2] != 'x' || p.back() != '>') return -1;
		int v = 0;
		for (size_t i = 3; i + 1 < p.size(); i++) {
			const char c = p[i];
			int d;
			if (c >= '0' && c <= '9') d = c - '0';
			else if (c >= 'a' && c <= 'f') d = c - 'a' + 10;
			else if (c >= 'A' && c <= 'F') d = c - 'A' + 10;
			else return -1;
			v = v * 16 + d;
		}
		return v;
	}

   public:
	Tokenizer(const std::string &model_path, const int bos_id, const int eos_id, const int vocab_size, bool chat_format)
	    : bos_id(bos_id), eos_id(eos_id), vocab_size(vocab_size), chat_format(chat_format) {
		std::ifstream f(model_path, std::ios::binary);
		if (!f) throw std::runtime_error("Cannot open model file: " + model_path);  // tokenizer.hpp:87-89
		uint32_t max_len = 0;
		f.read(reinterpret_cast<char *>(&max_len), sizeof(uint32_t));
		max_token_length = (int)max_len;
		vocab.resize((size_t)vocab_size);
		vocab_scores.resize((size_t)vocab_size);
		lookup.reserve((size_t)vocab_size * 2);
		for (int i = 0; i < vocab_size; i++) {
			float score = 0.0f;
			uint32_t nbytes = 0;
			f.read(reinterpret_cast<char *>(&score), sizeof(float));
			f.read(reinterpret_cast<char *>(&nbytes), sizeof(uint32_t));
			if (!f) throw std::runtime_error("Tokenizer file is shorter than vocab_size entries: " + model_path);
			std::string token((size_t)nbytes, '\0');
			f.read(token.data(), nbytes);
			vocab_scores[(size_t)i] = score;
			lookup.emplace(token, i);  // keeps the first (lowest) id of a repeated string
			vocab[(size_t)i] = std::move(token);
		}
	}

	std::vector<int> encode(const std::string &text) const {
		std::vector<int> tokens;
		tokens.push_back(bos_id);
		if (chat_format) tokens.insert(tokens.end(), {sot_id, user_id, newline_id});

		// code points: a byte that is not a continuation byte starts a new one; at most 4 bytes are collected
		std::string cp;
		for (size_t i = 0; i < text.size(); i++) {
			const uint8_t b = (uint8_t)text[i];
			if ((b & 0xC0) != 0x80) cp.clear();
			cp.push_back(text[i]);
			if (i + 1 < text.size() && ((uint8_t)text[i + 1] & 0xC0) == 0x80 && cp.size() < 4) continue;
			const int id = str_lookup(cp);
			if (id != -1) {
				tokens.push_back(id);
			} else {
				for (char c : cp) tokens.push_back((int)(uint8_t)c + 3);  // byte fallback behind <unk>, <s>, </s>
			}
		}

		// merges: cand[i] is the merge of tokens[i], tokens[i + 1]
		std::vector<Merge> cand(tokens.size());
		for (size_t i = 0; i + 1 < tokens.size(); i++) cand[i] = merge_of(tokens[i], tokens[i + 1]);
		while (true) {
			float best_score = -1e10f;
			int best_idx = -1;
			const int n = (int)tokens.size();
			for (int i = 0; i < n - 1; i++) {
				if (cand[(size_t)i].id != -1 && cand[(size_t)i].score > best_score) {
					best_score = cand[(size_t)i].score;
					best_idx = i;
				}
			}
			if (best_idx == -1) break;
			tokens[(size_t)best_idx] = cand[(size_t)best_idx].id;
			tokens.erase(tokens.begin() + best_idx + 1);
			cand.erase(cand.begin() + best_idx + 1);
			if (best_idx > 0) cand[(size_t)best_idx - 1] = merge_of(tokens[(size_t)best_idx - 1], tokens[(size_t)best_idx]);
			cand[(size_t)best_idx] =
			    (size_t)best_idx + 1 < tokens.size() ? merge_of(tokens[(size_t)best_idx], tokens[(size_t)best_idx + 1]) : Merge{};
		}

		if (chat_format) tokens.insert(tokens.end(), {eot_id, newline_id, sot_id, model_id, newline_id});
		return tokens;
	}

	// An id outside [0, vocab_size) has no piece (the reference indexes its vocabulary unchecked, tokenizer.hpp:203-218;
	// such an id can reach a caller: the argmax of a row of NaN logits is -1, ops.hpp:749-757): it decodes to nothing.
	bool has_piece(int token) const { return token >= 0 && (size_t)token < vocab.size(); }

	std::string decode(int token, int prev_token) const {
		if (!has_piece(token)) return std::string();
		std::string piece = vocab[(size_t)token];
		if (prev_token == 1 && !piece.empty() && piece[0] == ' ') piece = piece.substr(1);
		if (byte_piece_value(piece) >= 0) throw std::invalid_argument("stoi");  // as the reference does, see the header comment
		return piece;
	}

	// The byte a piece of the form <0xHH> stands for, -1 for any other token (no counterpart in the reference).
	int byte_of(int token) const {
		if (!has_piece(token)) return -1;
		const int v = byte_piece_value(vocab[(size_t)token]);
		return v < 256 ? v : -1;
	}

	std::string decode(const std::vector<int> &tokens) const {
		std::string result;
		int prev_token = bos_id;
		result += decode(prev_token, -1);
		for (int token : tokens) {
			if (token != bos_id && token != eos_id) result += decode(token, prev_token);
			prev_token = token;
		}
		return result;
	}

	int get_bos_id() const { return bos_id; }
	int get_eos_id() const { return eos_id; }
	int get_eot_id() const { return eot_id; }
	int get_vocab_size() const { return vocab_size; }
};

}  // namespace sentencepiece
}  // namespace tinygemma

// Drives the C++ mirror (tiny-gemma_amd/host/tinygemma.hpp) the way the reference's own harnesses
// drive its headers (tests/csrc/test_generation.cpp:35-127 of the reference): construct, read_weights,
// forward_prefill, argmax_logits, then a forward_decode loop.  Prints the greedy ids, one per line.
//
// usage: host_mirror_test <weights.bin> <n_layers> <prompt_ids.i32> <n_decode>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>

#include "../../tiny-gemma_amd/host/tinygemma.hpp"

using namespace tinygemma;

static int expect_throw(const char *what, const std::string &needle, void (*fn)()) {
	try {
		fn();
	} catch (const std::runtime_error &e) {
		if (std::string(e.what()).find(needle) == std::string::npos) {
			std::printf("FAIL %s: message '%s' lacks '%s'\n", what, e.what(), needle.c_str());
			return 1;
		}
		std::printf("ok %s: %s\n", what, e.what());
		return 0;
	}
	std::printf("FAIL %s: no exception\n", what);
	return 1;
}

int main(int argc, char **argv) {
	if (argc != 5) {
		std::fprintf(stderr, "usage: %s weights.bin n_layers prompt.i32 n_decode\n", argv[0]);
		return 2;
	}
	int failures = 0;
	failures += expect_throw("unsupported dimension", "Unsupported ROW dimension: 512", [] {
		std::vector<float> c(256), a(512), s(256, 1.0f);
		std::vector<int8_t> b(512 * 256);
		gemv::launch_qgemv(c.data(), a.data(), b.data(), s.data(), 512, 256);
	});
	failures += expect_throw("missing weight file", "Could not open file.", [] {
		config::Config cfg = config::CONFIG_MAP.at("270m");
		cfg.n_layers = 1;
		gemma::Transformer t(cfg);
		gemma::read_weights(&t, "/nonexistent/gemma_i8.bin");
	});

	config::Config cfg = config::CONFIG_MAP.at("270m");
	cfg.n_layers = std::atoi(argv[2]);
	gemma::Transformer t(cfg);
	gemma::read_weights(&t, argv[1]);

	std::ifstream f(argv[3], std::ios::binary | std::ios::ate);
	const size_t n_prompt = (size_t)f.tellg() / sizeof(int);
	f.seekg(0);
	tensor::tokens tokens(1, n_prompt);
	f.read(reinterpret_cast<char *>(tokens.data.data()), (std::streamsize)(n_prompt * sizeof(int)));
	const int n_decode = std::atoi(argv[4]);

	decode::RoPE rope(&cfg, false), rope_sw(&cfg, true);
	lut::GeLUTable table{-4.0, 4.0, 1024};
	decode::DecodeState d(1, &cfg);
	tensor::activation o(1, 1, cfg.n_vocab);

	gemma::forward_prefill(&o, &tokens, &t, &d, &rope, &rope_sw, &table);
	tensor::tokens tokens_decode(1, 1);
	ops::argmax_logits(&tokens_decode, &o);
	std::printf("id %d\n", tokens_decode.data[0]);
	size_t pos_offset = tokens.y;
	for (int step = 0; step < n_decode; step++, pos_offset++) {
		gemma::forward_decode(&o, &tokens_decode, &t, &d, &rope, &rope_sw, pos_offset, &table);
		ops::argmax_logits(&tokens_decode, &o);
		std::printf("id %d\n", tokens_decode.data[0]);
	}
	std::printf("position %d\n", d.position());

	std::vector<int> prompt(tokens.data.begin(), tokens.data.end());
	auto [n_gen, ids, s_prefill, s_decode] = gemma::generate_greedy(prompt, n_decode, &t);
	for (int id : ids) std::printf("gid %d\n", id);

	// the sampling branch (transformer.hpp:208-211, 232-235): the reference's loop spelled out with ops::minp_logits,
	// against generate_ids with an equally seeded generator
	{
		const float minp = 0.05f, temp = 0.9f;
		std::mt19937 gen(123), gen2(123);
		std::uniform_real_distribution<float> unif(0.0, 1.0);
		decode::DecodeState d2(1, &cfg);
		gemma::forward_prefill(&o, &tokens, &t, &d2, &rope, &rope_sw, &table);
		std::vector<int> stepwise;
		ops::minp_logits(&tokens_decode, &o, minp, temp, unif(gen));
		stepwise.push_back(tokens_decode.data[0]);
		size_t off = tokens.y;
		for (int step = 0; step < n_decode; step++, off++) {
			gemma::forward_decode(&o, &tokens_decode, &t, &d2, &rope, &rope_sw, off, &table);
			ops::minp_logits(&tokens_decode, &o, minp, temp, unif(gen));
			stepwise.push_back(tokens_decode.data[0]);
		}
		auto [n2, sids, sp2, sd2] = gemma::generate_ids(prompt, n_decode, &t, minp, temp, gen2);
		for (size_t i = 0; i < sids.size(); i++) {
			std::printf("sid %d %d\n", stepwise[i], sids[i]);
			if (stepwise[i] != sids[i]) failures++;
		}
	}
	std::printf("failures %d\n", failures);
	return failures ? 1 : 0;
}

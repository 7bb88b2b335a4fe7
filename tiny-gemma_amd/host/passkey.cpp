// Pass key retrieval run with the options, the flow and the output of the reference's tests/passkey.cpp
// (passkey.cpp:56-117) on top of the host mirror: a number is hidden at a random place in n_garbage characters
// of filler, the model is asked for it in chat format, greedy, 50 tokens at most, stopping at <end_of_turn>,
// and the run reports whether the generated text contains the number, then the closing tok/s line.
//
//   passkey --weights_path w.bin --model_size 1B --n_garbage 20000 [--tokenizer_path weights/tokenizer_gemma3.bin]
//           [--seed N] [--n_garbage_prefix P --passkey K]
//
// --seed makes the two random draws repeatable (the reference always seeds from std::random_device, the default
// here); --n_garbage_prefix with --passkey fixes them instead, for sweeps over the depth of the hidden line.
//
// Build: g++ -std=c++20 -O2 passkey.cpp -o passkey -L.. -ltinygemma_hip -Wl,-rpath,'$ORIGIN/..'

#include <chrono>
#include <cstdio>
#include <iostream>
#include <random>
#include <string>

#include "options.hpp"
#include "passkey.hpp"
#include "tinygemma.hpp"

int main(int argc, char **argv) {
	using namespace tinygemma;
	std::string weights_path, model_size;
	std::string tokenizer_path = "weights/tokenizer_gemma3.bin";
	int n_garbage = 0;
	int seed = -1;
	int n_garbage_prefix = 0;
	int key = 0;
	const int n_decode = 50;

	Options app("CLI Application for Gemma 3 Passkey retrieval.");
	app.add("weights_path", weights_path, "File path for model weights.");
	app.add("model_size", model_size, "Model size to load.");
	app.add("n_garbage", n_garbage, "Total number of garbage characters.");
	app.add("tokenizer_path", tokenizer_path, "File path for tokenizer.");
	app.add("seed", seed, "Seed of the two random draws (default: from std::random_device).");
	app.add("n_garbage_prefix", n_garbage_prefix, "Garbage characters before the pass key line (with --passkey: no random draw).");
	app.add("passkey", key, "The pass key (with --n_garbage_prefix: no random draw).");
	try {
		if (int rc = app.parse(argc, argv)) return rc;
	} catch (const std::exception &ex) {
		std::cerr << "Parse error: " << ex.what() << '\n';
		return 1;
	}
	if (n_garbage < 1) return app.usage(argv[0], "--n_garbage must be at least 1");
	if ((n_garbage_prefix != 0) != (key != 0)) return app.usage(argv[0], "--n_garbage_prefix and --passkey go together");
	if (n_garbage_prefix < 0 || n_garbage_prefix > n_garbage || key < 0) return app.usage(argv[0], "--n_garbage_prefix must lie in 1..n_garbage");

	try {
		config::Config cfg = config::CONFIG_MAP.at(model_size);
		gemma::Transformer t(cfg);
		gemma::read_weights(&t, weights_path.c_str());
		printf("Weights loaded!\n");
		sentencepiece::Tokenizer tokenizer(tokenizer_path, constants::bos_id, constants::eos_id, (int)constants::vocab, true);

		if (key == 0) {
			std::random_device rd;
			std::mt19937 gen(seed >= 0 ? (unsigned)seed : rd());
			std::tie(n_garbage_prefix, key) = passkey::draw(n_garbage, gen);
		}
		const std::string prompt = passkey::build_prompt(n_garbage, n_garbage_prefix, key);
		const std::string number = std::to_string(key);

		auto t0 = std::chrono::high_resolution_clock::now();
		auto generations = gemma::generate(prompt, n_decode, &tokenizer, &t, 1.0f, 0.0f, true);
		auto t1 = std::chrono::high_resolution_clock::now();
		const double s = std::chrono::duration<double>(t1 - t0).count();

		const int n_generated_tokens = std::get<0>(generations);
		if (std::get<1>(generations).find(number) == std::string::npos)
			printf("\nPasskey=%s not found!\n", number.c_str());
		else
			printf("\nPasskey=%s found!\n", number.c_str());
		printf("\n\nGenerating %u tokens took %f seconds. Tok/s: %f ms/token: %f\n", n_generated_tokens, s, n_generated_tokens / s,
		       1e3 * s / n_generated_tokens);
	} catch (const std::exception &ex) {
		std::cerr << "error: " << ex.what() << '\n';
		return 1;
	}
	return 0;
}

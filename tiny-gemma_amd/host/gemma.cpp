// Command line front end with the options, the flow and the closing line of the reference's gemma.cpp
// (gemma.cpp:7-60), on top of the host mirror: load weights, load the tokenizer, generate, report tok/s as
// prompt tokens / prefill seconds and generated tokens / decode seconds (gemma.cpp:51-57).
//
//   gemma --weights_path w.bin --model_size 1B --prompt "..." --n_dec 256 [--minp 2.0] [--temp 1.0]
//         [--chat_format 0|1] [--terminate_on_eos 0|1] [--tokenizer_path weights/tokenizer_gemma3.bin]
//
// Options are "--name value" pairs as in the reference's parser (argparse.hpp:31-53): anything else is a usage
// error with exit status 1.  The reference leaves n_dec, temp, chat_format and terminate_on_eos uninitialised when
// they are not given; here they default to 64, 1.0, 0 and 0.
//
// Build: g++ -std=c++20 -O2 gemma.cpp -o gemma -L.. -ltinygemma_hip -Wl,-rpath,'$ORIGIN/..'

#include <cstdio>
#include <iostream>
#include <string>

#include "options.hpp"
#include "tinygemma.hpp"

int main(int argc, char **argv) {
	using namespace tinygemma;
	std::string weights_path, model_size, prompt;
	std::string tokenizer_path = "weights/tokenizer_gemma3.bin";
	int n_decode = 64;
	float minp = 2.0f;
	float temp = 1.0f;
	int chat_format = 0;
	int terminate_on_eos = 0;

	Options app("CLI Application for Gemma 3 text generation.");
	app.add("weights_path", weights_path, "File path for model weights.");
	app.add("model_size", model_size, "Model size to load.");
	app.add("prompt", prompt, "The prompt.");
	app.add("n_dec", n_decode, "Number of tokens to generate.");
	app.add("minp", minp, "Minp sampler, defaults to greedy sampling if `minp >= 1`.");
	app.add("temp", temp, "Sampler temperature.");
	app.add("chat_format", chat_format, "Flag to enable using chat template.");
	app.add("terminate_on_eos", terminate_on_eos, "Flag to enable early termination if model generates an EOS/EOT token.");
	app.add("tokenizer_path", tokenizer_path, "File path for tokenizer.");
	try {
		if (int rc = app.parse(argc, argv)) return rc;
	} catch (const std::exception &ex) {
		std::cerr << "Parse error: " << ex.what() << '\n';
		return 1;
	}

	try {
		config::Config cfg = config::CONFIG_MAP.at(model_size);
		gemma::Transformer t(cfg);
		gemma::read_weights(&t, weights_path.c_str());
		printf("Weights loaded!\n");
		sentencepiece::Tokenizer tokenizer(tokenizer_path, constants::bos_id, constants::eos_id, (int)constants::vocab, bool(chat_format));
		auto generations = gemma::generate(prompt, n_decode, &tokenizer, &t, minp, temp, bool(terminate_on_eos));
		const int n_generated_tokens = std::get<0>(generations);
		const int n_prompt_tokens = (int)tokenizer.encode(prompt).size();
		const float total_s = std::get<2>(generations) + std::get<3>(generations);
		const float prefill_tok_s = n_prompt_tokens / std::get<2>(generations);
		const float decode_tok_s = n_generated_tokens / std::get<3>(generations);
		printf("\n\nGenerating %u tokens took %f seconds. Prefill Tok/s: %f  Decode Tok/s %f ms/token: %f\n", n_generated_tokens, total_s,
		       prefill_tok_s, decode_tok_s, 1e3 * std::get<3>(generations) / n_generated_tokens);
	} catch (const std::exception &ex) {
		std::cerr << "error: " << ex.what() << '\n';
		return 1;
	}
	return 0;
}

// Text generation from the command line on top of the host mirror: the reference's gemma.cpp (gemma.cpp:7-60) as far
// as a user sees it — same option names, same flow (weights, tokenizer, generate), same closing line with tok/s
// as prompt tokens / prefill seconds and generated tokens / decode seconds (gemma.cpp:51-57).
//
//   gemma --weights_path w.bin --model_size 1B --prompt "..." --n_dec 256 [--minp 2.0] [--temp 1.0]
//         [--chat_format 0|1] [--terminate_on_eos 0|1] [--tokenizer_path weights/tokenizer_gemma3.bin]
//
// Every option is a "--name value" pair (argparse.hpp:31-53); anything else ends with a usage message and exit
// status 1.  Where the reference leaves n_dec, temp, chat_format and terminate_on_eos uninitialised when they are not
// given, the defaults here are 64, 1.0, 0 and 0.
//
// Build: g++ -std=c++20 -O2 gemma.cpp -o gemma -L.. -ltinygemma_hip -Wl,-rpath,'$ORIGIN/..'

#include <cstdio>
#include <iostream>
#include <string>

#include "options.hpp"
#include "tinygemma.hpp"

namespace {

struct Args {
	std::string weights, size, text;
	std::string tokenizer = "weights/tokenizer_gemma3.bin";
	int steps = 64;
	float min_p = 2.0f;  // >= 1: greedy
	float temperature = 1.0f;
	int chat = 0;
	int stop_at_end = 0;
};

// 0: parsed; otherwise the exit status
int read_args(int argc, char **argv, Args &a) {
	tinygemma::Options cli("CLI Application for Gemma 3 text generation.");
	cli.add("weights_path", a.weights, "weight file (int8 matrices with fp32 column scales)");
	cli.add("model_size", a.size, "270m or 1B");
	cli.add("prompt", a.text, "text to continue");
	cli.add("n_dec", a.steps, "tokens to generate");
	cli.add("minp", a.min_p, "min-p threshold of the sampler; 1 or more selects the most likely token");
	cli.add("temp", a.temperature, "sampling temperature");
	cli.add("chat_format", a.chat, "1: wrap the prompt in the chat template");
	cli.add("terminate_on_eos", a.stop_at_end, "1: stop at the end-of-turn token");
	cli.add("tokenizer_path", a.tokenizer, "tokenizer file");
	try {
		return cli.parse(argc, argv);
	} catch (const std::exception &ex) {
		std::cerr << "Parse error: " << ex.what() << '\n';
		return 1;
	}
}

void run(const Args &a) {
	using namespace tinygemma;
	gemma::Transformer model(config::CONFIG_MAP.at(a.size));
	gemma::read_weights(&model, a.weights.c_str());
	printf("Weights loaded!\n");
	sentencepiece::Tokenizer tok(a.tokenizer, constants::bos_id, constants::eos_id, (int)constants::vocab, a.chat != 0);
	const auto [n_out, text, s_prefill, s_decode] = gemma::generate(a.text, a.steps, &tok, &model, a.min_p, a.temperature, a.stop_at_end != 0);
	(void)text;
	const size_t n_in = tok.encode(a.text).size();
	printf("\n\nGenerating %u tokens took %f seconds. Prefill Tok/s: %f  Decode Tok/s %f ms/token: %f\n", n_out, s_prefill + s_decode,
	       n_in / s_prefill, n_out / s_decode, 1e3 * s_decode / n_out);
}

}  // namespace

int main(int argc, char **argv) {
	Args a;
	if (int rc = read_args(argc, argv, a)) return rc;
	try {
		run(a);
	} catch (const std::exception &ex) {
		std::cerr << "error: " << ex.what() << '\n';
		return 1;
	}
	return 0;
}

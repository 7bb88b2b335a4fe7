// Prompt of the reference's pass key retrieval test (tests/passkey.cpp:10-54): a task description, filler
// sentences, one line that states a number, more filler, and the question.
//
//   n_garbage        characters of filler in total
//   n_garbage_prefix characters of it before the line with the number (1..n_garbage)
//
// The filler is the 90-character sentence block repeated and cut to length.  The reference cuts the block after
// the number with the remainder of the PREFIX length (passkey.cpp:33-37), so the filler behind the number is
// (n_garbage - n_garbage_prefix) / 90 whole blocks plus n_garbage_prefix % 90 characters; kept, since the
// prompt is what the published retrieval results were measured on.
#pragma once

#include <random>
#include <string>
#include <utility>

namespace tinygemma {
namespace passkey {

inline const std::string kTask =
    "There is an important info hidden inside a lot of irrelevant text. Find it and memorize them. I will quiz you about the "
    "important information there. ";
inline const std::string kFiller = "The grass is green. The sky is blue. The sun is yellow. Here we go. There and back again. ";
inline const std::string kQuestion = "\nWhat is the pass key? The pass key is";

inline std::string filler(int whole_blocks, int extra_chars) {
	std::string s;
	s.reserve((size_t)whole_blocks * kFiller.size() + (size_t)extra_chars);
	for (int i = 0; i < whole_blocks; i++) s += kFiller;
	s.append(kFiller, 0, (size_t)extra_chars);
	return s;
}

inline std::string build_prompt(int n_garbage, int n_garbage_prefix, int key) {
	const int block = (int)kFiller.size();
	const std::string number = std::to_string(key);
	const int cut = n_garbage_prefix % block;
	std::string prompt = kTask;
	prompt += filler(n_garbage_prefix / block, cut);
	prompt += "\nThe pass key is " + number + ". Remember it. " + number + " is the pass key.\n";
	prompt += filler((n_garbage - n_garbage_prefix) / block, cut);
	prompt += kQuestion;
	return prompt;
}

// The two draws of the reference, in its order (passkey.cpp:14-20): where the number goes, then the number.
inline std::pair<int, int> draw(int n_garbage, std::mt19937 &gen) {
	std::uniform_int_distribution<int> where(1, n_garbage);
	std::uniform_int_distribution<int> what(1, 50000);
	const int n_garbage_prefix = where(gen);
	const int key = what(gen);
	return {n_garbage_prefix, key};
}

}  // namespace passkey
}  // namespace tinygemma

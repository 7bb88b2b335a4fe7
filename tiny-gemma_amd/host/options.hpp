// "--name value" command line options shared by the front ends (gemma.cpp, passkey.cpp), with the behaviour of
// the reference's parser (argparse.hpp:31-53): every option takes one value, anything else is a usage error
// with exit status 1, a value that does not convert throws std::invalid_argument("expected integer for ...").
#pragma once

#include <functional>
#include <iostream>
#include <map>
#include <stdexcept>
#include <string>
#include <utility>

namespace tinygemma {

struct Options {
	std::string description;
	std::map<std::string, std::pair<std::function<void(const std::string &)>, std::string>> opts;

	explicit Options(std::string description) : description(std::move(description)) {}

	void add(const std::string &name, std::string &dst, const std::string &help) {
		opts[name] = {[&dst](const std::string &v) { dst = v; }, help};
	}
	void add(const std::string &name, int &dst, const std::string &help) {
		opts[name] = {[&dst](const std::string &v) {
			              try {
				              dst = std::stoi(v);
			              } catch (...) {
				              throw std::invalid_argument("expected integer for " + v);
			              }
		              },
		              help};
	}
	void add(const std::string &name, float &dst, const std::string &help) {
		opts[name] = {[&dst](const std::string &v) {
			              try {
				              dst = std::stof(v);
			              } catch (...) {
				              throw std::invalid_argument("expected float for " + v);
			              }
		              },
		              help};
	}
	int usage(const char *prog, const std::string &msg) const {
		std::cerr << "Error: " << msg << "\n\n" << description << "\nUsage: " << prog << " [options]\n\nOptions:\n";
		for (const auto &[name, o] : opts) std::cerr << "  --" << name << "\t" << o.second << '\n';
		return 1;
	}
	int parse(int argc, char **argv) const {
		for (int i = 1; i < argc; ++i) {
			const std::string arg = argv[i];
			if (arg.rfind("--", 0) != 0) return usage(argv[0], "unexpected token: " + arg);
			auto it = opts.find(arg.substr(2));
			if (it == opts.end()) return usage(argv[0], "unknown option: " + arg);
			if (i + 1 == argc) return usage(argv[0], "missing value for " + arg);
			it->second.first(argv[++i]);
		}
		return 0;
	}
};

}  // namespace tinygemma

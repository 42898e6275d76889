// Command-line options shared by the gradhip command-line callers: the sampling
// flags of grad.cpp's commands (add_sampling_options, src/cli/common.cpp:316-332)
// and the positional arguments of this library's variants of them.
#pragma once

#include <cstdint>
#include <optional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace gradhip::cli {

struct Usage : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Options {
    std::vector<std::string> positional;
    int max_tokens = 150;
    float temperature = 0.8f;
    int top_k = 0;
    float top_p = 1.0f;
    float repetition_penalty = 1.2f;
    bool greedy = false;
    std::optional<std::uint64_t> seed;
    bool stop_at_eos = false;   // not in grad.cpp: end a streamed reply at the tokenizer's end-of-text id
    bool keep_context = false;  // not in grad.cpp: chat lines continue one live context
    // grad.cpp's way of naming the tokenizer: the corpus the checkpoint was trained on
    // (a positional argument there) and --tokenizer v1|v2 (add_tokenizer_option,
    // src/cli/common.cpp:148-150); the file follows from them and the checkpoint.
    std::optional<std::string> corpus;
    std::optional<std::string> tokenizer_flag;
};

template <class T>
T number(const std::string& flag, const std::string& text) {
    std::istringstream in(text);
    T v{};
    if (!(in >> v) || !in.eof()) throw Usage(flag + ": expected a number, got '" + text + "'");
    return v;
}

// defaults: the values a command starts from (generate: 150 tokens, chat: 200).
inline Options parse(int argc, char** argv, Options o) {
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        const auto value = [&]() -> std::string {
            if (i + 1 >= argc) throw Usage(a + ": missing value");
            return argv[++i];
        };
        if (a == "--max-tokens") {
            o.max_tokens = number<int>(a, value());
            if (o.max_tokens < 1) throw Usage("--max-tokens: must be at least 1");
        } else if (a == "--temperature") {
            o.temperature = number<float>(a, value());
            if (!(o.temperature > 0.0f)) throw Usage("--temperature: must be positive");
        } else if (a == "--top-k") {
            o.top_k = number<int>(a, value());
            if (o.top_k < 0) throw Usage("--top-k: must be at least 0");
        } else if (a == "--top-p") {
            o.top_p = number<float>(a, value());
            if (!(o.top_p > 0.0f) || o.top_p > 1.0f) throw Usage("--top-p: must be positive and at most 1");
        } else if (a == "--repetition-penalty") {
            o.repetition_penalty = number<float>(a, value());
            if (!(o.repetition_penalty > 0.0f)) throw Usage("--repetition-penalty: must be positive");
        } else if (a == "--greedy") {
            o.greedy = true;
        } else if (a == "--stop-at-eos") {
            o.stop_at_eos = true;
        } else if (a == "--keep-context") {
            o.keep_context = true;
        } else if (a == "--corpus") {
            o.corpus = value();
        } else if (a == "--tokenizer") {
            o.tokenizer_flag = value();
        } else if (a == "--seed") {
            o.seed = number<std::uint64_t>(a, value());
        } else if (a.rfind("--", 0) == 0) {
            throw Usage("unknown option " + a);
        } else {
            o.positional.push_back(a);
        }
    }
    return o;
}

}  // namespace gradhip::cli

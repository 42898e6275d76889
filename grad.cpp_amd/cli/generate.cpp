// gradhip-generate: a greedy and a sampled continuation of one prompt from a saved
// checkpoint, on the GPU.  The command-line shape of `grad generate`
// (src/cli/generate.cpp:61-107 of grad.cpp) for the part this library covers:
//
//   gradhip-generate <checkpoint> <tokenizer.tok> <prompt text>
//       [--max-tokens N] [--temperature T] [--top-k K] [--top-p P]
//       [--repetition-penalty R] [--greedy] [--seed S]
//
// grad.cpp finds the tokenizer file from the corpus path and vocabulary size
// (src/cli/common.cpp:160-187); here it is named explicitly.  The fingerprint
// guard is the same: a checkpoint that records a tokenizer is only used with it.
// Exit codes follow src/cli/main.cpp:94-103: 2 for a usage error, 1 for any failure.
#include "gradhip.hpp"

#include <cstdlib>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

namespace {

struct Usage : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Options {
    std::string checkpoint, tokenizer, prompt;
    int max_tokens = 150;  // generate.cpp:67
    float temperature = 0.8f;
    int top_k = 0;
    float top_p = 1.0f;
    float repetition_penalty = 1.2f;
    bool greedy = false;
    std::optional<std::uint64_t> seed;
};

template <class T>
T number(const std::string& flag, const std::string& text) {
    std::istringstream in(text);
    T v{};
    if (!(in >> v) || !in.eof()) throw Usage(flag + ": expected a number, got '" + text + "'");
    return v;
}

Options parse(int argc, char** argv) {
    Options o;
    std::vector<std::string> positional;
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
        } else if (a == "--seed") {
            o.seed = number<std::uint64_t>(a, value());
        } else if (a.rfind("--", 0) == 0) {
            throw Usage("unknown option " + a);
        } else {
            positional.push_back(a);
        }
    }
    if (positional.size() != 3) throw Usage("usage: gradhip-generate <checkpoint> <tokenizer.tok> <prompt> [options]");
    o.checkpoint = positional[0];
    o.tokenizer = positional[1];
    o.prompt = positional[2];
    return o;
}

// "temp=0.8", plus any cut that is on (generate.cpp:50-57).
std::string describe(const Options& o) {
    std::ostringstream out;
    out << "temp=" << o.temperature;
    if (o.top_k > 0) out << ", top-k=" << o.top_k;
    if (o.top_p < 1.0f) out << ", top-p=" << o.top_p;
    return out.str();
}

}  // namespace

int main(int argc, char** argv) {
    try {
        const Options o = parse(argc, argv);
        std::cout << "\ngradhip Generation\n" << std::endl;
        const gradhip::GPTModel model = gradhip::GPTModel::load(o.checkpoint);
        const std::unique_ptr<gradhip::Tokenizer> tokenizer = gradhip::load_tokenizer(o.tokenizer);
        std::cout << "Tokenizer: " << o.tokenizer << " (" << gradhip::tokenizer_kind_flag(tokenizer->kind())
                  << ", vocab " << tokenizer->vocab_size() << ")" << std::endl;
        if (tokenizer->vocab_size() != model.getVocabSize()) {
            throw std::runtime_error("tokenizer vocab " + std::to_string(tokenizer->vocab_size())
                                     + " does not match the checkpoint's vocab of "
                                     + std::to_string(model.getVocabSize()));
        }
        gradhip::check_tokenizer_matches(model, *tokenizer, o.checkpoint);
        const std::vector<int> prompt = tokenizer->encode(o.prompt);
        if (prompt.empty()) throw Usage("the prompt is empty");

        gradhip::TextGen generator(model, tokenizer.get());
        if (o.seed) generator.set_seed(*o.seed);

        std::cout << "\n--- Greedy Decoding ---\n" << std::endl;
        std::cout << "Prompt: \"" << o.prompt << "\"" << std::endl;
        std::cout << generator.generate_greedy(prompt, o.max_tokens, o.repetition_penalty) << std::endl;
        if (o.greedy) return 0;

        std::cout << "\n--- Sampling (" << describe(o) << ") ---\n" << std::endl;
        std::cout << "Prompt: \"" << o.prompt << "\"" << std::endl;
        std::cout << generator.generate_sample(prompt, o.temperature, o.max_tokens, o.repetition_penalty, o.top_k,
                                               o.top_p)
                  << std::endl;
        return 0;
    } catch (const Usage& e) {
        std::cerr << "gradhip-generate: " << e.what() << std::endl;
        return 2;
    } catch (const std::exception& e) {
        std::cerr << "Error: " << e.what() << std::endl;
        return 1;
    }
}

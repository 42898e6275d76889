// gradhip-generate: a greedy and a sampled continuation of one prompt from a saved
// checkpoint, on the GPU.  The command-line shape of `grad generate`
// (src/cli/generate.cpp:61-107 of grad.cpp) for the part this library covers:
//
//   gradhip-generate <checkpoint> <tokenizer file> <prompt text>
//   gradhip-generate <checkpoint> <prompt text> --corpus <corpus path> [--tokenizer v1|v2]
//       [--max-tokens N] [--temperature T] [--top-k K] [--top-p P]
//       [--repetition-penalty R] [--greedy] [--seed S]
//
// grad.cpp finds the tokenizer file from the corpus path and vocabulary size
// (src/cli/common.cpp:160-187); the second form does the same (resolve.h), the
// first names the file.  The fingerprint
// guard is the same: a checkpoint that records a tokenizer is only used with it.
// Exit codes follow src/cli/main.cpp:94-103: 2 for a usage error, 1 for any failure.
#include "gradhip.hpp"
#include "options.h"
#include "resolve.h"

#include <iostream>
#include <sstream>
#include <string>
#include <vector>

namespace {

using gradhip::cli::Options;
using gradhip::cli::Usage;

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
        const Options o = gradhip::cli::parse(argc, argv, Options{});
        const bool by_corpus = o.corpus.has_value();
        if (o.positional.size() != (by_corpus ? 2u : 3u))
            throw Usage("usage: gradhip-generate <checkpoint> <tokenizer file> <prompt> [options]\n"
                        "   or: gradhip-generate <checkpoint> <prompt> --corpus <corpus path> [--tokenizer v1|v2] [options]");
        if (!by_corpus && o.tokenizer_flag) throw Usage("--tokenizer needs --corpus (the file is named otherwise)");
        const std::string& checkpoint = o.positional[0];
        const std::string& text = o.positional[by_corpus ? 1 : 2];
        std::cout << "\ngradhip Generation\n" << std::endl;
        const gradhip::GPTModel model = gradhip::GPTModel::load(checkpoint);
        std::unique_ptr<gradhip::Tokenizer> tokenizer;
        if (by_corpus) {
            // load_for_inference (src/cli/common.cpp:346-358): the generation from the checkpoint,
            // the flag and the files, then the file from the corpus path and the checkpoint's vocabulary
            const gradhip::TokenizerKind kind = gradhip::cli::choose_tokenizer(
                *o.corpus, model.getVocabSize(), gradhip::cli::parse_tokenizer_flag(o.tokenizer_flag), true,
                model.getTokenizerFingerprint());
            tokenizer = gradhip::cli::load_tokenizer_for_inference(*o.corpus, model.getVocabSize(), kind);
            gradhip::cli::require_matching_vocab(*tokenizer, model.getVocabSize());
        } else {
            const std::string& tokenizer_path = o.positional[1];
            tokenizer = gradhip::load_tokenizer(tokenizer_path);
            std::cout << "Tokenizer: " << tokenizer_path << " (" << gradhip::tokenizer_kind_flag(tokenizer->kind())
                      << ", vocab " << tokenizer->vocab_size() << ")" << std::endl;
            if (tokenizer->vocab_size() != model.getVocabSize()) {
                throw std::runtime_error("tokenizer vocab " + std::to_string(tokenizer->vocab_size())
                                         + " does not match the checkpoint's vocab of "
                                         + std::to_string(model.getVocabSize()));
            }
        }
        gradhip::check_tokenizer_matches(model, *tokenizer, checkpoint);
        const std::vector<int> prompt = tokenizer->encode(text);
        if (prompt.empty()) throw Usage("the prompt is empty");

        gradhip::TextGen generator(model, tokenizer.get());
        if (o.seed) generator.set_seed(*o.seed);

        std::cout << "\n--- Greedy Decoding ---\n" << std::endl;
        std::cout << "Prompt: \"" << text << "\"" << std::endl;
        std::cout << generator.generate_greedy(prompt, o.max_tokens, o.repetition_penalty) << std::endl;
        if (o.greedy) return 0;

        std::cout << "\n--- Sampling (" << describe(o) << ") ---\n" << std::endl;
        std::cout << "Prompt: \"" << text << "\"" << std::endl;
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

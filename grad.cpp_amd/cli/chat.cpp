// gradhip-chat: every line typed is continued by the model, streamed token by
// token as it is sampled on the GPU.  The command-line shape of `grad chat`
// (src/cli/chat.cpp:18-71 of grad.cpp):
//
//   gradhip-chat <checkpoint> <tokenizer.tok> [--max-tokens N] [--temperature T] [--top-k K]
//       [--top-p P] [--repetition-penalty R] [--greedy] [--seed S] [--stop-at-eos] [--keep-context]
//
// An empty line, "exit" or "quit" ends the session.  As in the reference, each
// line starts from an empty context (text_gen.cpp:100) and --greedy means top-k 1.
// --stop-at-eos (not in grad.cpp, whose replies always run to --max-tokens) ends a
// reply after the tokenizer's end-of-text token.  --keep-context (not in grad.cpp
// either, which rebuilds the cache for every line) keeps one session alive: a line
// is appended to everything said so far, so only the new tokens are computed, until
// the context is full and the conversation starts over.
#include "gradhip.hpp"
#include "options.h"

#include <iostream>
#include <optional>
#include <random>
#include <string>
#include <vector>

int main(int argc, char** argv) {
    using gradhip::cli::Options;
    using gradhip::cli::Usage;
    try {
        Options defaults;
        defaults.max_tokens = 200;  // chat.cpp:23
        const Options o = gradhip::cli::parse(argc, argv, defaults);
        if (o.positional.size() != 2) throw Usage("usage: gradhip-chat <checkpoint> <tokenizer.tok> [options]");
        std::cout << "\ngradhip Chat\n" << std::endl;
        const gradhip::GPTModel model = gradhip::GPTModel::load(o.positional[0]);
        const std::unique_ptr<gradhip::Tokenizer> tokenizer = gradhip::load_tokenizer(o.positional[1]);
        if (tokenizer->vocab_size() != model.getVocabSize()) {
            throw std::runtime_error("tokenizer vocab " + std::to_string(tokenizer->vocab_size())
                                     + " does not match the checkpoint's vocab of "
                                     + std::to_string(model.getVocabSize()));
        }
        gradhip::check_tokenizer_matches(model, *tokenizer, o.positional[0]);
        gradhip::TextGen generator(model, tokenizer.get());
        if (o.seed) generator.set_seed(*o.seed);
        if (o.stop_at_eos) generator.set_stop_token(tokenizer->eos_id());
        const int top_k = o.greedy ? 1 : o.top_k;

        std::cout << "\nThis is a base language model: it continues text in the"
                  << " style of its training corpus.\nEmpty line or 'exit' quits.\n"
                  << std::endl;
        std::optional<gradhip::InferenceSession> live;  // --keep-context: the conversation so far
        std::uint64_t live_seed = o.seed ? *o.seed : std::random_device{}();
        std::string line;
        while (true) {
            std::cout << "> " << std::flush;
            if (!std::getline(std::cin, line)) break;
            if (line.empty() || line == "exit" || line == "quit") break;
            const std::vector<int> prompt = tokenizer->encode(line + "\n");
            std::cout << line << std::flush;
            if (o.keep_context) {
                if (!live) live.emplace(model);
                // room for the line and at least one token of reply
                if (live->position() + static_cast<int>(prompt.size()) >= live->capacity()) {
                    std::cout << "\n[context full: starting over]" << std::flush;
                    gradhip::check(gh_session_reset(live->handle()));
                    live_seed++;  // a reset session counts its draws from zero again
                }
                if (static_cast<int>(prompt.size()) >= live->capacity())
                    throw std::runtime_error("InferenceSession: context exceeds max_len");
                if (prompt.empty()) continue;
                const std::vector<int32_t> ids(prompt.begin(), prompt.end());
                gradhip::check(gh_session_prefill(live->handle(), ids.data(), static_cast<int32_t>(ids.size()), nullptr));
                const gh_sampling sampling{o.temperature, top_k, o.top_p, o.repetition_penalty, 0};
                const gh_token_callback print = [](void* user, const int32_t* picked, int32_t) -> int32_t {
                    const auto* tok = static_cast<const gradhip::Tokenizer*>(user);
                    std::cout << tok->decode(std::vector<int>{static_cast<int>(picked[0])}) << std::flush;
                    return 0;
                };
                const int stop = o.stop_at_eos && tokenizer->eos_id() ? *tokenizer->eos_id() : -1;
                int32_t made = 0;
                gradhip::check(gh_session_decode_stream(live->handle(), o.max_tokens, &sampling, nullptr, live_seed, stop,
                                                        print, tokenizer.get(), nullptr, &made));
                std::cout << "\n" << std::endl;
                continue;
            }
            generator.generate_stream(
                prompt, [](const std::string& piece) { std::cout << piece << std::flush; }, o.temperature,
                o.max_tokens, o.repetition_penalty, top_k, o.top_p);
            std::cout << "\n" << std::endl;
        }
        return 0;
    } catch (const Usage& e) {
        std::cerr << "gradhip-chat: " << e.what() << std::endl;
        return 2;
    } catch (const std::exception& e) {
        std::cerr << "Error: " << e.what() << std::endl;
        return 1;
    }
}

// gradhip-chat: every line typed is continued by the model, streamed token by
// token as it is sampled on the GPU.  The command-line shape of `grad chat`
// (src/cli/chat.cpp:18-71 of grad.cpp):
//
//   gradhip-chat <checkpoint> <tokenizer.tok> [--max-tokens N] [--temperature T] [--top-k K]
//       [--top-p P] [--repetition-penalty R] [--greedy] [--seed S] [--stop-at-eos]
//
// An empty line, "exit" or "quit" ends the session.  As in the reference, each
// line starts from an empty context (text_gen.cpp:100) and --greedy means top-k 1.
// --stop-at-eos (not in grad.cpp, whose replies always run to --max-tokens) ends a
// reply after the tokenizer's end-of-text token.
#include "gradhip.hpp"
#include "options.h"

#include <iostream>
#include <string>

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
        std::string line;
        while (true) {
            std::cout << "> " << std::flush;
            if (!std::getline(std::cin, line)) break;
            if (line.empty() || line == "exit" || line == "quit") break;
            const std::vector<int> prompt = tokenizer->encode(line + "\n");
            std::cout << line << std::flush;
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

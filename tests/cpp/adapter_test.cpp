// Drives the C++ adapter the way grad.cpp's callers drive its classes
// (src/cli/generate.cpp:86-99, tests/integration/sanity_tests.cpp:315-318).
// Usage: adapter_test <checkpoint> <prompt ids...>; prints results as lines the
// Python test compares with the CPU checker.
#include "gradhip.hpp"

#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

// Emits ids as decimal text, so TextGen's string result carries the ids.
class IdTokenizer : public gradhip::Tokenizer {
public:
    std::string decode(std::span<const int> ids) const override {
        std::ostringstream os;
        for (int id : ids) os << id << ' ';
        return os.str();
    }
};

int main(int argc, char** argv) {
    if (argc < 3) return 2;
    try {
        gradhip::GPTModel model = gradhip::GPTModel::load(argv[1]);
        std::vector<int> prompt;
        for (int i = 2; i < argc; i++) prompt.push_back(std::atoi(argv[i]));
        std::printf("dims %d %d %d %d %d %d\n", model.getVocabSize(), model.getDModel(), model.getNumLayers(),
                    model.getNumHeads(), model.getMaxLen(), static_cast<int>(model.getArch()));

        {   // InferenceSession: logits pointer valid until the next step
            gradhip::InferenceSession s(model);
            const float* logits = nullptr;
            for (int t : prompt) logits = s.step(t);
            std::printf("step %d %d %d", s.position(), s.capacity(), s.vocabSize());
            for (int i = 0; i < 8; i++) std::printf(" %.9g", logits[i]);
            std::printf("\n");
            try {
                (void)s.step(model.getVocabSize());
                std::printf("error none\n");
            } catch (const std::out_of_range& e) {
                std::printf("out_of_range %s\n", e.what());
            }
            try {
                for (int i = 0; i < model.getMaxLen() + 1; i++) (void)s.step(0);
                std::printf("error none\n");
            } catch (const std::runtime_error& e) {
                std::printf("runtime_error %s\n", e.what());
            }
        }

        IdTokenizer tok;
        gradhip::TextGen gen(model, &tok);
        gen.set_seed(77);
        std::printf("greedy %s\n", gen.generate_greedy(prompt, 12, 1.2f).c_str());
        std::printf("sample %s\n", gen.generate_sample(prompt, 0.8f, 12, 1.1f, 5, 0.9f).c_str());
        std::string streamed;
        std::vector<int> streamed_ids;
        const int n = gen.generate_stream(prompt, [&](const std::string& t) {
            streamed += t;
            streamed_ids.push_back(std::atoi(t.c_str()));
        }, 0.8f, 12, 1.1f, 5, 0.9f);
        std::printf("stream %d %s\n", n, streamed.c_str());
        // what the callback throws reaches the caller, with its type, once the run has ended
        try {
            int calls = 0;
            (void)gen.generate_stream(prompt, [&](const std::string&) {
                if (++calls == 3) throw std::domain_error("third token");
            }, 0.8f, 12, 1.1f, 5, 0.9f);
            std::printf("callback_error none\n");
        } catch (const std::domain_error& e) {
            std::printf("callback_error %s\n", e.what());
        }
        // a stop token (not in grad.cpp): the stream ends after the first time it is picked
        {
            gradhip::TextGen stopper(model, &tok);
            stopper.set_seed(77);
            stopper.set_stop_token(streamed_ids.at(4));
            std::string cut;
            const int m = stopper.generate_stream(prompt, [&](const std::string& t) { cut += t; }, 0.8f, 12, 1.1f, 5, 0.9f);
            std::printf("stopped %d %s\n", m, cut.c_str());
        }
        std::printf("empty [%s]\n", gen.generate_greedy({}, 5).c_str());
        // capacity rule: asks for more tokens than the context can take
        std::printf("overflow %s\n", gen.generate_greedy(prompt, model.getMaxLen() + 10, 1.0f).c_str());
        gradhip::TextGen raw(model);  // no tokenizer: ids become bytes
        std::printf("bytes %zu\n", raw.generate_greedy(prompt, 4, 1.0f).size());
    } catch (const std::exception& e) {
        std::printf("FATAL %s\n", e.what());
        return 1;
    }
    try {
        (void)gradhip::GPTModel::load("/nonexistent/model.bin");
    } catch (const std::runtime_error& e) {
        std::printf("load_error %s\n", e.what());
    }
    return 0;
}

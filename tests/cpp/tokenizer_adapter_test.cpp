// Drives the tokenizer half of the C++ adapter the way grad.cpp's CLI does
// (src/cli/common.cpp:228-268: load_tokenizer, encode the prompt, decode ids).
// Usage: tokenizer_adapter_test <tokenizer file> <text>; prints lines the Python
// test compares with the CPU checker.  Needs no GPU.
#include "gradhip.hpp"

#include <cstdio>
#include <string>
#include <vector>

int main(int argc, char** argv) {
    if (argc < 3) return 2;
    try {
        const std::unique_ptr<gradhip::Tokenizer> tok = gradhip::load_tokenizer(argv[1]);
        std::printf("kind %s vocab %d eos %d\n", gradhip::tokenizer_kind_flag(tok->kind()), tok->vocab_size(),
                    tok->eos_id().value_or(-1));
        std::printf("identity %s\n", gradhip::to_string(tok->identity()).c_str());
        const std::string text = argv[2];
        const std::vector<int> ids = tok->encode(text);
        std::printf("ids");
        for (int id : ids) std::printf(" %d", id);
        std::printf("\n");
        std::printf("round_trip %d\n", tok->decode(ids) == text ? 1 : 0);
        std::printf("special %d %d\n", tok->special_id("<|endoftext|>").value_or(-1),
                    tok->special_id("<eos>").has_value() ? 1 : 0);
        try {
            const std::vector<int> bad = {tok->vocab_size()};
            (void)tok->decode(bad);
            std::printf("error none\n");
        } catch (const std::out_of_range& e) {
            std::printf("out_of_range %s\n", e.what());
        }
        try {
            (void)gradhip::load_tokenizer("/nonexistent/tok.tok");
            std::printf("error none\n");
        } catch (const std::runtime_error& e) {
            std::printf("runtime_error %s\n", e.what());
        }
        try {
            (void)gradhip::ByteBpe({{97, 98}, {97, 98}}, {});
            std::printf("error none\n");
        } catch (const std::invalid_argument& e) {
            std::printf("invalid_argument %s\n", e.what());
        }
        const gradhip::ByteBpe tiny({{97, 98}});
        std::printf("tiny %s\n", gradhip::to_string(tiny.identity()).c_str());
        if (argc >= 4) {  // a v1 cache through the same loader
            const std::unique_ptr<gradhip::Tokenizer> v1 = gradhip::load_tokenizer(argv[3]);
            std::printf("v1 %s vocab %d eos %d unk %d\n", gradhip::to_string(v1->identity()).c_str(), v1->vocab_size(),
                        v1->eos_id().value_or(-1), v1->special_id("<unk>").value_or(-1));
            const std::vector<int> v1_ids = v1->encode(text);
            std::printf("v1ids");
            for (int id : v1_ids) std::printf(" %d", id);
            std::printf("\nv1text %s\n", v1->decode(v1_ids).c_str());
            try {
                (void)gradhip::ByteBpe::load(argv[3]);
                std::printf("error none\n");
            } catch (const std::runtime_error& e) {
                std::printf("runtime_error %s\n", e.what());
            }
        }
    } catch (const std::exception& e) {
        std::printf("FATAL %s\n", e.what());
        return 1;
    }
    return 0;
}

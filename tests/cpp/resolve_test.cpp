// Drives cli/resolve.h (which tokenizer file belongs to a checkpoint) from the
// command line; needs no GPU.  argv: <directory with prepared files> <corpus name>
#include "resolve.h"

#include <iostream>

using namespace gradhip;
using namespace gradhip::cli;

namespace {

template <class F>
void show(const char* label, F f) {
    try {
        const auto value = f();  // may print a line of its own first
        std::cout << label << " " << value << std::endl;
    } catch (const Usage& e) {
        std::cout << label << " usage: " << e.what() << std::endl;
    } catch (const std::exception& e) {
        std::cout << label << " error: " << e.what() << std::endl;
    }
}

std::string flag(TokenizerKind k) { return tokenizer_kind_flag(k); }

}  // namespace

int main(int argc, char** argv) {
    if (argc != 3) return 2;
    const std::string dir = argv[1], corpus = dir + "/" + argv[2];
    // names
    std::cout << "v2 " << tokenizer_path("data/c.txt", 8000, TokenizerKind::ByteBpe) << std::endl;
    std::cout << "v1 " << tokenizer_path("data/c.txt", 8000, TokenizerKind::BpeV1) << std::endl;
    std::cout << "v1-default " << tokenizer_path(kDefaultCorpus, 5000, TokenizerKind::BpeV1) << std::endl;
    std::cout << "v2-default " << tokenizer_path(kDefaultCorpus, 5000, TokenizerKind::ByteBpe) << std::endl;
    std::cout << "bin-v1 " << token_bin_path("data/c.txt", 8000, "train", TokenizerKind::BpeV1) << std::endl;
    std::cout << "bin-v2 " << token_bin_path("data/c.txt", 8000, "val", TokenizerKind::ByteBpe) << std::endl;
    // the flag
    show("flag-v1", [] { return flag(*parse_tokenizer_flag(std::string("v1"))); });
    show("flag-v2", [] { return flag(*parse_tokenizer_flag(std::string("v2"))); });
    show("flag-none", [] { return parse_tokenizer_flag(std::nullopt) ? "set" : "unset"; });
    show("flag-bad", [] { return flag(*parse_tokenizer_flag(std::string("v3"))); });
    // the choice with a checkpoint
    const TokenizerFingerprint fp2{TokenizerKind::ByteBpe, 0x1122334455667788ull};
    const TokenizerFingerprint fp1{TokenizerKind::BpeV1, 0x99ull};
    show("ckpt-recorded-v2", [&] { return flag(choose_tokenizer(corpus, 300, std::nullopt, true, fp2)); });
    show("ckpt-recorded-v2-asked-v2", [&] { return flag(choose_tokenizer(corpus, 300, TokenizerKind::ByteBpe, true, fp2)); });
    show("ckpt-recorded-v2-asked-v1", [&] { return flag(choose_tokenizer(corpus, 300, TokenizerKind::BpeV1, true, fp2)); });
    show("ckpt-recorded-v1", [&] { return flag(choose_tokenizer(corpus, 300, std::nullopt, true, fp1)); });
    show("ckpt-unrecorded", [&] { return flag(choose_tokenizer(corpus, 300, std::nullopt, true, std::nullopt)); });
    show("ckpt-unrecorded-asked-v2", [&] { return flag(choose_tokenizer(corpus, 300, TokenizerKind::ByteBpe, true, std::nullopt)); });
    // the choice from the files alone: vocab 300 has a v2 file, 301 a v1 cache, 302 both,
    // 303 nothing, 304 the two v1 token files, 305 one v2 token file only
    for (int vocab = 300; vocab <= 305; vocab++) {
        const std::string label = "files-" + std::to_string(vocab);
        show(label.c_str(), [&] { return flag(choose_tokenizer(corpus, vocab, std::nullopt, false, std::nullopt)); });
    }
    show("files-302-asked-v1", [&] { return flag(choose_tokenizer(corpus, 302, TokenizerKind::BpeV1, false, std::nullopt)); });
    // loading
    show("load-v2", [&] { return load_tokenizer_for_inference(corpus, 300, TokenizerKind::ByteBpe)->vocab_size(); });
    show("load-v1", [&] { return load_tokenizer_for_inference(corpus, 301, TokenizerKind::BpeV1)->vocab_size(); });
    show("load-missing", [&] { return load_tokenizer_for_inference(corpus, 303, TokenizerKind::ByteBpe)->vocab_size(); });
    show("load-wrong-kind", [&] { return load_tokenizer_for_inference(corpus, 306, TokenizerKind::ByteBpe)->vocab_size(); });
    show("vocab-mismatch", [&] {
        require_matching_vocab(*load_tokenizer_for_inference(corpus, 300, TokenizerKind::ByteBpe), 999);
        return 0;
    });
    return 0;
}

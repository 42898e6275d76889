// Which tokenizer file belongs to a checkpoint: grad.cpp's commands do not take a
// tokenizer path, they derive it from the corpus path, the vocabulary size and the
// tokenizer generation (src/cli/common.cpp:101-124), choose the generation from the
// checkpoint's recorded fingerprint, the --tokenizer flag and the files on disk
// (choose_tokenizer, :160-187) and load the file for inference (:43-59, :236-252).
// The same rules here, so the gradhip commands can be called the way `grad
// generate <checkpoint> <prompt> [corpus] [vocab]` is.  Host code only.
//
// One difference: grad.cpp trains a tokenizer on the spot when a small corpus has
// none (load_or_train_tokenizer, :196-234).  Training is not part of this library;
// a missing file is reported with the command that makes it, whatever the corpus size.
#pragma once

#include "gradhip.hpp"
#include "options.h"

#include <sys/stat.h>

#include <fstream>
#include <iostream>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>

namespace gradhip::cli {

inline constexpr const char* kDefaultCorpus = "data/shakespeare.txt";  // src/cli/common.h:22

inline bool readable(const std::string& path) { return std::ifstream(path).good(); }

inline bool present(const std::string& path) {
    struct stat st {};
    return ::stat(path.c_str(), &st) == 0;
}

inline bool is_default_corpus(const std::string& corpus) { return corpus == kDefaultCorpus; }

// The v1 cache of the default corpus lives beside the working directory as
// "tokenizer_<vocab>.cache"; every other name hangs off the corpus path.
inline std::string tokenizer_path(const std::string& corpus, int vocab, TokenizerKind kind) {
    const std::string n = std::to_string(vocab);
    if (kind == TokenizerKind::ByteBpe) return corpus + ".bytebpe_" + n + ".tok";
    return (is_default_corpus(corpus) ? std::string("tokenizer") : corpus + ".tokenizer") + "_" + n + ".cache";
}

// Token files written by `grad prepare`: "<corpus>.<vocab>.<split>.bin" for v1, with ".v2" before the vocab for v2.
inline std::string token_bin_path(const std::string& corpus, int vocab, const std::string& split, TokenizerKind kind) {
    return corpus + (kind == TokenizerKind::ByteBpe ? ".v2." : ".") + std::to_string(vocab) + "." + split + ".bin";
}

inline bool is_prepared(const std::string& corpus, int vocab, TokenizerKind kind) {
    return present(token_bin_path(corpus, vocab, "train", kind)) && present(token_bin_path(corpus, vocab, "val", kind));
}

// A generation "is there" for a corpus when its tokenizer file or both of its token files exist.
inline bool has_artifacts(const std::string& corpus, int vocab, TokenizerKind kind) {
    return readable(tokenizer_path(corpus, vocab, kind)) || is_prepared(corpus, vocab, kind);
}

inline std::optional<TokenizerKind> parse_tokenizer_flag(const std::optional<std::string>& flag) {
    if (!flag) return std::nullopt;
    if (*flag == "v1") return TokenizerKind::BpeV1;
    if (*flag == "v2") return TokenizerKind::ByteBpe;
    throw Usage("--tokenizer: expected v1 or v2, got '" + *flag + "'");
}

// In order: the checkpoint's recorded generation (a different --tokenizer is an
// error); the flag; v1 for a checkpoint that records nothing (it predates v2);
// without a checkpoint, whichever generation has files for this corpus and
// vocabulary, v2 when neither has, an error when both have.
inline TokenizerKind choose_tokenizer(const std::string& corpus, int vocab, std::optional<TokenizerKind> requested,
                                      bool have_checkpoint, const std::optional<TokenizerFingerprint>& recorded) {
    if (have_checkpoint && recorded) {
        if (requested && *requested != recorded->kind)
            throw std::runtime_error(std::string("--tokenizer ") + tokenizer_kind_flag(*requested)
                                     + " does not match the checkpoint, which was trained with tokenizer "
                                     + to_string(*recorded));
        return recorded->kind;
    }
    if (requested) return *requested;
    if (have_checkpoint) return TokenizerKind::BpeV1;
    const bool v1 = has_artifacts(corpus, vocab, TokenizerKind::BpeV1);
    const bool v2 = has_artifacts(corpus, vocab, TokenizerKind::ByteBpe);
    if (v1 && v2)
        throw std::runtime_error("both a v1 tokenizer (" + tokenizer_path(corpus, vocab, TokenizerKind::BpeV1)
                                 + ") and a v2 tokenizer (" + tokenizer_path(corpus, vocab, TokenizerKind::ByteBpe)
                                 + ") exist for " + corpus + " at vocab " + std::to_string(vocab)
                                 + "; pass --tokenizer v1 or --tokenizer v2");
    return v1 ? TokenizerKind::BpeV1 : TokenizerKind::ByteBpe;
}

// The tokenizer file of (corpus, vocab, kind), loaded and checked to hold that generation.
inline std::unique_ptr<Tokenizer> load_tokenizer_for_inference(const std::string& corpus, int vocab, TokenizerKind kind) {
    const std::string path = tokenizer_path(corpus, vocab, kind);
    const std::string remedy = "; run: ./build/grad prepare " + corpus + " " + std::to_string(vocab) + " --tokenizer "
                               + tokenizer_kind_flag(kind);
    if (!readable(path)) {
        struct stat st {};
        if (::stat(corpus.c_str(), &st) == 0 && static_cast<std::size_t>(st.st_size) > (32ull << 20))
            throw std::runtime_error("No tokenizer " + path + " for a " + std::to_string(st.st_size >> 20)
                                     + "MB corpus" + remedy);
        throw std::runtime_error("No " + std::string(tokenizer_kind_flag(kind)) + " tokenizer " + path + remedy);
    }
    std::unique_ptr<Tokenizer> tokenizer = load_tokenizer(path);
    if (tokenizer->kind() != kind)
        throw std::runtime_error(path + " holds a " + tokenizer_kind_flag(tokenizer->kind()) + " tokenizer, not "
                                 + tokenizer_kind_flag(kind));
    std::cout << "Tokenizer: " << path << " (" << tokenizer_kind_flag(kind) << ", vocab " << tokenizer->vocab_size()
              << ")" << std::endl;
    return tokenizer;
}

// require_matching_vocab (src/cli/common.cpp:61-68).
inline void require_matching_vocab(const Tokenizer& tokenizer, int model_vocab) {
    if (tokenizer.vocab_size() != model_vocab)
        throw std::runtime_error("tokenizer has " + std::to_string(tokenizer.vocab_size())
                                 + " tokens but the checkpoint expects " + std::to_string(model_vocab)
                                 + "; the cache was built for a different vocab or corpus");
}

}  // namespace gradhip::cli

// gradhip.hpp — header-only C++20 adapter over the C ABI of gradhip.h.
//
// It gives callers written against grad.cpp's generation API the same class
// names, signatures, ownership rules and exception types, so that a caller like
// src/cli/generate.cpp or src/cli/chat.cpp changes one include and one
// namespace:
//
//     grad::GPTModel::load            -> gradhip::GPTModel::load      (gpt_model.h:87)
//     grad::InferenceSession          -> gradhip::InferenceSession    (inference.h:16-29)
//     grad::TextGen                   -> gradhip::TextGen             (text_gen.h:12-38)
//     grad::Tokenizer                 -> gradhip::Tokenizer           (tokenizer.h:20-43)
//     grad::ByteBpe, grad::BpeV1,     -> gradhip::ByteBpe, gradhip::BpeV1, gradhip::load_tokenizer
//     load_tokenizer                                                   (byte_bpe.h:37-113, bpe_v1.h, tokenizer.h:52)
//
// The model lives on the GPU; there is no CPU path behind these classes.
#pragma once

#include "gradhip.h"

#include <cstdint>
#include <cstdio>
#include <exception>
#include <functional>
#include <memory>
#include <optional>
#include <random>
#include <span>
#include <stdexcept>
#include <string>
#include <string_view>
#include <utility>
#include <vector>

namespace gradhip {

// Maps a C-ABI status to the exception grad.cpp throws at the same point.
inline void check(gh_status st) {
    if (st == GH_OK) return;
    const std::string msg = gh_last_error();
    switch (st) {
        case GH_ERR_OUT_OF_RANGE: throw std::out_of_range(msg);
        case GH_ERR_INVALID_ARGUMENT: throw std::invalid_argument(msg);
        default: throw std::runtime_error(msg);
    }
}

enum class GPTArch { GPT2 = 0, Modern = 1 };            // gpt_model.h:31
enum class TokenizerKind { BpeV1 = 1, ByteBpe = 2 };    // grad/tokenizer/fingerprint.h

struct TokenizerFingerprint {
    TokenizerKind kind;
    std::uint64_t hash;
    bool operator==(const TokenizerFingerprint&) const = default;
};

// "v1" / "v2" and "v2:0123456789abcdef" (tokenizer.cpp:17-32).
inline const char* tokenizer_kind_flag(TokenizerKind kind) {
    return kind == TokenizerKind::BpeV1 ? "v1" : kind == TokenizerKind::ByteBpe ? "v2" : "unknown";
}
inline std::string to_string(const TokenizerFingerprint& f) {
    char hex[17];
    std::snprintf(hex, sizeof hex, "%016llx", static_cast<unsigned long long>(f.hash));
    return std::string(tokenizer_kind_flag(f.kind)) + ":" + hex;
}

// grad::Tokenizer (tokenizer.h:20-43).  The generation path only calls decode
// (text_gen.cpp:122-125), so a wrapper around another tokenizer need only
// override that; the other members throw std::logic_error unless overridden.
class Tokenizer {
public:
    virtual ~Tokenizer() = default;
    [[nodiscard]] virtual std::string decode(std::span<const int> ids) const = 0;
    [[nodiscard]] virtual std::vector<int> encode(std::string_view) const { unsupported("encode"); }
    [[nodiscard]] virtual TokenizerKind kind() const { unsupported("kind"); }
    [[nodiscard]] virtual int vocab_size() const { unsupported("vocab_size"); }
    [[nodiscard]] virtual std::optional<int> eos_id() const { unsupported("eos_id"); }
    [[nodiscard]] virtual std::optional<int> special_id(std::string_view) const { unsupported("special_id"); }
    [[nodiscard]] virtual std::uint64_t fingerprint() const { unsupported("fingerprint"); }
    [[nodiscard]] TokenizerFingerprint identity() const { return {kind(), fingerprint()}; }
    virtual void save(const std::string&) const { unsupported("save"); }

private:
    [[noreturn]] static void unsupported(const char* what) {
        throw std::logic_error(std::string("gradhip::Tokenizer::") + what + " is not implemented by this tokenizer");
    }
};

// grad::ByteBpe (byte_bpe.h:37-113) without the trainer: the lossless byte-level
// BPE of "GTOK" version 2 files.  Runs on the host.
class ByteBpe final : public Tokenizer {
public:
    using Merge = std::pair<int, int>;
    static constexpr std::string_view kEndOfText = "<|endoftext|>";

    // Throws std::invalid_argument with the reference constructor's messages.
    explicit ByteBpe(const std::vector<Merge>& merges,
                     const std::vector<std::string>& specials = {std::string(kEndOfText)}) {
        std::vector<int32_t> flat;
        for (const Merge& m : merges) {
            flat.push_back(m.first);
            flat.push_back(m.second);
        }
        std::vector<const char*> ptrs;
        std::vector<int32_t> lens;
        for (const std::string& sp : specials) {
            ptrs.push_back(sp.data());
            lens.push_back(static_cast<int32_t>(sp.size()));
        }
        check(gh_tokenizer_from_merges(flat.data(), static_cast<int32_t>(merges.size()), ptrs.data(), lens.data(),
                                       static_cast<int32_t>(specials.size()), &t_));
        check(gh_tokenizer_get_info(t_, &info_));
    }
    // Throws std::runtime_error("Tokenizer file <path>: ...") like ByteBpe::load (byte_bpe.cpp:676-744).
    [[nodiscard]] static ByteBpe load(const std::string& path) {
        gh_tokenizer* t = nullptr;
        check(gh_tokenizer_load(path.c_str(), &t));
        ByteBpe out(t);
        if (out.info_.kind != 2) throw std::runtime_error("Tokenizer file " + path + ": not a GTOK tokenizer file");
        return out;
    }
    ByteBpe(const ByteBpe&) = delete;
    ByteBpe& operator=(const ByteBpe&) = delete;
    ByteBpe(ByteBpe&& o) noexcept : t_(std::exchange(o.t_, nullptr)), info_(o.info_) {}
    ~ByteBpe() override { gh_tokenizer_free(t_); }

    [[nodiscard]] TokenizerKind kind() const override { return TokenizerKind::ByteBpe; }
    [[nodiscard]] std::vector<int> encode(std::string_view text) const override { return run_encode(text, 1); }
    [[nodiscard]] std::vector<int> encode_ordinary(std::string_view text) const { return run_encode(text, 0); }
    // Throws std::out_of_range for an id outside the vocabulary.
    [[nodiscard]] std::string decode(std::span<const int> ids) const override {
        std::size_t len = 0;
        check(gh_tokenizer_decode(t_, ids.data(), ids.size(), nullptr, 0, &len));
        std::string out(len, '\0');
        check(gh_tokenizer_decode(t_, ids.data(), ids.size(), out.data(), out.size(), &len));
        return out;
    }
    [[nodiscard]] int vocab_size() const override { return info_.vocab_size; }
    [[nodiscard]] std::optional<int> eos_id() const override {
        return info_.eos_id < 0 ? std::nullopt : std::optional<int>(info_.eos_id);
    }
    [[nodiscard]] std::optional<int> special_id(std::string_view token) const override {
        int32_t id = -1;
        check(gh_tokenizer_special_id(t_, token.data(), token.size(), &id));
        return id < 0 ? std::nullopt : std::optional<int>(id);
    }
    [[nodiscard]] std::uint64_t fingerprint() const override { return info_.fingerprint; }
    void save(const std::string& path) const override { check(gh_tokenizer_save(t_, path.c_str())); }

private:
    explicit ByteBpe(gh_tokenizer* t) : t_(t) { check(gh_tokenizer_get_info(t_, &info_)); }
    std::vector<int> run_encode(std::string_view text, int32_t with_specials) const {
        std::vector<int> ids(text.size());  // never more ids than bytes
        std::size_t n = 0;
        check(gh_tokenizer_encode(t_, text.data(), text.size(), with_specials, ids.data(), ids.size(), &n));
        ids.resize(n);
        return ids;
    }
    gh_tokenizer* t_ = nullptr;
    gh_tokenizer_info info_{};
};

// grad::BpeV1 (bpe_v1.h) without the trainer: the original whitespace BPE read
// from a tokenizer cache.  decode is lossy ('_' and white-space runs read back as
// one space); ids missing from the vocabulary are skipped.
class BpeV1 final : public Tokenizer {
public:
    // Throws std::runtime_error with BPETokenizer::load's messages (bpe_tokenizer.cpp:373-417).
    [[nodiscard]] static BpeV1 load(const std::string& path) {
        gh_tokenizer* t = nullptr;
        check(gh_tokenizer_load(path.c_str(), &t));
        BpeV1 out(t);
        if (out.info_.kind != 1) throw std::runtime_error(path + " holds a v2 tokenizer, not v1");
        return out;
    }
    BpeV1(const BpeV1&) = delete;
    BpeV1& operator=(const BpeV1&) = delete;
    BpeV1(BpeV1&& o) noexcept : t_(std::exchange(o.t_, nullptr)), info_(o.info_) {}
    ~BpeV1() override { gh_tokenizer_free(t_); }

    [[nodiscard]] TokenizerKind kind() const override { return TokenizerKind::BpeV1; }
    [[nodiscard]] std::vector<int> encode(std::string_view text) const override {
        std::vector<int> ids(text.size());  // at most one id per byte
        std::size_t n = 0;
        check(gh_tokenizer_encode(t_, text.data(), text.size(), 1, ids.data(), ids.size(), &n));
        ids.resize(n);
        return ids;
    }
    [[nodiscard]] std::string decode(std::span<const int> ids) const override {
        std::size_t len = 0;
        check(gh_tokenizer_decode(t_, ids.data(), ids.size(), nullptr, 0, &len));
        std::string out(len, '\0');
        check(gh_tokenizer_decode(t_, ids.data(), ids.size(), out.data(), out.size(), &len));
        return out;
    }
    [[nodiscard]] int vocab_size() const override { return info_.vocab_size; }
    [[nodiscard]] std::optional<int> eos_id() const override {
        return info_.eos_id < 0 ? std::nullopt : std::optional<int>(info_.eos_id);
    }
    [[nodiscard]] std::optional<int> special_id(std::string_view token) const override {
        int32_t id = -1;
        check(gh_tokenizer_special_id(t_, token.data(), token.size(), &id));
        return id < 0 ? std::nullopt : std::optional<int>(id);
    }
    [[nodiscard]] std::uint64_t fingerprint() const override { return info_.fingerprint; }
    void save(const std::string& path) const override { check(gh_tokenizer_save(t_, path.c_str())); }

private:
    explicit BpeV1(gh_tokenizer* t) : t_(t) { check(gh_tokenizer_get_info(t_, &info_)); }
    gh_tokenizer* t_ = nullptr;
    gh_tokenizer_info info_{};
};

// load_tokenizer (tokenizer.h:52, tokenizer.cpp:119-124): a "GTOK" file is the
// byte-level BPE, anything else is taken for a v1 cache.
[[nodiscard]] inline std::unique_ptr<Tokenizer> load_tokenizer(const std::string& path) {
    gh_tokenizer* t = nullptr;
    check(gh_tokenizer_load(path.c_str(), &t));
    gh_tokenizer_info info{};
    const gh_status st = gh_tokenizer_get_info(t, &info);
    gh_tokenizer_free(t);
    check(st);
    if (info.kind == 1) return std::make_unique<BpeV1>(BpeV1::load(path));
    return std::make_unique<ByteBpe>(ByteBpe::load(path));
}

class GPTModel {
public:
    // Throws std::runtime_error with GPTModel::load's messages (gpt_model.cpp:383-525).
    [[nodiscard]] static GPTModel load(const std::string& filepath) {
        gh_model* m = nullptr;
        check(gh_model_load(filepath.c_str(), &m));
        return GPTModel(m);
    }

    // Checkpoint-order host tensors, (in, out) row-major (gpt_model.cpp:318-355).
    [[nodiscard]] static GPTModel from_host(const gh_config& cfg, const std::vector<const float*>& tensors) {
        gh_model* m = nullptr;
        check(gh_model_from_host(&cfg, tensors.data(), static_cast<int32_t>(tensors.size()), &m));
        return GPTModel(m);
    }

    // GPTModel::save (gpt_model.cpp:292-381); false when the file cannot be written.
    [[nodiscard]] bool save(const std::string& filepath, bool /*quiet*/ = false) const {
        return gh_model_save(m_, filepath.c_str()) == GH_OK;
    }

    int getVocabSize() const { return cfg_.vocab; }
    int getDModel() const { return cfg_.d_model; }
    int getNumLayers() const { return cfg_.layers; }
    int getNumHeads() const { return cfg_.heads; }
    int getMaxLen() const { return cfg_.max_len; }
    GPTArch getArch() const { return static_cast<GPTArch>(cfg_.arch); }
    std::optional<TokenizerFingerprint> getTokenizerFingerprint() const {
        if (!cfg_.has_fingerprint) return std::nullopt;
        return TokenizerFingerprint{static_cast<TokenizerKind>(cfg_.tokenizer_kind), cfg_.tokenizer_hash};
    }

    GPTModel(const GPTModel&) = delete;
    GPTModel& operator=(const GPTModel&) = delete;
    GPTModel(GPTModel&& o) noexcept : m_(std::exchange(o.m_, nullptr)), cfg_(o.cfg_) {}
    GPTModel& operator=(GPTModel&& o) noexcept {
        if (this != &o) {
            gh_model_free(m_);
            m_ = std::exchange(o.m_, nullptr);
            cfg_ = o.cfg_;
        }
        return *this;
    }
    ~GPTModel() { gh_model_free(m_); }

    gh_model* handle() const { return m_; }

private:
    explicit GPTModel(gh_model* m) : m_(m) { check(gh_model_get_config(m_, &cfg_)); }
    gh_model* m_ = nullptr;
    gh_config cfg_{};
};

// The CLI's guard before generating (src/cli/common.cpp:254-268): a checkpoint
// that records a tokenizer fingerprint is only used with that tokenizer.  Returns
// false (after a warning on stderr) when the checkpoint records none; throws
// std::runtime_error with the reference's message on a mismatch.
inline bool check_tokenizer_matches(const GPTModel& model, const Tokenizer& tokenizer,
                                    const std::string& checkpoint_path) {
    const std::optional<TokenizerFingerprint> recorded = model.getTokenizerFingerprint();
    if (!recorded) {
        std::fprintf(stderr,
                     "Warning: %s records no tokenizer fingerprint (it predates tokenizer v2); using the %s "
                     "tokenizer unverified\n",
                     checkpoint_path.c_str(), tokenizer_kind_flag(tokenizer.kind()));
        return false;
    }
    if (!(*recorded == tokenizer.identity())) {
        throw std::runtime_error("tokenizer " + to_string(tokenizer.identity()) + " is not the one "
                                 + checkpoint_path + " was trained with (" + to_string(*recorded)
                                 + "); its token ids would mean different text");
    }
    return true;
}

// Incremental decoding with a KV cache (inference.h:16-29).  The model must
// outlive the session; the pointer step() returns is valid until the next step().
class InferenceSession {
public:
    explicit InferenceSession(const GPTModel& model) : model_(model) {
        gh_session_opts o{};
        o.batch = 1;
        check(gh_session_create(model.handle(), &o, &s_));
    }
    InferenceSession(const InferenceSession&) = delete;
    InferenceSession& operator=(const InferenceSession&) = delete;
    ~InferenceSession() { gh_session_free(s_); }

    // Throws std::runtime_error("InferenceSession: context exceeds max_len") or
    // std::out_of_range("InferenceSession: token id out of vocab range") (inference.cpp:151-156).
    [[nodiscard]] const float* step(int token_id) {
        const int32_t id = token_id;
        check(gh_session_step(s_, &id, nullptr));
        const float* logits = nullptr;
        check(gh_session_logits(s_, &logits));
        return logits;
    }

    // Negative log-likelihood of targets[t] at every position of ids, all positions
    // in one pass (what training::mean_loss averages, src/training/trainer.cpp:319-340).
    // Continues from the current position and fills the cache like step() would.
    [[nodiscard]] std::vector<float> score(const std::vector<int>& ids, const std::vector<int>& targets) {
        if (ids.size() != targets.size()) throw std::invalid_argument("score: ids and targets differ in length");
        std::vector<float> nll(ids.size());
        check(gh_session_score(s_, ids.data(), targets.data(), static_cast<int32_t>(ids.size()), nll.data()));
        return nll;
    }

    int position() const { return gh_session_position(s_); }
    int capacity() const { return gh_session_capacity(s_); }
    int vocabSize() const { return gh_session_vocab(s_); }

    gh_session* handle() const { return s_; }

private:
    const GPTModel& model_;
    gh_session* s_ = nullptr;
};

class TextGen {
public:
    // Without a tokenizer, each token id is printed as the byte it equals (text_gen.cpp:127-132).
    explicit TextGen(const GPTModel& model, const Tokenizer* tok = nullptr) : model_(model), tokenizer_(tok) {}

    // grad.cpp draws from a process-wide std::mt19937 seeded by std::random_device
    // (text_gen.cpp:195-197), so its streams are not repeatable.  Here the draws
    // come from a counter-based generator on the GPU whose seed is random unless fixed.
    void set_seed(std::uint64_t seed) { seed_ = seed; }

    std::string generate_greedy(const std::vector<int>& prompt_tokens, int max_tokens = 50,
                                float repetition_penalty = 1.2f) {
        gh_sampling o{1.0f, 0, 1.0f, repetition_penalty, 1};
        return tokens_to_string(run(prompt_tokens, max_tokens, o));
    }

    std::string generate_sample(const std::vector<int>& prompt_tokens, float temperature = 1.0f,
                                int max_tokens = 50, float repetition_penalty = 1.2f, int top_k = 0,
                                float top_p = 1.0f) {
        gh_sampling o{temperature, top_k, top_p, repetition_penalty, 0};
        return tokens_to_string(run(prompt_tokens, max_tokens, o));
    }

    // Invokes on_text with each token's text as soon as it is sampled; returns
    // the number of tokens generated (text_gen.cpp:93-120).  The loop runs on the
    // GPU in one launch where the engine allows; on_text runs beside it.
    int generate_stream(const std::vector<int>& prompt_tokens,
                        const std::function<void(const std::string&)>& on_text, float temperature = 1.0f,
                        int max_tokens = 50, float repetition_penalty = 1.2f, int top_k = 0,
                        float top_p = 1.0f) {
        if (prompt_tokens.empty()) return 0;
        InferenceSession session(model_);
        std::vector<int32_t> ids(prompt_tokens.begin(), prompt_tokens.end());
        check(gh_session_prefill(session.handle(), ids.data(), static_cast<int32_t>(ids.size()), nullptr));
        gh_sampling o{temperature, top_k, top_p, repetition_penalty, 0};
        struct Relay {
            TextGen* self;
            const std::function<void(const std::string&)>* on_text;
            std::exception_ptr error;
        } relay{this, &on_text, nullptr};
        const gh_token_callback hand_on = [](void* user, const int32_t* picked, int32_t) -> int32_t {
            Relay& r = *static_cast<Relay*>(user);
            if (r.error) return 1;
            try {
                (*r.on_text)(r.self->tokens_to_string({static_cast<int>(picked[0])}));
                return 0;
            } catch (...) {
                r.error = std::current_exception();  // rethrown once the run has ended
                return 1;
            }
        };
        int32_t generated = 0;
        check(gh_session_decode_stream(session.handle(), max_tokens, &o, nullptr, next_seed(), stop_token_, hand_on,
                                       &relay, nullptr, &generated));
        if (relay.error) std::rethrow_exception(relay.error);
        return generated;
    }

    // Not in grad.cpp, whose loops always run to max_tokens or capacity:
    // generate_stream ends after the round that picks this id (an end-of-text id).
    void set_stop_token(std::optional<int> id) { stop_token_ = id ? *id : -1; }

    // The token ids of the last generate_greedy / generate_sample call.
    const std::vector<int>& last_tokens() const { return last_; }

private:
    std::vector<int> run(const std::vector<int>& prompt, int max_tokens, const gh_sampling& o) {
        last_.clear();
        if (prompt.empty()) return {};  // text_gen.cpp:40
        InferenceSession session(model_);
        std::vector<int32_t> ids(prompt.begin(), prompt.end());
        const int cap = static_cast<int>(ids.size()) + (max_tokens > 0 ? max_tokens : 0);
        std::vector<int32_t> out(static_cast<size_t>(cap));
        int32_t n = 0;
        check(gh_session_generate(session.handle(), ids.data(), static_cast<int32_t>(ids.size()), max_tokens,
                                  &o, nullptr, next_seed(), out.data(), &n, nullptr, nullptr));
        last_.assign(out.begin(), out.begin() + n);
        return last_;
    }

    std::string tokens_to_string(const std::vector<int>& tokens) const {
        if (tokenizer_ != nullptr) return tokenizer_->decode(tokens);
        std::string result;
        result.reserve(tokens.size());
        for (int token : tokens) result += static_cast<char>(token);
        return result;
    }

    std::uint64_t next_seed() {
        if (seed_) return *seed_;
        std::random_device rd;
        return (static_cast<std::uint64_t>(rd()) << 32) | rd();
    }

    const GPTModel& model_;
    const Tokenizer* tokenizer_;
    std::optional<std::uint64_t> seed_;
    std::vector<int> last_;
    int stop_token_ = -1;
};

}  // namespace gradhip

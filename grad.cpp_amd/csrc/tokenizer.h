// Host-side tokenizer for the token loop's two ends: prompt text -> ids before
// the GPU runs, ids -> text after it.  Reads and writes grad.cpp's "GTOK"
// version 2 files (byte-level BPE, src/tokenizer/byte_bpe.cpp:655-744) and splits
// text with GPT-2's pattern the way src/tokenizer/pretokenize.cpp does.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <string_view>
#include <unordered_map>
#include <utility>
#include <vector>

namespace gh {

namespace pretok {

enum CharClass : std::uint8_t { kOther = 0, kLetter = 1, kNumber = 2, kSpace = 3 };

struct Scalar {
    std::uint32_t value;   // code point; the byte itself for an invalid sequence
    std::uint32_t length;  // bytes consumed, 1..4
    CharClass cls;
};

// Class of a code point: \p{L}, \p{N}, White_Space, or other (pretokenize.cpp:96-102).
CharClass classify(std::uint32_t cp);

// Strict UTF-8 (RFC 3629) at text[pos]; any byte that does not start a valid
// sequence is one scalar of class kOther (pretokenize.cpp:53-90).
Scalar scalar_at(std::string_view text, std::size_t pos);

// End of the piece that starts at pos (pos < text.size()), for the pattern
//   's|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+
// (pretokenize.cpp:104-157).
std::size_t piece_end(std::string_view text, std::size_t pos);

}  // namespace pretok

// 64-bit FNV-1a over little-endian fields (src/tokenizer/byte_io.h:78-101).
class Fnv1a64 {
public:
    void bytes(std::string_view data);
    void u32(std::uint32_t v);
    void str(std::string_view s);  // length prefix, then the bytes
    std::uint64_t value() const { return h_; }

private:
    std::uint64_t h_ = 0xcbf29ce484222325ULL;
};

// Byte-level BPE (grad::ByteBpe, include/grad/tokenizer/byte_bpe.h:37-113): ids
// 0..255 are bytes, 256 + r is merge r, the special tokens follow the merges.
class ByteBpe {
public:
    using Merge = std::pair<int, int>;
    static constexpr int kByteTokens = 256;
    static constexpr std::uint32_t kFileVersion = 2;
    static constexpr std::uint32_t kPretokenizerId = 1;  // pretokenize.h: kGpt2Unicode16
    static constexpr std::uint32_t kKind = 2;            // fingerprint.h: TokenizerKind::ByteBpe

    // Throws std::invalid_argument with ByteBpe::rebuild's messages (byte_bpe.cpp:372-421).
    ByteBpe(std::vector<Merge> merges, std::vector<std::string> specials);

    // Throws std::runtime_error("Tokenizer file <path>: <why>") or
    // std::runtime_error("Failed to open tokenizer file: <path>") (byte_bpe.cpp:676-744).
    static ByteBpe load(const std::string& path);
    // The file image save() writes (byte_bpe.cpp:655-674).
    std::string file_image() const;
    void save(const std::string& path) const;

    // with_specials: special-token text becomes one id each (encode); otherwise it
    // is encoded as ordinary bytes (encode_ordinary).
    std::vector<int> encode(std::string_view text, bool with_specials = true) const;
    // Throws std::out_of_range("token id <id> is outside the vocabulary of <n>").
    std::string decode(const int* ids, std::size_t n) const;

    int vocab_size() const { return static_cast<int>(token_bytes_.size()); }
    std::uint64_t fingerprint() const { return fingerprint_; }
    int special_id(std::string_view token) const;  // -1 when it is not a special token
    const std::vector<Merge>& merges() const { return merges_; }
    const std::vector<std::string>& specials() const { return specials_; }

private:
    int rank_of(int left, int right) const;
    static constexpr std::size_t kScanLimit = 24;  // longer pieces use the heap
    void merge_piece(std::string_view piece, std::vector<int>& out) const;
    void merge_long_piece(std::string_view piece, std::vector<int>& out) const;
    void encode_plain(std::string_view text, std::vector<int>& out) const;

    std::vector<Merge> merges_;
    std::vector<std::string> specials_;
    std::vector<std::string> token_bytes_;
    std::unordered_map<std::uint64_t, int> rank_;
    std::uint64_t fingerprint_ = 0;
};

// The original whitespace BPE (grad::BPETokenizer behind grad::BpeV1,
// include/grad/tokenizer/bpe_tokenizer.h:21-55, src/tokenizer/bpe_tokenizer.cpp): text is
// split at white space, every word but the first gets a leading '_', a word's
// characters are joined by the merge list in order, strings missing from the
// vocabulary become <unk>; decode turns every '_' into a space, so it is lossy.
class BpeV1 {
public:
    static constexpr std::uint32_t kKind = 1;  // fingerprint.h: TokenizerKind::BpeV1
    using Merge = std::pair<std::string, std::string>;

    // vocab: (token string, id) in any order, as the cache stores them.
    BpeV1(std::vector<std::pair<std::string, int>> vocab, std::vector<Merge> merges);
    // Reads a tokenizer cache (bpe_tokenizer.cpp:373-417): host size_t and int
    // fields as an x86-64 / AArch64 Linux build writes them (8 and 4 bytes, little
    // endian).  Throws std::runtime_error with BPETokenizer::load's messages.
    static BpeV1 load(const std::string& path);
    // Entries in id order (grad.cpp writes its hash map's order; it reads any order).
    void save(const std::string& path) const;

    std::vector<int> encode(std::string_view text) const;
    std::string decode(const int* ids, std::size_t n) const;  // unknown ids are skipped

    int vocab_size() const { return static_cast<int>(vocab_.size()); }  // getCurrentVocabSize
    // "<pad>", "<eos>" and "<unk>" when the vocabulary has them (tokenizer.cpp:99-104); else -1.
    int special_id(std::string_view token) const;
    std::uint64_t fingerprint() const { return fingerprint_; }  // tokenizer.cpp:39-60
    std::size_t merge_count() const { return merges_.size(); }

private:
    void encode_word(const std::string& word, std::vector<int>& out) const;

    std::unordered_map<std::string, int> vocab_;
    std::unordered_map<int, std::string> id_to_token_;
    std::vector<Merge> merges_;
    // (left, right) -> ranks in the merge list, ascending; '\0' cannot occur in a
    // word, so it separates the two strings of a key
    std::unordered_map<std::string, std::vector<int>> ranks_;
    std::uint64_t fingerprint_ = 0;
};

// True when the file starts with "GTOK" (tokenizer.cpp: detect_tokenizer_file);
// throws std::runtime_error("Failed to open tokenizer file: <path>").
bool is_gtok_file(const std::string& path);

}  // namespace gh

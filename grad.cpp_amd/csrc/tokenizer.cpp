// Byte-level BPE tokenizer and GPT-2 pre-tokenizer (host code).  Follows the
// behaviour of grad.cpp's src/tokenizer/pretokenize.cpp and byte_bpe.cpp; the
// file format, fingerprint and message texts are the reference's, the
// algorithms are written for this library (the UTF-8 decoder is driven by a
// lead-byte table, the splitter tries the pattern's alternatives in order).
#include "tokenizer.h"

#include "unicode_classes.h"

#include <algorithm>
#include <climits>
#include <cstring>
#include <fstream>
#include <functional>
#include <iterator>
#include <queue>
#include <stdexcept>

namespace gh {

// ---------------------------------------------------------------------------
// pre-tokenizer

namespace pretok {

CharClass classify(std::uint32_t cp) { return static_cast<CharClass>(unicode::class_of(cp)); }

namespace {

// What a lead byte promises: the sequence length (0: this byte cannot start a
// sequence), the payload bits it carries itself, and the range its first
// continuation byte must lie in.  The narrowed ranges are what makes the decoder
// strict (RFC 3629): E0 and F0 refuse overlong forms, ED refuses surrogates, F4
// refuses anything past U+10FFFF; C0, C1 and F5..FF promise nothing.
struct LeadByte {
    std::uint8_t length, payload_mask, second_lo, second_hi;
};

constexpr LeadByte lead_entry(unsigned b) {
    if (b < 0x80) return {1, 0x7F, 0, 0};
    if (b >= 0xC2 && b <= 0xDF) return {2, 0x1F, 0x80, 0xBF};
    if (b >= 0xE0 && b <= 0xEF)
        return {3, 0x0F, static_cast<std::uint8_t>(b == 0xE0 ? 0xA0 : 0x80), static_cast<std::uint8_t>(b == 0xED ? 0x9F : 0xBF)};
    if (b >= 0xF0 && b <= 0xF4)
        return {4, 0x07, static_cast<std::uint8_t>(b == 0xF0 ? 0x90 : 0x80), static_cast<std::uint8_t>(b == 0xF4 ? 0x8F : 0xBF)};
    return {0, 0, 0, 0};
}

struct LeadTable {
    LeadByte at[256];
    constexpr LeadTable() : at{} {
        for (unsigned b = 0; b < 256; b++) at[b] = lead_entry(b);
    }
};
constexpr LeadTable kLead{};

}  // namespace

// Table-driven: the lead byte's entry says how many bytes to take and what the
// second one may be; every further byte must be 10xxxxxx.  Anything else makes
// the lead byte a scalar of its own (class Other), so the scan always advances.
Scalar scalar_at(std::string_view text, std::size_t pos) {
    const auto* bytes = reinterpret_cast<const unsigned char*>(text.data());
    const LeadByte lead = kLead.at[bytes[pos]];
    if (lead.length == 1) return {bytes[pos], 1, classify(bytes[pos])};
    const Scalar lone{bytes[pos], 1, kOther};
    if (lead.length == 0 || text.size() - pos < lead.length) return lone;
    std::uint32_t cp = bytes[pos] & lead.payload_mask;
    for (std::uint32_t k = 1; k < lead.length; k++) {
        const unsigned char b = bytes[pos + k];
        const unsigned char lo = k == 1 ? lead.second_lo : 0x80, hi = k == 1 ? lead.second_hi : 0xBF;
        if (b < lo || b > hi) return lone;
        cp = (cp << 6) | (b & 0x3Fu);
    }
    return {cp, lead.length, classify(cp)};
}

namespace {

// The split pattern, alternative by alternative, in the order a regex engine
// tries them:  's|'t|'re|'ve|'m|'ll|'d | ?\p{L}+ | ?\p{N}+ | ?[^\s\p{L}\p{N}]+ | \s+(?!\S) | \s+
// Each matcher returns the number of bytes it takes at pos, 0 when it does not match.

// Bytes and scalars of the longest run of class `cls` starting at pos.
struct Run {
    std::size_t bytes = 0, scalars = 0, last_scalar_bytes = 0;
};

Run run_of(std::string_view text, std::size_t pos, CharClass cls) {
    Run r;
    while (pos + r.bytes < text.size()) {
        const Scalar s = scalar_at(text, pos + r.bytes);
        if (s.cls != cls) break;
        r.bytes += s.length;
        r.last_scalar_bytes = s.length;
        r.scalars++;
    }
    return r;
}

// 's 't 're 've 'm 'll 'd: lower case only.
std::size_t match_contraction(std::string_view text, std::size_t pos) {
    static constexpr std::string_view kSuffixes[] = {"s", "t", "re", "ve", "m", "ll", "d"};
    if (text[pos] != '\'') return 0;
    const std::string_view rest = text.substr(pos + 1);
    for (const std::string_view suffix : kSuffixes)
        if (rest.substr(0, suffix.size()) == suffix) return 1 + suffix.size();
    return 0;
}

//  ?X+ for one of the three non-space classes: an optional U+0020, then the run.
std::size_t match_spaced_run(std::string_view text, std::size_t pos, CharClass cls) {
    const std::size_t lead_space = text[pos] == ' ' ? 1 : 0;
    const Run run = run_of(text, pos + lead_space, cls);
    if (run.scalars > 0) return lead_space + run.bytes;
    return 0;  // without the space the run would have to start with a space of another class: no match either
}

// \s+(?!\S): white space not followed by text.  The greedy run gives back its last
// scalar when text follows it, and fails when that leaves nothing.
std::size_t match_space_before_space(std::string_view text, std::size_t pos) {
    const Run run = run_of(text, pos, kSpace);
    if (run.scalars == 0) return 0;
    if (pos + run.bytes == text.size()) return run.bytes;
    return run.bytes - run.last_scalar_bytes;  // 0 for a run of one scalar
}

}  // namespace

std::size_t piece_end(std::string_view text, std::size_t pos) {
    if (const std::size_t n = match_contraction(text, pos)) return pos + n;
    for (const CharClass cls : {kLetter, kNumber, kOther})
        if (const std::size_t n = match_spaced_run(text, pos, cls)) return pos + n;
    if (const std::size_t n = match_space_before_space(text, pos)) return pos + n;
    return pos + run_of(text, pos, kSpace).bytes;  // \s+
}

}  // namespace pretok

// ---------------------------------------------------------------------------
// little-endian fields and the fingerprint hash

namespace {

void put_u32(std::string& out, std::uint32_t v) {
    const char b[4] = {static_cast<char>(v), static_cast<char>(v >> 8), static_cast<char>(v >> 16),
                       static_cast<char>(v >> 24)};
    out.append(b, 4);
}

void put_u64(std::string& out, std::uint64_t v) {
    put_u32(out, static_cast<std::uint32_t>(v));
    put_u32(out, static_cast<std::uint32_t>(v >> 32));
}

// Cursor over a file image; every failure names the file and the field
// (byte_io.h:32-74).
class Cursor {
public:
    Cursor(std::string_view data, const std::string& path) : data_(data), path_(path) {}

    [[noreturn]] void fail(const std::string& why) const {
        throw std::runtime_error("Tokenizer file " + path_ + ": " + why);
    }
    std::string_view take(std::size_t n, const char* what) {
        if (data_.size() - at_ < n) fail(std::string("truncated reading ") + what);
        const std::string_view out = data_.substr(at_, n);
        at_ += n;
        return out;
    }
    std::uint32_t u32(const char* what) {
        const auto* b = reinterpret_cast<const unsigned char*>(take(4, what).data());
        return b[0] | (std::uint32_t{b[1]} << 8) | (std::uint32_t{b[2]} << 16) | (std::uint32_t{b[3]} << 24);
    }
    std::uint64_t u64(const char* what) {
        if (data_.size() - at_ < 8) fail(std::string("truncated reading ") + what);
        const std::uint64_t lo = u32(what);
        return lo | (std::uint64_t{u32(what)} << 32);
    }
    std::size_t remaining() const { return data_.size() - at_; }

private:
    std::string_view data_;
    const std::string& path_;
    std::size_t at_ = 0;
};

constexpr std::uint32_t kMaxVocab = 1u << 24;    // byte_bpe.cpp:27
constexpr std::uint32_t kMaxSpecials = 1024;     // byte_bpe.cpp:28
constexpr std::size_t kMaxSpecialBytes = 1024;   // byte_bpe.h:96

std::uint64_t pair_key(int left, int right) {
    return (std::uint64_t{static_cast<std::uint32_t>(left)} << 32) | static_cast<std::uint32_t>(right);
}

std::string slurp(const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("Failed to open tokenizer file: " + path);
    std::string data((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (f.bad()) throw std::runtime_error("Failed to read tokenizer file: " + path);
    return data;
}

}  // namespace

void Fnv1a64::bytes(std::string_view data) {
    for (const char c : data) h_ = (h_ ^ static_cast<unsigned char>(c)) * 0x100000001b3ULL;
}
void Fnv1a64::u32(std::uint32_t v) {
    std::string b;
    put_u32(b, v);
    bytes(b);
}
void Fnv1a64::str(std::string_view s) {
    u32(static_cast<std::uint32_t>(s.size()));
    bytes(s);
}

// ---------------------------------------------------------------------------
// ByteBpe

ByteBpe::ByteBpe(std::vector<Merge> merges, std::vector<std::string> specials)
    : merges_(std::move(merges)), specials_(std::move(specials)) {
    // validation order and texts of ByteBpe::rebuild (byte_bpe.cpp:372-421)
    if (specials_.size() > kMaxSpecials)
        throw std::invalid_argument("too many special tokens (" + std::to_string(specials_.size()) + ")");
    for (std::size_t i = 0; i < specials_.size(); i++) {
        const std::string& s = specials_[i];
        if (s.empty() || s.size() > kMaxSpecialBytes)
            throw std::invalid_argument("special token " + std::to_string(i) + " has " + std::to_string(s.size())
                                        + " bytes; allowed 1 to " + std::to_string(kMaxSpecialBytes));
        for (std::size_t j = 0; j < i; j++)
            if (specials_[j] == s) throw std::invalid_argument("special token '" + s + "' is listed twice");
    }
    const std::size_t vocab = kByteTokens + merges_.size() + specials_.size();
    if (vocab > kMaxVocab) throw std::invalid_argument("vocabulary of " + std::to_string(vocab) + " is too large");

    token_bytes_.reserve(vocab);
    for (int b = 0; b < kByteTokens; b++) token_bytes_.emplace_back(1, static_cast<char>(b));
    rank_.reserve(merges_.size());
    for (std::size_t r = 0; r < merges_.size(); r++) {
        const int left = merges_[r].first, right = merges_[r].second;
        const int known = kByteTokens + static_cast<int>(r);
        if (left < 0 || right < 0 || left >= known || right >= known)
            throw std::invalid_argument("merge " + std::to_string(r) + " joins tokens " + std::to_string(left)
                                        + " and " + std::to_string(right) + ", which it does not follow");
        if (!rank_.emplace(pair_key(left, right), static_cast<int>(r)).second)
            throw std::invalid_argument("merge " + std::to_string(r) + " repeats an earlier merge");
        token_bytes_.push_back(token_bytes_[left] + token_bytes_[right]);
    }
    for (const std::string& s : specials_) token_bytes_.push_back(s);

    // compute_fingerprint (byte_bpe.cpp:333-347)
    Fnv1a64 h;
    h.str("grad.tokenizer.bytebpe");
    h.u32(kFileVersion);
    h.u32(kPretokenizerId);
    h.u32(static_cast<std::uint32_t>(specials_.size()));
    for (const std::string& s : specials_) h.str(s);
    h.u32(static_cast<std::uint32_t>(merges_.size()));
    for (const Merge& m : merges_) {
        h.u32(static_cast<std::uint32_t>(m.first));
        h.u32(static_cast<std::uint32_t>(m.second));
    }
    fingerprint_ = h.value();
}

int ByteBpe::special_id(std::string_view token) const {
    for (std::size_t i = 0; i < specials_.size(); i++)
        if (specials_[i] == token) return kByteTokens + static_cast<int>(merges_.size() + i);
    return -1;
}

int ByteBpe::rank_of(int left, int right) const {
    const auto it = rank_.find(pair_key(left, right));
    return it == rank_.end() ? INT_MAX : it->second;
}

// Merges the adjacent pair of lowest rank, leftmost first, until no pair has a
// rank (byte_bpe.cpp:474-476: this replays the merges in training order).  The
// symbols stay in one array; rank[i] caches the rank of (sym[i], sym[i+1]) and
// only the two entries around a merge are recomputed.
void ByteBpe::merge_piece(std::string_view piece, std::vector<int>& out) const {
    const std::size_t n = piece.size();
    if (n > kScanLimit) {
        merge_long_piece(piece, out);
        return;
    }
    std::vector<int> sym(n), rank(n, INT_MAX);
    for (std::size_t i = 0; i < n; i++) sym[i] = static_cast<unsigned char>(piece[i]);
    for (std::size_t i = 0; i + 1 < n; i++) rank[i] = rank_of(sym[i], sym[i + 1]);
    std::size_t len = n;
    while (len > 1) {
        std::size_t best = 0;
        int best_rank = INT_MAX;
        for (std::size_t i = 0; i + 1 < len; i++) {
            if (rank[i] < best_rank) {
                best_rank = rank[i];
                best = i;
            }
        }
        if (best_rank == INT_MAX) break;
        sym[best] = kByteTokens + best_rank;
        sym.erase(sym.begin() + static_cast<std::ptrdiff_t>(best) + 1);
        rank.erase(rank.begin() + static_cast<std::ptrdiff_t>(best) + 1);
        len--;
        rank[best] = best + 1 < len ? rank_of(sym[best], sym[best + 1]) : INT_MAX;
        if (best > 0) rank[best - 1] = rank_of(sym[best - 1], sym[best]);
    }
    out.insert(out.end(), sym.begin(), sym.begin() + static_cast<std::ptrdiff_t>(len));
}

// The same result for long pieces in O(n log n): symbols in a doubly linked list
// over the byte positions, candidate pairs in a min-heap ordered by (rank,
// position).  A popped candidate is acted on only if both of its symbols are
// still what they were when it was pushed.
void ByteBpe::merge_long_piece(std::string_view piece, std::vector<int>& out) const {
    const std::size_t n = piece.size();
    struct Pair {
        int rank;
        std::uint32_t at;  // position of the left symbol
        int left, right;
        bool operator>(const Pair& o) const { return rank != o.rank ? rank > o.rank : at > o.at; }
    };
    std::vector<int> sym(n);
    std::vector<std::uint32_t> nxt(n), prv(n);
    std::priority_queue<Pair, std::vector<Pair>, std::greater<Pair>> heap;
    const auto none = static_cast<std::uint32_t>(n);
    for (std::size_t i = 0; i < n; i++) {
        sym[i] = static_cast<unsigned char>(piece[i]);
        nxt[i] = static_cast<std::uint32_t>(i + 1);
        prv[i] = i == 0 ? none : static_cast<std::uint32_t>(i - 1);
    }
    const auto offer = [&](std::uint32_t at) {
        const std::uint32_t r = nxt[at];
        if (r >= none) return;
        const int rank = rank_of(sym[at], sym[r]);
        if (rank != INT_MAX) heap.push({rank, at, sym[at], sym[r]});
    };
    for (std::uint32_t i = 0; i + 1 < none; i++) offer(i);
    while (!heap.empty()) {
        const Pair c = heap.top();
        heap.pop();
        const std::uint32_t r = nxt[c.at];
        if (sym[c.at] != c.left || r >= none || sym[r] != c.right) continue;  // stale
        sym[c.at] = kByteTokens + c.rank;
        sym[r] = -1;  // a removed position never matches a candidate again
        nxt[c.at] = nxt[r];
        if (nxt[r] < none) prv[nxt[r]] = c.at;
        if (prv[c.at] != none) offer(prv[c.at]);
        offer(c.at);
    }
    for (std::uint32_t i = 0; i < none; i = nxt[i]) out.push_back(sym[i]);
}

void ByteBpe::encode_plain(std::string_view text, std::vector<int>& out) const {
    // pieces repeat a lot in natural text: remember what each one became
    std::unordered_map<std::string_view, std::pair<std::size_t, std::size_t>> seen;
    std::vector<int> seen_ids;
    for (std::size_t pos = 0; pos < text.size();) {
        const std::size_t end = pretok::piece_end(text, pos);
        const std::string_view piece = text.substr(pos, end - pos);
        pos = end;
        if (piece.size() == 1) {
            out.push_back(static_cast<unsigned char>(piece[0]));
            continue;
        }
        if (const auto hit = seen.find(piece); hit != seen.end()) {
            out.insert(out.end(), seen_ids.begin() + static_cast<std::ptrdiff_t>(hit->second.first),
                       seen_ids.begin() + static_cast<std::ptrdiff_t>(hit->second.first + hit->second.second));
            continue;
        }
        const std::size_t before = out.size();
        merge_piece(piece, out);
        if (seen.size() >= (std::size_t{1} << 20)) {
            seen.clear();
            seen_ids.clear();
        }
        seen.emplace(piece, std::make_pair(seen_ids.size(), out.size() - before));
        seen_ids.insert(seen_ids.end(), out.begin() + static_cast<std::ptrdiff_t>(before), out.end());
    }
}

std::vector<int> ByteBpe::encode(std::string_view text, bool with_specials) const {
    std::vector<int> out;
    if (!with_specials || specials_.empty()) {
        encode_plain(text, out);
        return out;
    }
    // Special tokens are taken left to right: the earliest occurrence of any of
    // them, the longest when two start at the same place (byte_bpe.cpp:60-86).
    const int first_special = kByteTokens + static_cast<int>(merges_.size());
    std::vector<std::size_t> next(specials_.size(), 0);
    std::vector<char> fresh(specials_.size(), 0);
    std::size_t pos = 0;
    for (;;) {
        std::size_t at = std::string_view::npos, len = 0;
        int which = -1;
        for (std::size_t i = 0; i < specials_.size(); i++) {
            if (!fresh[i] || (next[i] != std::string_view::npos && next[i] < pos)) {
                next[i] = text.find(specials_[i], pos);
                fresh[i] = 1;
            }
            if (next[i] == std::string_view::npos) continue;
            if (next[i] < at || (next[i] == at && specials_[i].size() > len)) {
                at = next[i];
                len = specials_[i].size();
                which = static_cast<int>(i);
            }
        }
        const std::size_t stop = which < 0 ? text.size() : at;
        encode_plain(text.substr(pos, stop - pos), out);
        if (which < 0) break;
        out.push_back(first_special + which);
        pos = at + len;
    }
    return out;
}

std::string ByteBpe::decode(const int* ids, std::size_t n) const {
    std::string out;
    for (std::size_t i = 0; i < n; i++) {
        const int id = ids[i];
        if (id < 0 || static_cast<std::size_t>(id) >= token_bytes_.size())
            throw std::out_of_range("token id " + std::to_string(id) + " is outside the vocabulary of "
                                    + std::to_string(token_bytes_.size()));
        out += token_bytes_[static_cast<std::size_t>(id)];
    }
    return out;
}

std::string ByteBpe::file_image() const {
    std::string buf = "GTOK";
    put_u32(buf, kFileVersion);
    put_u32(buf, kPretokenizerId);
    put_u32(buf, static_cast<std::uint32_t>(vocab_size()));
    put_u32(buf, static_cast<std::uint32_t>(merges_.size()));
    put_u32(buf, static_cast<std::uint32_t>(specials_.size()));
    for (std::size_t k = 0; k < specials_.size(); k++) {
        put_u32(buf, static_cast<std::uint32_t>(kByteTokens + merges_.size() + k));
        put_u32(buf, static_cast<std::uint32_t>(specials_[k].size()));
        buf += specials_[k];
    }
    for (const Merge& m : merges_) {
        put_u32(buf, static_cast<std::uint32_t>(m.first));
        put_u32(buf, static_cast<std::uint32_t>(m.second));
    }
    put_u64(buf, fingerprint_);
    return buf;
}

void ByteBpe::save(const std::string& path) const {
    const std::string buf = file_image();
    std::ofstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("Failed to open file for saving: " + path);
    f.write(buf.data(), static_cast<std::streamsize>(buf.size()));
    f.close();
    if (!f) throw std::runtime_error("Failed while writing tokenizer file: " + path);
}

ByteBpe ByteBpe::load(const std::string& path) {
    const std::string data = slurp(path);
    Cursor in(data, path);
    if (in.take(4, "magic") != "GTOK") in.fail("not a GTOK tokenizer file");
    const std::uint32_t version = in.u32("version");
    if (version != kFileVersion) in.fail("unsupported version " + std::to_string(version));
    const std::uint32_t pre = in.u32("pre-tokenizer id");
    if (pre != kPretokenizerId) in.fail("unknown pre-tokenizer id " + std::to_string(pre));
    const std::uint32_t vocab = in.u32("vocab size");
    const std::uint32_t n_merges = in.u32("merge count");
    const std::uint32_t n_specials = in.u32("special token count");
    if (vocab > kMaxVocab || n_merges > kMaxVocab || n_specials > kMaxSpecials
        || std::uint64_t{kByteTokens} + n_merges + n_specials != vocab) {
        in.fail("implausible header: vocab " + std::to_string(vocab) + ", " + std::to_string(n_merges)
                + " merges, " + std::to_string(n_specials) + " special tokens");
    }
    std::vector<std::string> specials;
    specials.reserve(n_specials);
    for (std::uint32_t k = 0; k < n_specials; k++) {
        const std::uint32_t id = in.u32("special token id");
        if (id != kByteTokens + n_merges + k)
            in.fail("special token " + std::to_string(k) + " has id " + std::to_string(id)
                    + "; special ids follow the merges");
        const std::uint32_t len = in.u32("special token length");
        if (len == 0 || len > kMaxSpecialBytes)
            in.fail("special token " + std::to_string(k) + " has an implausible length (" + std::to_string(len)
                    + " bytes)");
        specials.emplace_back(in.take(len, "special token"));
    }
    if (in.remaining() / 8 < n_merges) in.fail("truncated reading merges");
    std::vector<Merge> merges;
    merges.reserve(n_merges);
    for (std::uint32_t r = 0; r < n_merges; r++) {
        const std::uint32_t left = in.u32("merge"), right = in.u32("merge");
        if (left >= kByteTokens + r || right >= kByteTokens + r)
            in.fail("merge " + std::to_string(r) + " joins tokens " + std::to_string(left) + " and "
                    + std::to_string(right) + ", which it does not follow");
        merges.emplace_back(static_cast<int>(left), static_cast<int>(right));
    }
    const std::uint64_t stored = in.u64("fingerprint");
    if (in.remaining() != 0) in.fail("unexpected bytes after the fingerprint");
    try {
        ByteBpe tok(std::move(merges), std::move(specials));
        if (tok.fingerprint() != stored) in.fail("fingerprint does not match the contents (corrupt file)");
        return tok;
    } catch (const std::invalid_argument& e) {
        in.fail(e.what());
    }
}

// ---------------------------------------------------------------------------
// BpeV1

namespace {

constexpr std::uint64_t kMaxCacheEntries = 1u << 24;  // bpe_tokenizer.cpp:343
constexpr std::uint64_t kMaxTokenBytes = 1u << 16;    // bpe_tokenizer.cpp:344

std::string pair_string(const std::string& left, const std::string& right) {
    std::string key;
    key.reserve(left.size() + right.size() + 1);
    key += left;
    key += '\0';
    key += right;
    return key;
}

// Cache fields are the writer's host types: 64-bit size_t, 32-bit int, little endian.
std::uint64_t cache_u64(std::istream& in, const std::string& path, const char* what) {
    unsigned char b[8];
    in.read(reinterpret_cast<char*>(b), 8);
    if (!in) throw std::runtime_error("Tokenizer cache truncated reading " + std::string(what) + ": " + path);
    std::uint64_t v = 0;
    for (int i = 7; i >= 0; i--) v = (v << 8) | b[i];
    return v;
}

std::string cache_token(std::istream& in, const std::string& path) {
    const std::uint64_t len = cache_u64(in, path, "token length");
    if (len > kMaxTokenBytes)
        throw std::runtime_error("Tokenizer cache has an implausible token length (" + std::to_string(len)
                                 + " bytes): " + path);
    std::string token(len, '\0');
    in.read(token.data(), static_cast<std::streamsize>(len));
    if (!in) throw std::runtime_error("Tokenizer cache truncated reading a token: " + path);
    return token;
}

bool c_space(char c) { return c == ' ' || (c >= '\t' && c <= '\r'); }  // what `stream >> word` skips

}  // namespace

BpeV1::BpeV1(std::vector<std::pair<std::string, int>> vocab, std::vector<Merge> merges)
    : merges_(std::move(merges)) {
    for (auto& [token, id] : vocab) {
        id_to_token_[id] = token;
        vocab_[std::move(token)] = id;
    }
    for (std::size_t r = 0; r < merges_.size(); r++)
        ranks_[pair_string(merges_[r].first, merges_[r].second)].push_back(static_cast<int>(r));

    // v1_fingerprint (tokenizer.cpp:39-60): the id-ordered token table, then the merges
    std::vector<std::pair<int, const std::string*>> by_id;
    by_id.reserve(id_to_token_.size());
    for (const auto& [id, token] : id_to_token_) by_id.emplace_back(id, &token);
    std::sort(by_id.begin(), by_id.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    Fnv1a64 h;
    h.str("grad.tokenizer.bpe_v1");
    h.u32(static_cast<std::uint32_t>(by_id.size()));
    for (const auto& [id, token] : by_id) {
        h.u32(static_cast<std::uint32_t>(id));
        h.str(*token);
    }
    h.u32(static_cast<std::uint32_t>(merges_.size()));
    for (const Merge& m : merges_) {
        h.str(m.first);
        h.str(m.second);
    }
    fingerprint_ = h.value();
}

BpeV1 BpeV1::load(const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("Failed to open file for loading: " + path);
    const std::uint64_t n_vocab = cache_u64(f, path, "vocab size");
    if (n_vocab > kMaxCacheEntries)
        throw std::runtime_error("Tokenizer cache has an implausible vocab size (" + std::to_string(n_vocab)
                                 + "): " + path);
    std::vector<std::pair<std::string, int>> vocab;
    vocab.reserve(n_vocab);
    for (std::uint64_t i = 0; i < n_vocab; i++) {
        std::string token = cache_token(f, path);
        unsigned char b[4];
        f.read(reinterpret_cast<char*>(b), 4);
        if (!f) throw std::runtime_error("Tokenizer cache truncated reading token id: " + path);
        const auto id = static_cast<std::int32_t>(b[0] | (std::uint32_t{b[1]} << 8) | (std::uint32_t{b[2]} << 16)
                                                  | (std::uint32_t{b[3]} << 24));
        if (id < 0) throw std::runtime_error("Tokenizer cache has a negative token id: " + path);
        vocab.emplace_back(std::move(token), id);
    }
    const std::uint64_t n_merges = cache_u64(f, path, "merge count");
    if (n_merges > kMaxCacheEntries)
        throw std::runtime_error("Tokenizer cache has an implausible merge count (" + std::to_string(n_merges)
                                 + "): " + path);
    std::vector<Merge> merges;
    merges.reserve(n_merges);
    for (std::uint64_t i = 0; i < n_merges; i++) {
        std::string left = cache_token(f, path);
        std::string right = cache_token(f, path);
        merges.emplace_back(std::move(left), std::move(right));
    }
    return BpeV1(std::move(vocab), std::move(merges));
}

void BpeV1::save(const std::string& path) const {
    std::string buf;
    const auto token = [&](const std::string& t) {
        put_u64(buf, t.size());
        buf += t;
    };
    std::vector<std::pair<int, const std::string*>> by_id;
    for (const auto& [t, id] : vocab_) by_id.emplace_back(id, &t);
    std::sort(by_id.begin(), by_id.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    put_u64(buf, by_id.size());
    for (const auto& [id, t] : by_id) {
        token(*t);
        put_u32(buf, static_cast<std::uint32_t>(id));
    }
    put_u64(buf, merges_.size());
    for (const Merge& m : merges_) {
        token(m.first);
        token(m.second);
    }
    std::ofstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("Failed to open file for saving: " + path);
    f.write(buf.data(), static_cast<std::streamsize>(buf.size()));
    f.close();
    if (!f) throw std::runtime_error("Failed while writing tokenizer cache: " + path);
}

int BpeV1::special_id(std::string_view token) const {
    if (token != "<pad>" && token != "<eos>" && token != "<unk>") return -1;
    const auto it = vocab_.find(std::string(token));
    return it == vocab_.end() ? -1 : it->second;
}

// The merge list is walked once, in order, and a merge joins every occurrence of
// its pair from left to right (bpe_tokenizer.cpp:222-247).  Instead of testing
// all merges against the word, the next merge to act is the lowest rank, at or
// after the last one applied, among the pairs the word holds now.
void BpeV1::encode_word(const std::string& word, std::vector<int>& out) const {
    std::vector<std::string> parts;
    parts.reserve(word.size());
    for (const char c : word) parts.emplace_back(1, c);
    int from = 0;
    while (parts.size() > 1) {
        int best = INT_MAX;
        for (std::size_t i = 0; i + 1 < parts.size(); i++) {
            const auto it = ranks_.find(pair_string(parts[i], parts[i + 1]));
            if (it == ranks_.end()) continue;
            const auto r = std::lower_bound(it->second.begin(), it->second.end(), from);
            if (r != it->second.end()) best = std::min(best, *r);
        }
        if (best == INT_MAX) break;
        const Merge& m = merges_[static_cast<std::size_t>(best)];
        std::vector<std::string> next;
        next.reserve(parts.size());
        for (std::size_t i = 0; i < parts.size(); i++) {
            if (i + 1 < parts.size() && parts[i] == m.first && parts[i + 1] == m.second) {
                next.push_back(m.first + m.second);
                i++;
            } else {
                next.push_back(std::move(parts[i]));
            }
        }
        parts = std::move(next);
        from = best + 1;
    }
    for (const std::string& p : parts) {
        const auto it = vocab_.find(p);
        out.push_back(it == vocab_.end() ? 2 : it->second);  // unk_token_id, bpe_tokenizer.h:30
    }
}

std::vector<int> BpeV1::encode(std::string_view text) const {
    std::vector<int> out;
    std::unordered_map<std::string, std::pair<std::size_t, std::size_t>> seen;
    bool first = true;
    for (std::size_t pos = 0; pos < text.size();) {
        while (pos < text.size() && c_space(text[pos])) pos++;
        std::size_t end = pos;
        while (end < text.size() && !c_space(text[end])) end++;
        if (end == pos) break;
        std::string word = first ? std::string() : std::string("_");
        word.append(text.substr(pos, end - pos));
        first = false;
        pos = end;
        if (const auto hit = seen.find(word); hit != seen.end()) {
            // out may reallocate while it grows: copy through indices
            for (std::size_t i = 0; i < hit->second.second; i++) {
                const int id = out[hit->second.first + i];
                out.push_back(id);
            }
            continue;
        }
        const std::size_t before = out.size();
        encode_word(word, out);
        seen.emplace(std::move(word), std::make_pair(before, out.size() - before));
    }
    return out;
}

std::string BpeV1::decode(const int* ids, std::size_t n) const {
    std::string out;
    for (std::size_t i = 0; i < n; i++) {
        const auto it = id_to_token_.find(ids[i]);
        if (it != id_to_token_.end()) out += it->second;
    }
    for (char& c : out)
        if (c == '_') c = ' ';
    return out;
}

bool is_gtok_file(const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("Failed to open tokenizer file: " + path);
    char magic[4] = {0, 0, 0, 0};
    f.read(magic, 4);
    return f.gcount() == 4 && std::memcmp(magic, "GTOK", 4) == 0;
}

}  // namespace gh

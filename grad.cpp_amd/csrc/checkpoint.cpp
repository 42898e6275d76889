#include "checkpoint.h"

#include <cstdio>
#include <cstring>
#include <memory>

namespace gh {

namespace {

constexpr uint32_t kMagic = 0x4750544D;  // "GPTM"
constexpr uint32_t kTrailerPayload = 12;
constexpr uint32_t kMaxTrailerPayload = 1u << 20;
constexpr int kMaxVocab = 1 << 24, kMaxDModel = 1 << 16, kMaxLayers = 1 << 12, kMaxLen = 1 << 20;

struct FileCloser {
    void operator()(std::FILE* f) const {
        if (f) std::fclose(f);
    }
};
using File = std::unique_ptr<std::FILE, FileCloser>;

[[noreturn]] void fail(const std::string& msg) { throw std::runtime_error(msg); }

template <typename T>
T read_scalar(std::FILE* f, const std::string& what) {
    T v{};
    if (std::fread(&v, sizeof(T), 1, f) != 1) fail("file ends while reading " + what);
    return v;
}

void check_range(const char* name, int v, int lo, int hi) {
    if (v < lo || v > hi) {
        fail(std::string("header field ") + name + " = " + std::to_string(v) + " is outside ["
             + std::to_string(lo) + ", " + std::to_string(hi) + "]");
    }
}

uint64_t get_le(const unsigned char* p, int n) {
    uint64_t v = 0;
    for (int i = 0; i < n; i++) v |= static_cast<uint64_t>(p[i]) << (8 * i);
    return v;
}

void put_le(std::string& out, uint64_t v, int n) {
    for (int i = 0; i < n; i++) out.push_back(static_cast<char>((v >> (8 * i)) & 0xFF));
}

}  // namespace

std::vector<TensorSpec> tensor_specs(const Shape& s) {
    const int d = s.d_model, F = s.d_ff();
    std::vector<TensorSpec> t;
    t.push_back({"token embedding", s.vocab, d});
    if (!s.modern()) t.push_back({"position embedding", s.max_len, d});
    for (int l = 0; l < s.layers; l++) {
        const std::string p = "layer " + std::to_string(l) + " ";
        for (const char* n : {"W_q", "W_k", "W_v", "W_o"}) t.push_back({p + n, d, d});
        for (const char* n : {"b_q", "b_k", "b_v", "b_o"}) t.push_back({p + n, 1, d});
        if (s.modern()) {
            t.push_back({p + "FFN gate", d, F});
            t.push_back({p + "FFN up", d, F});
            t.push_back({p + "FFN down", F, d});
        } else {
            t.push_back({p + "FFN W1", d, F});
            t.push_back({p + "FFN b1", 1, F});
            t.push_back({p + "FFN W2", F, d});
            t.push_back({p + "FFN b2", 1, d});
        }
        for (const char* n : {"norm1 gamma", "norm1 beta", "norm2 gamma", "norm2 beta"})
            t.push_back({p + n, 1, d});
    }
    t.push_back({"final norm gamma", 1, d});
    t.push_back({"final norm beta", 1, d});
    return t;
}

// gpt_model.cpp:419-430, then the constructor check of
// multihead_attention.cpp:333-335 that load() runs into next.
void validate_shape(const Shape& s) {
    check_range("vocab_size", s.vocab, 1, kMaxVocab);
    check_range("d_model", s.d_model, 1, kMaxDModel);
    check_range("num_layers", s.layers, 1, kMaxLayers);
    check_range("num_heads", s.heads, 1, s.d_model);
    check_range("max_len", s.max_len, 1, kMaxLen);
    if (s.d_model % s.heads != 0) {
        fail("d_model " + std::to_string(s.d_model) + " is not divisible by num_heads "
             + std::to_string(s.heads));
    }
    if (!(s.dropout >= 0.0f && s.dropout < 1.0f)) {
        fail("dropout_rate " + std::to_string(s.dropout) + " is outside [0, 1)");
    }
    if (s.modern() && (s.d_model / s.heads) % 2 != 0) fail("RoPE requires an even head size");
}

HostModel read_checkpoint(const std::string& path) {
    File file(std::fopen(path.c_str(), "rb"));
    if (!file) throw std::runtime_error("Could not open checkpoint for reading: " + path);
    std::FILE* f = file.get();
    try {
        HostModel m;
        if (read_scalar<uint32_t>(f, "magic number") != kMagic)
            fail("not a grad.cpp checkpoint (wrong magic number)");
        const uint32_t version = read_scalar<uint32_t>(f, "format version");
        if (version != 1 && version != 2)
            fail("unsupported format version " + std::to_string(version));
        if (version == 2) {
            const uint32_t tag = read_scalar<uint32_t>(f, "architecture tag");
            if (tag > 1) fail("unknown architecture tag " + std::to_string(tag));
            m.shape.arch = static_cast<int>(tag);
        }
        m.shape.vocab = read_scalar<int32_t>(f, "vocab_size");
        m.shape.d_model = read_scalar<int32_t>(f, "d_model");
        m.shape.layers = read_scalar<int32_t>(f, "num_layers");
        m.shape.heads = read_scalar<int32_t>(f, "num_heads");
        m.shape.max_len = read_scalar<int32_t>(f, "max_len");
        m.shape.dropout = read_scalar<float>(f, "dropout_rate");
        validate_shape(m.shape);

        for (const TensorSpec& spec : tensor_specs(m.shape)) {
            const int rows = read_scalar<int32_t>(f, spec.name);
            const int cols = read_scalar<int32_t>(f, spec.name);
            if (rows <= 0 || cols <= 0 || rows != spec.rows || cols != spec.cols) {
                fail(spec.name + " is " + std::to_string(rows) + "x" + std::to_string(cols)
                     + ", model expects " + std::to_string(spec.rows) + "x"
                     + std::to_string(spec.cols));
            }
            std::vector<float> data(static_cast<size_t>(rows) * static_cast<size_t>(cols));
            if (std::fread(data.data(), sizeof(float), data.size(), f) != data.size())
                fail("file ends inside " + spec.name);
            m.tensors.push_back(std::move(data));
        }

        // Trailer sections: tag[4], u32 length, payload (gpt_model.cpp:489-515).
        for (;;) {
            const int c = std::fgetc(f);
            if (c == EOF) break;
            std::ungetc(c, f);
            unsigned char hdr[8];
            if (std::fread(hdr, 1, 8, f) != 8) fail("file ends while reading trailer section header");
            const uint32_t len = static_cast<uint32_t>(get_le(hdr + 4, 4));
            if (len > kMaxTrailerPayload) {
                fail("trailer section has an implausible length (" + std::to_string(len)
                     + " bytes)");
            }
            if (std::memcmp(hdr, "TKFP", 4) != 0) {
                std::vector<unsigned char> sink(len);
                if (len && std::fread(sink.data(), 1, len, f) != len)
                    fail("file ends inside trailer section");
                continue;
            }
            if (len != kTrailerPayload) {
                fail("tokenizer trailer has length " + std::to_string(len) + ", expected "
                     + std::to_string(kTrailerPayload));
            }
            unsigned char pl[kTrailerPayload];
            if (std::fread(pl, 1, kTrailerPayload, f) != kTrailerPayload)
                fail("file ends while reading tokenizer trailer");
            const uint32_t kind = static_cast<uint32_t>(get_le(pl, 4));
            if (kind != 1 && kind != 2) fail("unknown tokenizer kind " + std::to_string(kind));
            m.tokenizer = Fingerprint{kind, get_le(pl + 4, 8)};
        }
        return m;
    } catch (const std::exception& e) {
        throw std::runtime_error("Failed to load model from " + path + ": " + e.what());
    }
}

bool write_checkpoint(const std::string& path, const Shape& s,
                      const std::vector<const float*>& tensors,
                      const std::optional<Fingerprint>& tokenizer, std::string& why) {
    File file(std::fopen(path.c_str(), "wb"));
    if (!file) {
        why = "Error: Could not open file for writing: " + path;
        return false;
    }
    std::FILE* f = file.get();
    const std::vector<TensorSpec> specs = tensor_specs(s);
    bool ok = tensors.size() == specs.size();
    const uint32_t head[3] = {kMagic, 2u, static_cast<uint32_t>(s.arch)};
    const int32_t dims[5] = {s.vocab, s.d_model, s.layers, s.heads, s.max_len};
    ok = ok && std::fwrite(head, 4, 3, f) == 3 && std::fwrite(dims, 4, 5, f) == 5
         && std::fwrite(&s.dropout, 4, 1, f) == 1;
    for (size_t i = 0; ok && i < specs.size(); i++) {
        const int32_t rc[2] = {specs[i].rows, specs[i].cols};
        const size_t n = static_cast<size_t>(rc[0]) * static_cast<size_t>(rc[1]);
        ok = std::fwrite(rc, 4, 2, f) == 2 && std::fwrite(tensors[i], 4, n, f) == n;
    }
    if (ok && tokenizer) {
        std::string tr("TKFP");
        put_le(tr, kTrailerPayload, 4);
        put_le(tr, tokenizer->kind, 4);
        put_le(tr, tokenizer->hash, 8);
        ok = std::fwrite(tr.data(), 1, tr.size(), f) == tr.size();
    }
    if (std::fclose(file.release()) != 0) ok = false;
    if (!ok) why = "Error: writing checkpoint failed: " + path;
    return ok;
}

}  // namespace gh

// Host-side reader/writer for grad.cpp's "GPTM" checkpoint files
// (src/transformer/gpt_model.cpp:187-525 of grad.cpp).
#pragma once

#include <cstdint>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace gh {

struct Shape {
    int arch = 0;  // 0 GPT-2, 1 Modern
    int vocab = 0, d_model = 0, layers = 0, heads = 0, max_len = 0;
    float dropout = 0.0f;

    bool modern() const { return arch == 1; }
    int head_size() const { return d_model / heads; }
    // include/grad/transformer/feedforward.h:24-28
    int d_ff() const { return modern() ? ((8 * d_model / 3) + 63) / 64 * 64 : 4 * d_model; }
};

struct TensorSpec {
    std::string name;  // the name GPTModel::load uses in its messages
    int rows, cols;
};

// Tensor records in file order (gpt_model.cpp:318-355).
std::vector<TensorSpec> tensor_specs(const Shape& s);

struct Fingerprint {
    uint32_t kind;
    uint64_t hash;
};

struct HostModel {
    Shape shape;
    std::vector<std::vector<float>> tensors;  // file order, (rows, cols) row-major
    std::optional<Fingerprint> tokenizer;
};

// Header validation shared by the file loader and gh_model_from_host; throws
// std::runtime_error with GPTModel::load's message texts.
void validate_shape(const Shape& s);

// Throws std::runtime_error("Could not open checkpoint for reading: <path>") or
// std::runtime_error("Failed to load model from <path>: <why>").
HostModel read_checkpoint(const std::string& path);

// Returns false (after setting `why`) when the file cannot be written.
bool write_checkpoint(const std::string& path, const Shape& shape,
                      const std::vector<const float*>& tensors,
                      const std::optional<Fingerprint>& tokenizer, std::string& why);

}  // namespace gh

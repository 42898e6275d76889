// gradhip-eval: the loss of a checkpoint over a pre-tokenized split, in
// non-overlapping windows, all positions of a batch of windows in one pass on the
// GPU.  The scoring half of `grad eval` (src/cli/eval.cpp:44-133 of grad.cpp):
//
//   gradhip-eval <checkpoint> <tokens.bin> [--seq N] [--batches N] [--sampled [--seed S]] [--print-windows]
//
// <tokens.bin> is a "TOK1" file (include/grad/data/token_file.h:10-12: magic, u32
// vocabulary size, u64 token count, u16 ids).  Window i covers tokens
// [i * seq, i * seq + seq] (src/data/token_file.cpp:149-176), eight windows to a
// batch (eval.cpp:77), loss = sum over batches of (batch mean x rows) / rows
// (src/training/trainer.cpp:319-340).  --batches N scores the first N batches in file
// order; with --sampled the windows of every batch are drawn the way grad.cpp's
// DataLoader draws them when `grad eval` is given --max-batches (eval.cpp:84-89,
// src/data/dataloader.cpp:36-44): with replacement, std::uniform_int_distribution
// over the window indices on a std::mt19937 seeded 20260921 for the validation
// split (20260922 for the train split: --seed).  What that distribution returns
// for given engine outputs is the C++ library's choice, so the sample equals
// grad.cpp's when both are built with the same library; --print-windows lists
// the indices drawn.  The split is named explicitly; grad.cpp derives both of
// its splits from a corpus path and also reports bits per byte from the corpus size.
#include "gradhip.hpp"

#include <chrono>
#include <cmath>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <random>
#include <sstream>
#include <string>
#include <vector>

namespace {

struct Usage : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct TokenFile {
    int vocab = 0;
    std::vector<std::uint16_t> tokens;
};

// The checks and messages of MappedTokenDataset's constructor (token_file.cpp:83-147).
TokenFile read_token_file(const std::string& path, int seq) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) throw std::runtime_error("Cannot open token file: " + path);
    const std::streamoff bytes = f.tellg();
    constexpr std::streamoff kHeader = 16;
    if (bytes < kHeader) throw std::runtime_error("Token file truncated or unreadable: " + path);
    f.seekg(0);
    char header[kHeader];
    f.read(header, kHeader);
    if (std::memcmp(header, "TOK1", 4) != 0) throw std::runtime_error("Not a token file (bad magic): " + path);
    std::uint32_t vocab = 0;
    std::uint64_t count = 0;
    std::memcpy(&vocab, header + 4, 4);
    std::memcpy(&count, header + 8, 8);
    if (vocab == 0 || vocab > 65536)
        throw std::runtime_error("Token file vocab " + std::to_string(vocab) + " outside (0, 65536]: " + path);
    if (count > static_cast<std::uint64_t>(bytes - kHeader) / 2)
        throw std::runtime_error("Token file shorter than its header claims: " + path);
    if (count < static_cast<std::uint64_t>(seq) + 1)
        throw std::runtime_error("Not enough tokens for even one sequence: " + path);
    TokenFile out;
    out.vocab = static_cast<int>(vocab);
    out.tokens.resize(count);
    f.read(reinterpret_cast<char*>(out.tokens.data()), static_cast<std::streamsize>(count * 2));
    if (!f) throw std::runtime_error("Token file truncated or unreadable: " + path);
    return out;
}

int to_int(const std::string& flag, const std::string& text, int least) {
    std::istringstream in(text);
    int v = 0;
    if (!(in >> v) || !in.eof() || v < least)
        throw Usage(flag + ": expected an integer of at least " + std::to_string(least) + ", got '" + text + "'");
    return v;
}

}  // namespace

int main(int argc, char** argv) {
    try {
        std::vector<std::string> positional;
        int seq = 256, max_batches = 0;  // eval.cpp:140-141
        bool sampled = false, print_windows = false;
        unsigned seed = 20260921;  // eval.cpp:83
        for (int i = 1; i < argc; i++) {
            const std::string a = argv[i];
            const auto value = [&]() -> std::string {
                if (i + 1 >= argc) throw Usage(a + ": missing value");
                return argv[++i];
            };
            if (a == "--seq") seq = to_int(a, value(), 1);
            else if (a == "--batches") max_batches = to_int(a, value(), 0);
            else if (a == "--sampled") sampled = true;
            else if (a == "--print-windows") print_windows = true;
            else if (a == "--seed") seed = static_cast<unsigned>(to_int(a, value(), 0));
            else if (a.rfind("--", 0) == 0) throw Usage("unknown option " + a);
            else positional.push_back(a);
        }
        if (positional.size() != 2)
            throw Usage("usage: gradhip-eval <checkpoint> <tokens.bin> [--seq N] [--batches N] [--sampled [--seed S]] "
                        "[--print-windows]");
        if (sampled && max_batches == 0) throw Usage("--sampled needs --batches N (a sample of the whole split is the split)");

        std::cout << "\ngradhip Evaluation\n" << std::endl;
        const gradhip::GPTModel model = gradhip::GPTModel::load(positional[0]);
        if (seq > model.getMaxLen())
            throw std::runtime_error("seq length exceeds the model's context (" + std::to_string(model.getMaxLen()) + ")");
        const TokenFile file = read_token_file(positional[1], seq);
        if (file.vocab != model.getVocabSize())
            throw std::runtime_error("token files and checkpoint disagree on vocab size");

        constexpr int kBatch = 8;  // eval.cpp:77
        const size_t windows = (file.tokens.size() - static_cast<size_t>(seq) - 1) / static_cast<size_t>(seq) + 1;
        size_t batches = (windows + kBatch - 1) / kBatch;
        if (max_batches > 0) batches = std::min<size_t>(batches, static_cast<size_t>(max_batches));

        std::cout << "Scoring\n" << std::endl;
        const auto start = std::chrono::steady_clock::now();
        double weighted = 0.0;
        size_t rows = 0;
        gh_session* full = nullptr;
        std::mt19937 rng(seed);
        for (size_t b = 0; b < batches; b++) {
            const size_t first = b * kBatch;
            const int n = static_cast<int>(std::min<size_t>(kBatch, windows - first));
            std::vector<int32_t> ids(static_cast<size_t>(n) * seq), targets(ids.size());
            std::vector<size_t> index(static_cast<size_t>(n));
            for (int w = 0; w < n; w++) index[static_cast<size_t>(w)] = first + static_cast<size_t>(w);
            if (sampled) {
                std::uniform_int_distribution<size_t> pick(0, windows - 1);  // dataloader.cpp:40-44
                for (int w = 0; w < n; w++) index[static_cast<size_t>(w)] = pick(rng);
            }
            if (print_windows) {
                std::cout << "windows";
                for (const size_t i : index) std::cout << " " << i;
                std::cout << std::endl;
            }
            for (int w = 0; w < n; w++) {
                const size_t at = index[static_cast<size_t>(w)];
                const std::uint16_t* win = file.tokens.data() + at * static_cast<size_t>(seq);
                for (int t = 0; t <= seq; t++) {
                    if (win[t] >= file.vocab)  // token_file.cpp:164-170
                        throw std::runtime_error("token id " + std::to_string(win[t]) + " at offset "
                                                 + std::to_string(at * static_cast<size_t>(seq) + t)
                                                 + " is outside the file's vocab of " + std::to_string(file.vocab));
                }
                for (int t = 0; t < seq; t++) {
                    ids[static_cast<size_t>(w) * seq + t] = win[t];
                    targets[static_cast<size_t>(w) * seq + t] = win[t + 1];
                }
            }
            // one session serves every full batch; a short last batch gets its own
            gh_session* s = nullptr;
            if (n == kBatch && full) {
                s = full;
                gradhip::check(gh_session_reset(s));
            } else {
                gh_session_opts o{};
                o.batch = n;
                gradhip::check(gh_session_create(model.handle(), &o, &s));
                if (n == kBatch) full = s;
            }
            std::vector<float> nll(ids.size());
            const gh_status st = gh_session_score(s, ids.data(), targets.data(), seq, nll.data());
            if (s != full) gh_session_free(s);
            if (st != GH_OK) {
                gh_session_free(full);
                gradhip::check(st);
            }
            double sum = 0.0;
            for (const float v : nll) sum += v;
            const float batch_loss = static_cast<float>(sum / static_cast<double>(nll.size()));  // the loss tensor is fp32
            weighted += static_cast<double>(batch_loss) * n;
            rows += static_cast<size_t>(n);
        }
        gh_session_free(full);
        const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
        const double loss = rows > 0 ? weighted / static_cast<double>(rows) : -1.0;
        // eval.cpp:107-118
        std::cout << std::left << std::setw(8) << "val" << std::right << std::fixed << " loss " << std::setprecision(4)
                  << loss << "  perplexity " << std::setprecision(3) << std::exp(loss) << "  ("
                  << rows * static_cast<size_t>(seq) << " tokens, " << std::setprecision(0) << seconds << "s)"
                  << std::defaultfloat << std::endl;
        std::cout << "Throughput: " << std::fixed << std::setprecision(0)
                  << static_cast<double>(rows * static_cast<size_t>(seq)) / seconds << " tokens/s" << std::endl;
        return 0;
    } catch (const Usage& e) {
        std::cerr << "gradhip-eval: " << e.what() << std::endl;
        return 2;
    } catch (const std::exception& e) {
        std::cerr << "Error: " << e.what() << std::endl;
        return 1;
    }
}

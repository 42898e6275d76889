// gradhip-bench: the "Generation throughput" section of `grad bench`
// (src/cli/bench.cpp:269-286 of grad.cpp) on the GPU, reported in the same JSON
// schema (bench.cpp:112-172) so the numbers drop into the same tables.
//
//   gradhip-bench [--checkpoint model.bin] [--trials N] [--json out.json]
//
// Protocol, as in the reference: `trials` timed calls of
// generate_sample(prompt, temperature 0.8, 64 tokens) with TextGen's defaults
// (penalty 1.2, no top-k / top-p); every call builds a fresh session
// (text_gen.cpp:74); the host clock runs around the whole call; tokens per second
// = 64 / seconds; the median is reported.  Without --checkpoint the model is the
// benchmark's pinned 22M configuration (bench.cpp:82-91) with N(0, 0.02) weights:
// throughput does not depend on the values.  The prompt is "ROMEO:\n" as seven
// byte ids (the reference encodes it with its corpus tokenizer, which is not
// available here; the prompt length differs by a few tokens at most).
// Training fields of the schema are present and empty: training is not on this path.
#include "gradhip.hpp"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <ctime>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <random>
#include <sstream>
#include <sys/resource.h>

namespace {

struct Usage : std::runtime_error {
    using std::runtime_error::runtime_error;
};

double median(std::vector<double> v) {
    if (v.empty()) return 0.0;
    std::sort(v.begin(), v.end());
    const size_t n = v.size();
    return n % 2 ? v[n / 2] : 0.5 * (v[n / 2 - 1] + v[n / 2]);
}

std::string timestamp_utc() {
    const std::time_t now = std::time(nullptr);
    std::tm utc{};
    gmtime_r(&now, &utc);
    std::ostringstream out;
    out << std::put_time(&utc, "%Y-%m-%dT%H:%M:%SZ");
    return out.str();
}

gradhip::GPTModel synthetic_model(size_t& parameters) {
    gh_config cfg{};
    cfg.arch = GH_ARCH_GPT2;
    cfg.vocab = 5000;
    cfg.d_model = 512;
    cfg.layers = 6;
    cfg.heads = 8;
    cfg.max_len = 1024;
    cfg.dropout = 0.1f;
    const int n = gh_config_num_tensors(&cfg);
    std::mt19937 gen(1000);
    std::normal_distribution<float> dist(0.0f, 0.02f);
    std::vector<std::vector<float>> store(static_cast<size_t>(n));
    std::vector<const float*> ptrs;
    parameters = 0;
    for (int i = 0; i < n; i++) {
        int32_t rows = 0, cols = 0;
        gradhip::check(gh_config_tensor_shape(&cfg, i, &rows, &cols));
        store[i].resize(static_cast<size_t>(rows) * cols);
        for (float& v : store[i]) v = dist(gen);
        parameters += store[i].size();
        ptrs.push_back(store[i].data());
    }
    return gradhip::GPTModel::from_host(cfg, ptrs);
}

size_t parameters_of(const gradhip::GPTModel& m) {
    gh_config cfg{};
    gradhip::check(gh_model_get_config(m.handle(), &cfg));
    size_t total = 0;
    for (int i = 0, n = gh_config_num_tensors(&cfg); i < n; i++) {
        int32_t rows = 0, cols = 0;
        gradhip::check(gh_config_tensor_shape(&cfg, i, &rows, &cols));
        total += static_cast<size_t>(rows) * cols;
    }
    return total;
}

}  // namespace

int main(int argc, char** argv) {
    try {
        std::string checkpoint, json_path;
        int trials = 5;
        for (int i = 1; i < argc; i++) {
            const std::string a = argv[i];
            const auto value = [&]() -> std::string {
                if (i + 1 >= argc) throw Usage(a + ": missing value");
                return argv[++i];
            };
            if (a == "--checkpoint") checkpoint = value();
            else if (a == "--json") json_path = value();
            else if (a == "--trials") {
                trials = std::atoi(value().c_str());
                if (trials < 1) throw Usage("--trials: must be at least 1");
            } else throw Usage("usage: gradhip-bench [--checkpoint model.bin] [--trials N] [--json out.json]");
        }

        std::cout << "\ngradhip Benchmark\n" << std::endl;
        size_t parameters = 0;
        gradhip::GPTModel model = checkpoint.empty() ? synthetic_model(parameters) : gradhip::GPTModel::load(checkpoint);
        if (!checkpoint.empty()) parameters = parameters_of(model);
        char device[256] = "";
        int32_t cus = 0, gfx950 = 0;
        gradhip::check(gh_device_info(device, sizeof device, &cus, &gfx950));
        std::cout << "Model: vocab " << model.getVocabSize() << ", d_model " << model.getDModel() << ", layers "
                  << model.getNumLayers() << ", heads " << model.getNumHeads() << ", " << parameters
                  << " parameters; device " << device << " (" << cus << " CUs)" << std::endl;

        std::cout << "\nGeneration throughput\n" << std::endl;
        constexpr int kGenTokens = 64;  // bench.cpp:270
        gradhip::TextGen generator(model, nullptr);
        std::vector<int> prompt;
        for (const char c : std::string("ROMEO:\n")) prompt.push_back(static_cast<unsigned char>(c));
        std::vector<double> rates;
        for (int trial = 0; trial < trials; trial++) {
            const auto start = std::chrono::steady_clock::now();
            (void)generator.generate_sample(prompt, 0.8f, kGenTokens);
            const double s = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
            rates.push_back(kGenTokens / s);
            std::cout << "  trial " << (trial + 1) << ": " << std::fixed << std::setprecision(1) << rates.back()
                      << " tok/s" << std::endl;
        }
        std::cout << "  median: " << std::fixed << std::setprecision(1) << median(rates) << " tok/s" << std::endl;

        rusage ru{};
        getrusage(RUSAGE_SELF, &ru);
        const size_t peak_rss_mb = static_cast<size_t>(ru.ru_maxrss) / 1024;
        std::cout << "\nPeak RSS: " << peak_rss_mb << " MB" << std::endl;

        if (!json_path.empty()) {
            std::ofstream out(json_path);
            if (!out) throw std::runtime_error("Cannot write benchmark JSON: " + json_path);
            out << "{\n"
                << "  \"schema_version\": 1,\n"
                << "  \"timestamp_utc\": \"" << timestamp_utc() << "\",\n"
                << "  \"engine\": \"gradhip\",\n"
                << "  \"version\": \"0.1.0\",\n"
                << "  \"git_sha\": \"\",\n"
                << "  \"build_type\": \"Release\",\n"
                << "  \"compiler\": \"" << __VERSION__ << "\",\n"
                << "  \"system\": \"Linux\",\n"
                << "  \"metal_available\": false,\n"
                << "  \"metal_fp16\": false,\n"
                << "  \"device\": \"" << device << "\",\n"
                << "  \"parameters\": " << parameters << ",\n"
                << "  \"config\": {\"vocab\": " << model.getVocabSize() << ", \"d_model\": " << model.getDModel()
                << ", \"layers\": " << model.getNumLayers() << ", \"heads\": " << model.getNumHeads()
                << ", \"sequence\": " << 0 << ", \"batch\": " << 1 << "},\n"
                << "  \"protocol\": {\"warmup_steps\": 0, \"steps_per_trial\": 0, \"trials\": " << trials << "},\n"
                << "  \"training_steps_per_second\": [],\n"
                << "  \"training_tokens_per_second\": [],\n"
                << "  \"generation_tokens_per_second\": [";
            for (size_t i = 0; i < rates.size(); i++)
                out << (i ? ", " : "") << std::fixed << std::setprecision(6) << rates[i];
            out << "],\n"
                << "  \"median_training_steps_per_second\": " << 0.0 << ",\n"
                << "  \"median_training_tokens_per_second\": " << 0.0 << ",\n"
                << "  \"median_generation_tokens_per_second\": " << median(rates) << ",\n"
                << "  \"peak_rss_mb\": " << peak_rss_mb << ",\n"
                << "  \"metal_stream_per_step\": {\"syncs\": 0, \"command_buffers\": 0, \"dispatches\": 0, "
                   "\"throttle_waits\": 0},\n"
                << "  \"metal_peak_live_mb\": 0\n"
                << "}\n";
            if (!out.good()) throw std::runtime_error("Failed while writing benchmark JSON: " + json_path);
            std::cout << "Benchmark JSON: " << json_path << std::endl;
        }
        return 0;
    } catch (const Usage& e) {
        std::cerr << "gradhip-bench: " << e.what() << std::endl;
        return 2;
    } catch (const std::exception& e) {
        std::cerr << "Error: " << e.what() << std::endl;
        return 1;
    }
}

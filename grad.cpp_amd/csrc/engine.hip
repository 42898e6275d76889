// gradhip engine: device model, paged KV cache, the per-token step (eager,
// hipGraph-replayed), the on-GPU generate loop, and the C ABI of
// include/gradhip.h.
#include "../../include/gradhip.h"
#include "checkpoint.h"
#include "tokenizer.h"
#include "kernels_attn.h"
#include "kernels_common.h"
#include "kernels_gemm.h"
#include "kernels_gemm_big.h"
#include "kernels_gemv.h"
#include "kernels_persist.h"
#include "kernels_pick.h"
#include "kernels_xcd.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <numeric>
#include <string>
#include <vector>

namespace gh {

// ------------------------------------------------------------------ errors

struct ApiError {
    gh_status code;
    std::string msg;
};

static thread_local std::string g_last_error;

[[noreturn]] static void throw_device(hipError_t e, const char* what, const char* file, int line) {
    throw ApiError{GH_ERR_DEVICE, std::string("HIP error in ") + what + ": " + hipGetErrorString(e)
                                      + " (" + file + ":" + std::to_string(line) + ")"};
}

#define HIP_CHECK(expr)                                                        \
    do {                                                                       \
        hipError_t e_ = (expr);                                                \
        if (e_ != hipSuccess) throw_device(e_, #expr, __FILE__, __LINE__);     \
    } while (0)

template <typename F>
static gh_status guard(F&& f) {
    try {
        f();
        return GH_OK;
    } catch (const ApiError& e) {
        g_last_error = e.msg;
        return e.code;
    } catch (const std::out_of_range& e) {
        g_last_error = e.what();
        return GH_ERR_OUT_OF_RANGE;
    } catch (const std::invalid_argument& e) {
        g_last_error = e.what();
        return GH_ERR_INVALID_ARGUMENT;
    } catch (const std::bad_alloc&) {
        g_last_error = "out of host memory";
        return GH_ERR_RUNTIME;
    } catch (const std::exception& e) {
        g_last_error = e.what();
        return GH_ERR_RUNTIME;
    }
}

static void require_gpu() {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        throw ApiError{GH_ERR_DEVICE,
                       "gradhip needs a gfx950 GPU: no HIP device is usable and there is no CPU "
                       "fallback"};
    }
}

// ------------------------------------------------------------ device model

// Layout kernels.  Matrices arrive (in, out) row-major as grad.cpp stores them
// (inference.cpp:13) and are kept (out, in) so that one output's weights are a
// contiguous stream.  dst row of source column c is c * row_mul + row_off.
__global__ void transpose_in_kernel(const float* __restrict__ src, int rows, int cols,
                                    float* __restrict__ dst, int row_mul, int row_off) {
    __shared__ float tile[32][33];
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    for (int i = threadIdx.y; i < 32; i += blockDim.y) {
        const int r = r0 + i, c = c0 + threadIdx.x;
        if (r < rows && c < cols) tile[i][threadIdx.x] = src[static_cast<size_t>(r) * cols + c];
    }
    __syncthreads();
    for (int i = threadIdx.y; i < 32; i += blockDim.y) {
        const int c = c0 + i, r = r0 + threadIdx.x;
        if (r < rows && c < cols)
            dst[(static_cast<size_t>(c) * row_mul + row_off) * rows + r] = tile[threadIdx.x][i];
    }
}

__global__ void transpose_out_kernel(const float* __restrict__ dev, int rows, int cols,
                                     float* __restrict__ out, int row_mul, int row_off) {
    __shared__ float tile[32][33];
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    for (int i = threadIdx.y; i < 32; i += blockDim.y) {
        const int c = c0 + i, r = r0 + threadIdx.x;
        if (r < rows && c < cols)
            tile[threadIdx.x][i] = dev[(static_cast<size_t>(c) * row_mul + row_off) * rows + r];
    }
    __syncthreads();
    for (int i = threadIdx.y; i < 32; i += blockDim.y) {
        const int r = r0 + i, c = c0 + threadIdx.x;
        if (r < rows && c < cols) out[static_cast<size_t>(r) * cols + c] = tile[i][threadIdx.x];
    }
}

struct LayerWeights {
    float *wqkv, *bqkv;  // (3d, d), 3d
    float *wo, *bo;      // (d, d), d
    float *w1, *b1;      // GPT-2: (F, d), F.  Modern: (2F, d) rows (gate_p, up_p) interleaved
    float *w2, *b2;      // (d, F), d (GPT-2 only)
    float *g1, *be1, *g2, *be2;
};

// Where tensor i of the file lives on the device.
struct Placement {
    float* dst;
    bool transpose;
    int row_mul, row_off;
};

struct Model {
    Shape shape;
    std::optional<Fingerprint> tokenizer;
    float* blob = nullptr;
    size_t blob_floats = 0;
    float* E = nullptr;
    float* P = nullptr;
    std::vector<LayerWeights> layers;
    float *gf = nullptr, *bf = nullptr;
    float *rope_cos = nullptr, *rope_sin = nullptr;  // (max_len, head_size/2)
    std::vector<Placement> place;                    // file order

    // The XCD-sharded persistent kernel reads the weights from a second copy laid
    // out as one contiguous stream per workgroup (kernels_xcd.h); built by the
    // first session that uses it.
    mutable std::mutex xcd_mutex;
    mutable char* xcd_stream = nullptr;
    mutable XcdGeom xcd_geom{};

    ~Model() {
        if (blob) (void)hipFree(blob);
        if (xcd_stream) (void)hipFree(xcd_stream);
    }
};

static size_t align_up(size_t n, size_t a) { return (n + a - 1) / a * a; }

// Carves the weight blob and records where each file tensor goes.
static void plan_model(Model& m) {
    const Shape& s = m.shape;
    const size_t d = s.d_model, F = s.d_ff(), V = s.vocab, C = s.max_len, L = s.layers;
    size_t off = 0;
    auto take = [&](size_t n) {
        const size_t at = off;
        off = align_up(off + n, 64);  // 256-byte alignment
        return at;
    };
    std::vector<size_t> o;
    o.push_back(take(V * d));
    if (!s.modern()) o.push_back(take(C * d));
    struct LO {
        size_t wqkv, bqkv, wo, bo, w1, b1, w2, b2, g1, be1, g2, be2;
    };
    std::vector<LO> lo(L);
    for (size_t l = 0; l < L; l++) {
        lo[l].wqkv = take(3 * d * d);
        lo[l].bqkv = take(3 * d);
        lo[l].wo = take(d * d);
        lo[l].bo = take(d);
        lo[l].w1 = take((s.modern() ? 2 : 1) * F * d);
        lo[l].b1 = take(F);
        lo[l].w2 = take(d * F);
        lo[l].b2 = take(d);
        lo[l].g1 = take(d);
        lo[l].be1 = take(d);
        lo[l].g2 = take(d);
        lo[l].be2 = take(d);
    }
    const size_t ogf = take(d), obf = take(d);
    const size_t half = s.head_size() / 2;
    const size_t ocos = take(C * half + 1), osin = take(C * half + 1);
    m.blob_floats = off;
    HIP_CHECK(hipMalloc(&m.blob, off * sizeof(float)));
    HIP_CHECK(hipMemset(m.blob, 0, off * sizeof(float)));

    float* B = m.blob;
    m.E = B + o[0];
    m.P = s.modern() ? nullptr : B + o[1];
    m.place.push_back({m.E, false, 1, 0});
    if (!s.modern()) m.place.push_back({m.P, false, 1, 0});
    m.layers.resize(L);
    for (size_t l = 0; l < L; l++) {
        LayerWeights& w = m.layers[l];
        w = {B + lo[l].wqkv, B + lo[l].bqkv, B + lo[l].wo, B + lo[l].bo, B + lo[l].w1,
             B + lo[l].b1,   B + lo[l].w2,   B + lo[l].b2, B + lo[l].g1, B + lo[l].be1,
             B + lo[l].g2,   B + lo[l].be2};
        for (int q = 0; q < 3; q++) m.place.push_back({w.wqkv + q * d * d, true, 1, 0});
        m.place.push_back({w.wo, true, 1, 0});
        for (int q = 0; q < 3; q++) m.place.push_back({w.bqkv + q * d, false, 1, 0});
        m.place.push_back({w.bo, false, 1, 0});
        if (s.modern()) {
            m.place.push_back({w.w1, true, 2, 0});  // gate -> even rows
            m.place.push_back({w.w1, true, 2, 1});  // up -> odd rows
            m.place.push_back({w.w2, true, 1, 0});  // down
        } else {
            m.place.push_back({w.w1, true, 1, 0});
            m.place.push_back({w.b1, false, 1, 0});
            m.place.push_back({w.w2, true, 1, 0});
            m.place.push_back({w.b2, false, 1, 0});
        }
        m.place.push_back({w.g1, false, 1, 0});
        m.place.push_back({w.be1, false, 1, 0});
        m.place.push_back({w.g2, false, 1, 0});
        m.place.push_back({w.be2, false, 1, 0});
    }
    m.gf = B + ogf;
    m.bf = B + obf;
    m.place.push_back({m.gf, false, 1, 0});
    m.place.push_back({m.bf, false, 1, 0});
    m.rope_cos = B + ocos;
    m.rope_sin = B + osin;
}

static std::unique_ptr<Model> upload_model(const Shape& shape, const std::vector<const float*>& t,
                                           const std::optional<Fingerprint>& fp) {
    require_gpu();
    auto m = std::make_unique<Model>();
    m->shape = shape;
    m->tokenizer = fp;
    plan_model(*m);
    const std::vector<TensorSpec> specs = tensor_specs(shape);
    if (specs.size() != t.size() || specs.size() != m->place.size())
        throw ApiError{GH_ERR_INVALID_ARGUMENT, "tensor count does not match the model shape"};

    size_t biggest = 0;
    for (size_t i = 0; i < specs.size(); i++)
        if (m->place[i].transpose)
            biggest = std::max(biggest, static_cast<size_t>(specs[i].rows) * specs[i].cols);
    float* stage = nullptr;
    HIP_CHECK(hipMalloc(&stage, std::max<size_t>(biggest, 1) * sizeof(float)));
    try {
        for (size_t i = 0; i < specs.size(); i++) {
            const size_t n = static_cast<size_t>(specs[i].rows) * specs[i].cols;
            const Placement& pl = m->place[i];
            if (!pl.transpose) {
                HIP_CHECK(hipMemcpy(pl.dst, t[i], n * sizeof(float), hipMemcpyHostToDevice));
                continue;
            }
            HIP_CHECK(hipMemcpy(stage, t[i], n * sizeof(float), hipMemcpyHostToDevice));
            const dim3 grid((specs[i].cols + 31) / 32, (specs[i].rows + 31) / 32);
            transpose_in_kernel<<<grid, dim3(32, 8)>>>(stage, specs[i].rows, specs[i].cols, pl.dst,
                                                       pl.row_mul, pl.row_off);
            HIP_CHECK(hipGetLastError());
            HIP_CHECK(hipDeviceSynchronize());
        }
    } catch (...) {
        (void)hipFree(stage);
        throw;
    }
    HIP_CHECK(hipFree(stage));

    if (shape.modern()) {
        // The rotation angles of every position, with the reference's own fp32
        // expression (inference.cpp:169-175).
        const size_t half = shape.head_size() / 2, C = shape.max_len;
        std::vector<float> cs(C * half), sn(C * half);
        for (size_t j = 0; j < half; j++) {
            const float theta = std::pow(10000.0f, -2.0f * static_cast<float>(j)
                                                       / static_cast<float>(shape.head_size()));
            for (size_t pos = 0; pos < C; pos++) {
                cs[pos * half + j] = std::cos(static_cast<float>(pos) * theta);
                sn[pos * half + j] = std::sin(static_cast<float>(pos) * theta);
            }
        }
        if (half > 0) {
            HIP_CHECK(hipMemcpy(m->rope_cos, cs.data(), cs.size() * 4, hipMemcpyHostToDevice));
            HIP_CHECK(hipMemcpy(m->rope_sin, sn.data(), sn.size() * 4, hipMemcpyHostToDevice));
        }
    }
    return m;
}

// Reads every tensor back in file layout.
static std::vector<std::vector<float>> download_model(const Model& m) {
    const std::vector<TensorSpec> specs = tensor_specs(m.shape);
    size_t biggest = 1;
    for (const TensorSpec& s : specs) biggest = std::max(biggest, static_cast<size_t>(s.rows) * s.cols);
    float* stage = nullptr;
    HIP_CHECK(hipMalloc(&stage, biggest * sizeof(float)));
    std::vector<std::vector<float>> out;
    try {
        for (size_t i = 0; i < specs.size(); i++) {
            const size_t n = static_cast<size_t>(specs[i].rows) * specs[i].cols;
            const Placement& pl = m.place[i];
            std::vector<float> host(n);
            if (!pl.transpose) {
                HIP_CHECK(hipMemcpy(host.data(), pl.dst, n * 4, hipMemcpyDeviceToHost));
            } else {
                const dim3 grid((specs[i].cols + 31) / 32, (specs[i].rows + 31) / 32);
                transpose_out_kernel<<<grid, dim3(32, 8)>>>(pl.dst, specs[i].rows, specs[i].cols,
                                                            stage, pl.row_mul, pl.row_off);
                HIP_CHECK(hipGetLastError());
                HIP_CHECK(hipMemcpy(host.data(), stage, n * 4, hipMemcpyDeviceToHost));
            }
            out.push_back(std::move(host));
        }
    } catch (...) {
        (void)hipFree(stage);
        throw;
    }
    HIP_CHECK(hipFree(stage));
    return out;
}

// ----------------------------------------------------------------- session

struct Session {
    const Model* m = nullptr;
    int B = 1;
    int engine = GH_ENGINE_GRAPH;
    int page_shift = 6;
    int pages_per_seq = 0, n_pages = 0;
    int attn_chunk = 64, attn_max_chunks = 1;
    bool pick_row_in_lds = false;  // the pick's working row (vocab floats) fits in LDS beside its work area
    int work_stride = 0;           // floats per sequence of the working rows in global memory
    bool pick_global_scratch = false;
    bool use_prompt_pass = true;
    int launches_per_step = 0;

    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    // Batched greedy decoding without a penalty: the logits launch leaves the largest
    // value of every run of 16 columns, and a second form of the step opens with the
    // launch that picks from those and embeds (no pick launch, no embedding launch).
    float2* best = nullptr;  // [B][best_stride]
    int best_stride = 0;
    hipGraph_t graph_fused = nullptr;
    hipGraphExec_t exec_fused = nullptr;
    hipEvent_t ev[3] = {nullptr, nullptr, nullptr};

    float* kv_pool = nullptr;
    int* page_table = nullptr;
    float *x = nullptr, *h = nullptr, *q = nullptr, *attn = nullptr, *hidden = nullptr,
          *logits = nullptr;
    float* work = nullptr;
    float* attn_part = nullptr;
    unsigned* attn_tickets = nullptr;
    int* tok = nullptr;   // [B] input ids of the next step
    int* hist = nullptr;  // [B][hist_stride]
    int hist_stride = 0;
    DevState* st = nullptr;
    float* uniforms = nullptr;  // device copy for generate
    size_t uniforms_cap = 0;
    float* logit_log = nullptr;  // per-step logits for gh_session_generate
    size_t logit_log_cap = 0;

    // prompt pass (all prompt tokens at once): row-major [rows][width] activations
    float *pp_x = nullptr, *pp_q = nullptr, *pp_attn = nullptr, *pp_norm = nullptr, *pp_hidden = nullptr;
    size_t pp_rows = 0;
    float* score_logits = nullptr;  // [score_rows][vocab] logits of a block of rows being scored
    size_t score_rows = 0;

    // persistent engine
    Cell* cells = nullptr;  // xa, xb, q, kn, vn, at (d each), hid (F), token (1)
    size_t cells_count = 0;
    PersistCtl* ctl = nullptr;
    unsigned epoch = 1;         // tag base; grows with every step, never reused
    unsigned arrive_total = 0;  // logits phases completed so far
    int persist_grid = 0;
    unsigned long long* prof = nullptr;  // phase timestamps when GRADHIP_PROF_DUMP is set
    int prof_cap = 0;
    size_t persist_lds = 0;
    // ... its XCD-sharded form (kernels_xcd.h)
    bool xcd = false;         // the kernel and its buffers are ready
    bool xcd_row_lds = false;
    bool row_picks_only = false;  // GH_FLAG_ROW_PICKS
    Cell* xcells = nullptr;
    unsigned xcd_cells_count = 0;
    unsigned xcd_launches = 0;
    unsigned xcd_ring_units = 0, xcd_ring_units_wg0 = 0;
    size_t xcd_lds = 0;
    bool xcd_all_slices = false;  // every workgroup of an XCD takes a slice of the attention at any context

    float* host_logits = nullptr;  // pinned, B * V
    int* host_ids = nullptr;       // pinned staging for ids
    int* host_err = nullptr;       // pinned landing spot for the device error flag
    // streaming from the persistent kernel: pinned words the kernel writes / reads directly
    unsigned long long* feed = nullptr;  // [hist_stride] {token, tag} per pick of a launch
    unsigned* stop_word = nullptr;       // set by the host to end a run at the next pick
    unsigned feed_base = 0;              // tags of a launch are feed_base + 1 ...; never reused

    int pos = 0;     // host mirror of DevState
    int n_hist = 0;
    int picks = 0;
    gh_timing timing{};

    ~Session() {
#ifdef GH_PICK_TICKS
        {
            unsigned long long t[32] = {};
            if (hipMemcpyFromSymbol(t, HIP_SYMBOL(g_pick_ticks), sizeof(t)) == hipSuccess) {
                std::fprintf(stderr, "pick ticks (10 ns, summed):");
                for (unsigned long long v : t) std::fprintf(stderr, " %llu", v);
                std::fprintf(stderr, "\n");
            }
        }
#endif
        if (prof) {
            // Developer aid: phase-end timestamps of the last persistent launch.
            std::vector<unsigned long long> host(prof_cap);
            if (hipMemcpy(host.data(), prof, host.size() * 8, hipMemcpyDeviceToHost) == hipSuccess) {
                if (std::FILE* f = std::fopen(std::getenv("GRADHIP_PROF_DUMP"), "w")) {
                    for (size_t i = 0; i < host.size() / 2 && host[i]; i++) std::fprintf(f, "%llu\n", host[i]);
                    std::fprintf(f, "0\n");
                    for (size_t i = host.size() / 2; i + 3 < host.size() - 112 && host[i]; i += 4)
                        std::fprintf(f, "%llu\n%llu\n%llu\n", host[i + 2], host[i], host[i + 1]);
                    std::fprintf(f, "0\n");
                    for (size_t i = host.size() - 112; i < host.size(); i++) std::fprintf(f, "%llu\n", host[i]);
                    std::fclose(f);
                }
            }
            (void)hipFree(prof);
        }
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        if (exec_fused) (void)hipGraphExecDestroy(exec_fused);
        if (graph_fused) (void)hipGraphDestroy(graph_fused);
        if (best) (void)hipFree(best);
        for (hipEvent_t e : ev)
            if (e) (void)hipEventDestroy(e);
        for (void* p : {static_cast<void*>(kv_pool), static_cast<void*>(page_table),
                        static_cast<void*>(x), static_cast<void*>(h), static_cast<void*>(q),
                        static_cast<void*>(attn), static_cast<void*>(hidden),
                        static_cast<void*>(logits), static_cast<void*>(work),
                        static_cast<void*>(attn_part), static_cast<void*>(attn_tickets),
                        static_cast<void*>(tok), static_cast<void*>(hist), static_cast<void*>(st),
                        static_cast<void*>(uniforms),
                        static_cast<void*>(logit_log), static_cast<void*>(cells), static_cast<void*>(xcells),
                        static_cast<void*>(ctl), static_cast<void*>(pp_x), static_cast<void*>(pp_q),
                        static_cast<void*>(pp_attn), static_cast<void*>(pp_norm),
                        static_cast<void*>(pp_hidden), static_cast<void*>(score_logits)})
            if (p) (void)hipFree(p);
        if (host_logits) (void)hipHostFree(host_logits);
        if (host_ids) (void)hipHostFree(host_ids);
        if (host_err) (void)hipHostFree(host_err);
        if (feed) (void)hipHostFree(feed);
        if (stop_word) (void)hipHostFree(stop_word);
        if (stream) (void)hipStreamDestroy(stream);
    }
};

// The persistent kernel's workgroups wait for one another, so all of them have to
// be resident at once: one per compute unit.  Two such launches in flight at the
// same time (two sessions on two host threads) could each hold a part of the
// GPU and wait for the rest for ever.  Every entry point that launches the
// kernel therefore holds this process-wide lock from before the launch until
// the stream has been synchronised; sessions on other engines never take it.
static std::mutex g_persist_gate;

static thread_local int g_gate_depth = 0;

struct PersistGate {
    std::unique_lock<std::mutex> lock;
    explicit PersistGate(const struct Session& s);
    ~PersistGate() {
        if (lock.owns_lock()) g_gate_depth--;
    }
    PersistGate(const PersistGate&) = delete;
    PersistGate& operator=(const PersistGate&) = delete;
};

PersistGate::PersistGate(const Session& s) {
    if (s.engine != GH_ENGINE_PERSISTENT) return;
    // a stream callback that calls into another persistent session would wait for itself
    if (g_gate_depth > 0)
        throw ApiError{GH_ERR_RUNTIME, "a persistent-engine call is already running on this thread "
                                       "(token callbacks must not call into persistent-engine sessions)"};
    lock = std::unique_lock<std::mutex>(g_persist_gate);
    g_gate_depth++;
}

static KvLayout kv_layout(const Session& s) {
    return KvLayout{s.kv_pool,         s.page_table,           s.n_pages, s.pages_per_seq,
                    s.m->shape.heads,  s.m->shape.head_size(), s.page_shift};
}

template <typename T>
static void dev_alloc(T*& p, size_t n) {
    HIP_CHECK(hipMalloc(&p, std::max<size_t>(n, 1) * sizeof(T)));
    HIP_CHECK(hipMemset(p, 0, std::max<size_t>(n, 1) * sizeof(T)));
}

// ---- kernel dispatch

template <int PRO, int EPI>
static void launch_gemv(const GemvParams& p, int batch, hipStream_t st) {
    const int K = p.K;
    const bool aligned = (K % 256 == 0) && (p.in_stride % 4 == 0);
    const int kv = aligned ? K / 256 : 0;
    auto go = [&](auto kernel, int rows_per_wave) {
        const int waves = (p.N + rows_per_wave - 1) / rows_per_wave;
        const dim3 grid((waves + 3) / 4, batch);
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, st, p);
    };
    switch (kv) {
        case 1: go(gemv_kernel<1, 2, PRO, EPI>, 4); break;
        case 2: go(gemv_kernel<2, 2, PRO, EPI>, 4); break;
        case 3: go(gemv_kernel<3, 2, PRO, EPI>, 4); break;
        case 4: go(gemv_kernel<4, 2, PRO, EPI>, 4); break;
        case 8: go(gemv_kernel<8, 1, PRO, EPI>, 2); break;
        case 12: go(gemv_kernel<12, 1, PRO, EPI>, 2); break;
        default: go(gemv_kernel<0, 1, PRO, EPI>, 2); break;
    }
    HIP_CHECK(hipGetLastError());
}

static void launch_attn(const AttnParams& p, int batch, hipStream_t st) {
    const int hs = p.kv.head_size;
    const dim3 grid(p.max_chunks, p.kv.heads, batch);
    if (hs == 64) {
        if (p.kv.page_shift >= 5 && p.chunk % 128 == 0)
            hipLaunchKernelGGL(attn_decode64_kernel<true>, grid, dim3(256), 0, st, p);
        else
            hipLaunchKernelGGL(attn_decode64_kernel<false>, grid, dim3(256), 0, st, p);
        HIP_CHECK(hipGetLastError());
        return;
    }
    const size_t lds = (static_cast<size_t>(p.chunk) + 4 * hs + 8) * sizeof(float);
    switch (hs) {
        case 8: hipLaunchKernelGGL(attn_decode_kernel<8>, grid, dim3(256), lds, st, p); break;
        case 16: hipLaunchKernelGGL(attn_decode_kernel<16>, grid, dim3(256), lds, st, p); break;
        case 32: hipLaunchKernelGGL(attn_decode_kernel<32>, grid, dim3(256), lds, st, p); break;
        case 64: hipLaunchKernelGGL(attn_decode_kernel<64>, grid, dim3(256), lds, st, p); break;
        case 128: hipLaunchKernelGGL(attn_decode_kernel<128>, grid, dim3(256), lds, st, p); break;
        default: hipLaunchKernelGGL(attn_decode_kernel<0>, grid, dim3(256), lds, st, p); break;
    }
    HIP_CHECK(hipGetLastError());
}

// Batches of this size and up go to the matrix cores.
constexpr int kMinGemmBatch = 2;

// One projection with its fused prologue / epilogue; returns the launches made.
template <int PRO, int EPI>
static int project(Session& s, GemvParams g, hipStream_t st) {
    const int B = s.B;
    if (B >= kMinGemmBatch && gemm_shape_ok(g.K, g.in_stride)) {
        if (PRO == PRO_RMSNORM) {
            // the norm rides inside the projection
            launch_gemm16<EPI, true>(g, B, st);
            HIP_CHECK(hipGetLastError());
            return 1;
        }
        int launches = 1;
        if (PRO != PRO_PLAIN) {
            hipLaunchKernelGGL(norm_rows_kernel, dim3((B + 3) / 4), dim3(256), 0, st, g.in, g.gamma,
                               g.beta, s.h, B, g.K, static_cast<int>(PRO));
            HIP_CHECK(hipGetLastError());
            g.in = s.h;
            g.in_stride = g.K;
            launches++;
        }
        launch_gemm16<EPI, false>(g, B, st);
        HIP_CHECK(hipGetLastError());
        return launches;
    }
    launch_gemv<PRO, EPI>(g, B, st);
    return 1;
}

// final norm -> logits = h @ E^T (inference.cpp:251-254) from the rows in s.x
// advance: the launch also ends the step (pos_++).
static int enqueue_logits(Session& s, bool advance) {
    const Model& m = *s.m;
    const Shape& sh = m.shape;
    const bool modern = sh.modern();
    GemvParams g{};
    g.W = m.E;
    g.bias = nullptr;
    g.N = sh.vocab;
    g.K = sh.d_model;
    g.in = s.x;
    g.in_stride = sh.d_model;
    g.gamma = m.gf;
    g.beta = m.bf;
    g.out = s.logits;
    g.out_stride = sh.vocab;
    g.advance = advance ? s.st : nullptr;
    g.best = s.best;
    g.best_stride = s.best_stride;
    return modern ? project<PRO_RMSNORM, EPI_STORE>(s, g, s.stream)
                  : project<PRO_LAYERNORM, EPI_STORE>(s, g, s.stream);
}

// One InferenceSession::step for every sequence (inference.cpp:150-258),
// enqueued on the session stream.  Returns the number of launches.
// pick_first: the step opens with the greedy pick from what the last logits launch
// left in s.best (text_gen.cpp:52-60), which also writes the input rows.
static int enqueue_step(Session& s, bool pick_first = false) {
    const Model& m = *s.m;
    const Shape& sh = m.shape;
    const int d = sh.d_model, F = sh.d_ff(), B = s.B;
    const bool modern = sh.modern();
    hipStream_t st = s.stream;
    int launches = 0;

    if (pick_first) {
        hipLaunchKernelGGL(argmax_embed_kernel, dim3(B), dim3(kArgmaxThreads), 0, st, s.best, s.best_stride, s.st,
                           s.hist, s.hist_stride, s.tok, m.E, m.P, s.x, d);
    } else {
        hipLaunchKernelGGL(embed_kernel, dim3((d + 255) / 256, B), dim3(256), 0, st, m.E, m.P, s.tok,
                           s.st, s.x, d);
    }
    HIP_CHECK(hipGetLastError());
    launches++;

    // What a projection launch touches into the L2s for the projection after it (NextWeights):
    // the whole matrix, in the 16-row tiles that launch reads it in; up to 48 sequences.
    const bool touch = B >= kMinGemmBatch && B <= 48;
    const auto next_matrix = [&](const float* W, int N, int K) {
        NextWeights f{};
        if (!touch || !gemm_shape_ok(K, K) || N % 16 != 0) return f;
        f.base = W;
        f.chunk_lines = K / 2;  // 16 rows of K floats
        f.chunks = N / 16;
        const long long lines = static_cast<long long>(f.chunks) * f.chunk_lines;
        f.blocks = static_cast<int>(std::min<long long>(128, (lines + 8191) / 8192 * 8));  // up to four lines per thread of 256
        return f;
    };

    for (int l = 0; l < sh.layers; l++) {
        const LayerWeights& w = m.layers[l];
        GemvParams g{};
        g.kv = kv_layout(s);
        g.layer = l;
        g.d_model = d;
        g.st = s.st;

        // norm1 -> fused Q,K,V projection (+bias, RoPE) -> q buffer / cache row
        g.W = w.wqkv;
        g.bias = w.bqkv;
        g.N = 3 * d;
        g.K = d;
        g.in = s.x;
        g.in_stride = d;
        g.gamma = w.g1;
        g.beta = w.be1;
        g.out = s.q;
        g.out_stride = d;
        g.rope = modern;
        g.rope_cos = m.rope_cos;
        g.rope_sin = m.rope_sin;
        g.next = NextWeights{};  // attention follows
        launches += modern ? project<PRO_RMSNORM, EPI_QKV>(s, g, st)
                           : project<PRO_LAYERNORM, EPI_QKV>(s, g, st);

        AttnParams a{};
        a.q = s.q;
        a.out = s.attn;
        a.kv = g.kv;
        a.layer = l;
        a.d_model = d;
        a.st = s.st;
        a.chunk = s.attn_chunk;
        a.max_chunks = s.attn_max_chunks;
        a.scale = 1.0f / std::sqrt(static_cast<float>(sh.head_size()));
        a.part = s.attn_part;
        a.tickets = s.attn_tickets;
        launch_attn(a, B, st);
        launches++;

        // x += b_o + attn @ W_o
        g.W = w.wo;
        g.bias = w.bo;
        g.N = d;
        g.K = d;
        g.in = s.attn;
        g.in_stride = d;
        g.out = s.x;
        g.out_stride = d;
        g.next = next_matrix(w.w1, modern ? 2 * F : F, d);
        launches += project<PRO_PLAIN, EPI_RESID>(s, g, st);

        // norm2 -> FFN
        g.in = s.x;
        g.in_stride = d;
        g.gamma = w.g2;
        g.beta = w.be2;
        g.out = s.hidden;
        g.out_stride = F;
        g.W = w.w1;
        g.K = d;
        g.next = next_matrix(w.w2, d, F);
        if (modern) {
            g.bias = nullptr;
            g.N = 2 * F;
            launches += project<PRO_RMSNORM, EPI_SWIGLU>(s, g, st);
        } else {
            g.bias = w.b1;
            g.N = F;
            launches += project<PRO_LAYERNORM, EPI_GELU>(s, g, st);
        }
        g.W = w.w2;
        g.bias = modern ? nullptr : w.b2;
        g.N = d;
        g.K = F;
        g.in = s.hidden;
        g.in_stride = F;
        g.out = s.x;
        g.out_stride = d;
        g.next = l + 1 < sh.layers ? next_matrix(m.layers[l + 1].wqkv, 3 * d, d) : NextWeights{};
        launches += project<PRO_PLAIN, EPI_RESID>(s, g, st);
    }

    launches += enqueue_logits(s, /*advance=*/true);
    return launches;
}

// ---- persistent engine

using PersistKernel = void (*)(const PersistParams);

// The shapes the persistent kernel is built for (head size 64, d_model and FFN
// width multiples of 256); nullptr for anything else.
// row_lds: the sampler's working row fits in LDS.
template <bool ROW_LDS, bool FEED>
static PersistKernel persist_kernel_of(const Shape& sh) {
    if (sh.head_size() != 64) return nullptr;
    const int d = sh.d_model, F = sh.d_ff();
    if (sh.modern()) {
        if (d == 768 && F == 2048) return persist_decode_kernel<3, 8, true, ROW_LDS, FEED>;
        return nullptr;
    }
    if (d == 512) return persist_decode_kernel<2, 8, false, ROW_LDS, FEED>;
    if (d == 768) return persist_decode_kernel<3, 12, false, ROW_LDS, FEED>;
    if (d == 1024) return persist_decode_kernel<4, 16, false, ROW_LDS, FEED>;
    return nullptr;
}
// feed: the variant that reports its picks to the host and can be told to stop.
static PersistKernel persist_kernel_for(const Shape& sh, bool row_lds, bool feed = false) {
    if (feed) return row_lds ? persist_kernel_of<true, true>(sh) : persist_kernel_of<false, true>(sh);
    return row_lds ? persist_kernel_of<true, false>(sh) : persist_kernel_of<false, false>(sh);
}


// ---- the XCD-sharded form of the persistent kernel (kernels_xcd.h)

// The XCD-sharded kernel runs only where GH_FLAG_XCD_PERSISTENT asks for it.  It used to
// be the default for launches that start at position 1024 or later, where it spreads a
// head's context over the workgroups of an XCD; since the all-to-all kernel shares a
// head's long context among idle workgroups itself it is the faster one at every
// position.  Per token on one box, Llama block d768 L8 V16000, greedy, XCD-sharded /
// all-to-all: positions 256..512 168 / 132, 512..768 178 / 144, 1024..1280 196 / 149,
// 2048..2304 228 / 156, 3072..3328 259 / 160, 3800..4056 277 / 162.

using XcdKernel = void (*)(const XcdParams);

static XcdKernel xcd_kernel_for(const Shape& sh, bool row_lds, bool feed) {
    if (!sh.modern() || sh.head_size() != 64 || sh.d_model != 768) return nullptr;
    if (feed) return row_lds ? xcd_decode_kernel<3, true, true> : xcd_decode_kernel<3, false, true>;
    return row_lds ? xcd_decode_kernel<3, true, false> : xcd_decode_kernel<3, false, false>;
}

// Splits the model over eight XCDs: heads g and g + 8, and a run of hidden units
// sized so that every XCD streams about the same number of bytes per layer.
// False when the kernel's split does not fit the shape.
static bool xcd_geometry(const Shape& sh, XcdGeom& gm) {
    if (!xcd_kernel_for(sh, true, false)) return false;
    const int D = sh.d_model, F = sh.d_ff(), H = sh.heads;
    if (H < kXcds || H > 2 * kXcds || F % 4 != 0 || sh.layers < 1 || sh.max_len > 4096) return false;
    gm = XcdGeom{};
    gm.D = D;
    gm.F = F;
    gm.V = sh.vocab;
    gm.L = sh.layers;
    gm.H = H;
    const double per_head = 4.0 * 64.0 * D, per_unit = 3.0 * D;
    const double target = (H * per_head + F * per_unit) / kXcds;
    double want_sum = 0.0;
    int at = 0;
    for (int g = 0; g < kXcds; g++) {
        XcdShard& x = gm.shard[g];
        x.nh = g + kXcds < H ? 2 : 1;
        x.head[0] = g;
        x.head[1] = g + kXcds < H ? g + kXcds : g;
        want_sum += (target - x.nh * per_head) / per_unit;
        int end = g == kXcds - 1 ? F : static_cast<int>(std::lround(want_sum / 4.0)) * 4;
        end = std::min(std::max(end, at), F);
        x.u0 = at;
        x.nu = end - at;
        at = end;
        if (x.nu < kWgPerXcd || x.nu > 512) return false;  // every workgroup owns a unit; the XCD's units fit the LDS row
    }
    unsigned stride = 0;
    for (int g = 0; g < kXcds; g++)
        for (int r = 0; r < kWgPerXcd; r++) {
            const XcdWg w = xcd_wg(gm, g, r);
            if (w.nu < 1 || w.nu > kXcdMaxUnitsPerWg) return false;
            stride = std::max(stride, w.layers_units + w.logits_units);
        }
    gm.stride_units = stride;
    return true;
}

// One block of a weight matrix on its way into a workgroup's stream: rows x cols
// floats from blob[src + row * src_ld] to stream[dst + row * dst_ld], each column
// multiplied by a norm gain when gamma >= 0 (the gain of the norm in front of the
// product is folded into the weights: (g * x) . w == x . (g * w)).
struct XcdCopy {
    unsigned long long dst, src;
    long long gamma;
    int rows, cols, src_ld, dst_ld;
};

__global__ void xcd_copy_kernel(const XcdCopy* list, const float* __restrict__ blob, float* __restrict__ out) {
    const XcdCopy c = list[blockIdx.x];
    const int n = c.rows * c.cols;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int row = i / c.cols, col = i - row * c.cols;
        float v = blob[c.src + static_cast<size_t>(row) * c.src_ld + col];
        if (c.gamma >= 0) v *= blob[c.gamma + col];
        out[c.dst + static_cast<size_t>(row) * c.dst_ld + col] = v;
    }
}

// Builds the per-workgroup weight streams of a model (once).
static void xcd_build_stream(const Model& m) {
    std::lock_guard<std::mutex> lock(m.xcd_mutex);
    if (m.xcd_stream) return;
    XcdGeom gm;
    if (!xcd_geometry(m.shape, gm)) throw ApiError{GH_ERR_RUNTIME, "no XCD split for this model shape"};
    const size_t D = gm.D, F = gm.F, RW = D / kWgPerXcd;
    const size_t stride_floats = static_cast<size_t>(gm.stride_units) * kXcdUnit / 4;
    auto at = [&](const float* ptr) { return static_cast<unsigned long long>(ptr - m.blob); };
    std::vector<XcdCopy> list;
    for (int g = 0; g < kXcds; g++)
        for (int r = 0; r < kWgPerXcd; r++) {
            const XcdWg w = xcd_wg(gm, g, r);
            const XcdShard& sh = gm.shard[g];
            const size_t base = static_cast<size_t>(g * kWgPerXcd + r) * stride_floats;
            for (int l = 0; l < gm.L; l++) {
                const LayerWeights& lw = m.layers[l];
                const size_t lb = base + static_cast<size_t>(l) * (w.layer_bytes / 4);
                // pairs of Q / K / V rows: pair i of the XCD is (head slot, section, j)
                for (int q = 0; q < w.ppw; q++) {
                    const int pi = r * w.ppw + q, hi = pi / 96, rem = pi % 96, sec = rem / 32, j = rem % 32;
                    const size_t row = static_cast<size_t>(sec) * D + static_cast<size_t>(sh.head[hi]) * 64 + 2 * j;
                    const size_t pb = lb + static_cast<size_t>(q) * (w.pair_bytes / 4);
                    list.push_back({pb, at(lw.wqkv) + row * D, static_cast<long long>(at(lw.g1)), 2,
                                    static_cast<int>(D), static_cast<int>(D), static_cast<int>(D)});
                    list.push_back({pb + 2 * D, at(lw.bqkv) + row, -1, 1, 2, 2, 2});
                }
                // W_o: this workgroup's rows, the columns of the XCD's heads
                for (int hi = 0; hi < w.nh; hi++)
                    list.push_back({lb + w.o_wo / 4 + static_cast<size_t>(hi) * 64,
                                    at(lw.wo) + (static_cast<size_t>(r) * RW) * D + static_cast<size_t>(sh.head[hi]) * 64,
                                    -1, static_cast<int>(RW), 64, static_cast<int>(D), w.KC});
                list.push_back({lb + w.o_bo / 4, at(lw.bo) + static_cast<size_t>(r) * RW, -1, 1, static_cast<int>(RW),
                                static_cast<int>(RW), static_cast<int>(RW)});
                // gate and up rows of this workgroup's hidden units (row 2u gate, 2u + 1 up)
                list.push_back({lb + w.o_gu / 4, at(lw.w1) + static_cast<size_t>(2 * w.ub) * D,
                                static_cast<long long>(at(lw.g2)), 2 * w.nu, static_cast<int>(D),
                                static_cast<int>(D), static_cast<int>(D)});
                // W_down: this workgroup's rows, the columns of the XCD's hidden units
                list.push_back({lb + w.o_dn / 4, at(lw.w2) + (static_cast<size_t>(r) * RW) * F + static_cast<size_t>(w.u0),
                                -1, static_cast<int>(RW), w.UG, static_cast<int>(F), w.UG});
            }
            // its rows of the logits matrix, with the final norm's gain
            if (w.nrows > 0)
                list.push_back({base + static_cast<size_t>(w.layers_units) * kXcdUnit / 4,
                                at(m.E) + static_cast<size_t>(w.v0) * D, static_cast<long long>(at(m.gf)), w.nrows,
                                static_cast<int>(D), static_cast<int>(D), static_cast<int>(D)});
        }
    const size_t total = static_cast<size_t>(kXcds * kWgPerXcd) * stride_floats;
    char* stream = nullptr;
    XcdCopy* dlist = nullptr;
    HIP_CHECK(hipMalloc(&stream, total * sizeof(float)));
    try {
        HIP_CHECK(hipMemset(stream, 0, total * sizeof(float)));
        HIP_CHECK(hipMalloc(&dlist, list.size() * sizeof(XcdCopy)));
        HIP_CHECK(hipMemcpy(dlist, list.data(), list.size() * sizeof(XcdCopy), hipMemcpyHostToDevice));
        hipLaunchKernelGGL(xcd_copy_kernel, dim3(static_cast<unsigned>(list.size())), dim3(256), 0, nullptr, dlist,
                           m.blob, reinterpret_cast<float*>(stream));
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipDeviceSynchronize());
    } catch (...) {
        if (dlist) (void)hipFree(dlist);
        (void)hipFree(stream);
        throw;
    }
    HIP_CHECK(hipFree(dlist));
    m.xcd_geom = gm;
    m.xcd_stream = stream;
}

static const char* persist_unavailable(const Session& s, int lds_bytes, int cus) {
    const Shape& sh = s.m->shape;
    if (s.B != 1) return "the persistent engine decodes one sequence";
    if (!persist_kernel_for(sh, s.pick_row_in_lds)) return "the persistent engine has no kernel for this model shape";
    if (sh.max_len > 4096) return "the persistent engine handles contexts up to 4096";
    if (cus < sh.heads) return "the GPU has fewer compute units than the model has heads";
    (void)lds_bytes;
    // The kernel finds a layer's tensors by address arithmetic (layer_at): they must
    // follow each other without gaps, layer after layer.
    {
        const size_t d = sh.d_model, F = sh.d_ff();
        const size_t per_layer = layer_floats(d, F, sh.modern());
        const float* base = s.m->layers[0].wqkv;
        for (size_t l = 0; l < s.m->layers.size(); l++) {
            const LayerWeights& w = s.m->layers[l];
            const float* b = base + l * per_layer;
            const float* want[12];
            size_t i = 0;
            for (const size_t n : {3 * d * d, 3 * d, d * d, d, (sh.modern() ? 2 : 1) * F * d, F, d * F, d, d, d, d, d}) {
                want[i++] = b;
                b += n;
            }
            const float* have[12] = {w.wqkv, w.bqkv, w.wo, w.bo, w.w1, w.b1, w.w2, w.b2, w.g1, w.be1, w.g2, w.be2};
            for (i = 0; i < 12; i++)
                if (have[i] != want[i]) return "the persistent engine needs the layers' tensors back to back";
        }
    }
    return nullptr;
}

// One launch: n_prompt steps fed from the history, then rounds of pick + step.
// feed: the kernel reports every pick in the session's pinned feed and honours its
// stop word and stop_token.
static void persist_run(Session& s, int n_prompt, int n_steps, int n_picks, bool start_with_pick,
                        const gh_sampling* o, const float* dev_uniforms, int u_stride, uint64_t seed,
                        float* logit_log, bool feed = false, int stop_token = -1, int tok0 = -1) {
    const Model& m = *s.m;
    const Shape& sh = m.shape;
    if (n_steps <= 0 && n_picks <= 0) return;
    // Tags are (epoch + step) * (layers + 1) * 8 + phase in 32 bits and are matched by
    // equality, so they must not come round to a value a stale cell may still hold:
    // long before that the cells are cleared on the stream (tag 0 is never used) and
    // the epoch starts over.  Arrival counts are compared by wrap-safe difference.
    {
        const unsigned long long per_step = static_cast<unsigned long long>(sh.layers + 1) * 8ull;
        const unsigned long long last = (static_cast<unsigned long long>(s.epoch) + n_steps + 2ull) * per_step + 8ull;
        if (last >= 0xF0000000ull) {
            HIP_CHECK(hipMemsetAsync(s.cells, 0, s.cells_count * sizeof(Cell), s.stream));
            if (s.xcells) HIP_CHECK(hipMemsetAsync(s.xcells, 0, s.xcd_cells_count * sizeof(Cell), s.stream));
            s.epoch = 1;
        }
    }
    PersistParams p{};
    p.E = m.E;
    p.P = m.P;
    p.layer0 = m.layers[0].wqkv;
    p.gf = m.gf;
    p.bf = m.bf;
    p.rope_cos = m.rope_cos;
    p.rope_sin = m.rope_sin;
    p.d = sh.d_model;
    p.F = sh.d_ff();
    p.V = sh.vocab;
    p.L = sh.layers;
    p.H = sh.heads;
    p.kv = kv_layout(s);
    p.cells = s.cells;
    p.logits = s.logits;
    p.logit_log = logit_log;
    p.ctl = s.ctl;
    p.hist = s.hist;
    p.pos0 = s.pos;
    p.n_prompt = n_prompt;
    p.n_steps = n_steps;
    p.n_picks = n_picks;
    p.start_with_pick = start_with_pick ? 1 : 0;
    p.tok0 = tok0;
    p.wg_picks = s.row_picks_only ? 0 : 1;
    p.epoch = s.epoch;
    p.arrive_base = s.arrive_total;
    p.spin_limit = 1u << 18;
    p.prof = s.prof;
    p.prof_cap = s.prof_cap;
    p.stop_token = -1;
    if (feed) {
        p.feed = s.feed;
        p.feed_base = s.feed_base;
        p.stop_request = s.stop_word;
        p.stop_token = stop_token;
        s.feed_base += static_cast<unsigned>(n_picks) + 1u;
    }
    PickParams& k = p.pick;
    k.logits = s.logits;
    k.V = sh.vocab;
    k.hist = s.hist;
    k.hist_stride = s.hist_stride;
    k.n_hist = s.n_hist + n_prompt;
    k.pick_idx = s.picks;
    k.tok = s.tok;
    if (o) {
        k.temperature = o->temperature;
        k.top_k = o->top_k;
        k.top_p = o->top_p;
        k.penalty = o->repetition_penalty;
        k.greedy = o->greedy;
    }
    k.uniforms = dev_uniforms;
    k.u_stride = u_stride;
    k.seed_lo = static_cast<unsigned>(seed & 0xFFFFFFFFu);
    k.seed_hi = static_cast<unsigned>(seed >> 32);
    k.work = s.work;
    k.work_stride = s.work_stride;
    k.sort_cap = kPickWorkFloats;

    if (s.xcd) {
        XcdParams x{};
        x.b = p;
        x.gm = m.xcd_geom;
        x.stream = m.xcd_stream;
        x.xc = s.xcells;
        x.ring_units = s.xcd_ring_units;
        x.ring_units_wg0 = s.xcd_ring_units_wg0;
        x.launch_base = s.xcd_launches * kWgPerXcd;
        // Eight slices per head keep the merge short; contexts beyond 256 positions give
        // every workgroup of the XCD a slice.
        x.attn_slices = (s.xcd_all_slices || s.pos + n_steps > 256) ? 0 : 8;
        s.xcd_launches++;
        hipLaunchKernelGGL(xcd_kernel_for(sh, s.xcd_row_lds, feed), dim3(kXcds * kWgPerXcd), dim3(kXcdThreads),
                           s.xcd_lds, s.stream, x);
    } else {
        PersistKernel kernel = persist_kernel_for(sh, s.pick_row_in_lds, feed);
        hipLaunchKernelGGL(kernel, dim3(s.persist_grid), dim3(kPersistThreads), s.persist_lds, s.stream, p);
    }
    HIP_CHECK(hipGetLastError());

    // Host mirrors.  Logits are produced by the last prompt step and every later one.
    int logits_phases = 0;
    for (int i = 0; i < n_steps; i++)
        if (i >= n_prompt - 1 || logit_log || i == n_steps - 1) logits_phases++;
    s.arrive_total += static_cast<unsigned>(logits_phases);
    s.epoch += static_cast<unsigned>(n_steps) + 1u;
    s.pos += n_steps;
    s.n_hist += n_prompt + n_picks;
    s.picks += n_picks;
}

// After a synchronisation: did the kernel give up waiting somewhere?
static void check_persist_abort(Session& s) {
    if (s.engine != GH_ENGINE_PERSISTENT) return;
    HIP_CHECK(hipMemcpy(s.host_err, &s.ctl->abort, sizeof(int), hipMemcpyDeviceToHost));
    if (*s.host_err) {
        unsigned where = 0;
        HIP_CHECK(hipMemcpy(s.host_err, &s.ctl->where, sizeof(int), hipMemcpyDeviceToHost));
        where = static_cast<unsigned>(*s.host_err);
        throw ApiError{GH_ERR_DEVICE, "persistent decode kernel abandoned a wait (phase tag "
                                          + std::to_string(where) + "); the session is unusable"};
    }
}

static void run_step(Session& s, bool pick_first = false) {
    if (s.engine == GH_ENGINE_GRAPH) {
        HIP_CHECK(hipGraphLaunch(pick_first ? s.exec_fused : s.exec, s.stream));
    } else {
        enqueue_step(s, pick_first);
    }
    s.pos++;
}

static void check_capacity(const Session& s) {
    // inference.cpp:151-153
    if (s.pos >= s.m->shape.max_len)
        throw ApiError{GH_ERR_RUNTIME, "InferenceSession: context exceeds max_len"};
}

static void check_ids(const Session& s, const int32_t* ids, size_t n) {
    // inference.cpp:154-156
    for (size_t i = 0; i < n; i++)
        if (ids[i] < 0 || ids[i] >= s.m->shape.vocab)
            throw ApiError{GH_ERR_OUT_OF_RANGE, "InferenceSession: token id out of vocab range"};
}

__global__ void set_state_kernel(DevState* st, int pos, int n_hist, int picks) {
    st->pos = pos;
    st->n_hist = n_hist;
    st->picks = picks;
    st->hist_lead = n_hist - pos;
}

// tok[b] = hist[b][t]
__global__ void load_tok_kernel(const int* hist, int stride, int t, int* tok, int B) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < B) tok[b] = hist[static_cast<size_t>(b) * stride + t];
}

// hist[b][t] = tok[b]
__global__ void store_hist_kernel(int* hist, int stride, int t, const int* tok, int B) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < B) hist[static_cast<size_t>(b) * stride + t] = tok[b];
}

static void reset_session(Session& s) {
    s.pos = 0;
    s.n_hist = 0;
    s.picks = 0;
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, s.stream, s.st, 0, 0, 0);
    HIP_CHECK(hipGetLastError());
}

static std::unique_ptr<Session> create_session(const Model& m, const gh_session_opts& o) {
    require_gpu();
    if (o.batch < 1) throw ApiError{GH_ERR_INVALID_ARGUMENT, "batch must be at least 1"};
    auto sp = std::make_unique<Session>();
    Session& s = *sp;
    s.m = &m;
    s.B = o.batch;
    s.engine = o.engine;
    if (s.engine < GH_ENGINE_AUTO || s.engine > GH_ENGINE_PERSISTENT)
        throw ApiError{GH_ERR_INVALID_ARGUMENT, "unknown engine"};
    const Shape& sh = m.shape;
    const int page_tokens = o.page_tokens > 0 ? o.page_tokens : 64;
    if (page_tokens & (page_tokens - 1))
        throw ApiError{GH_ERR_INVALID_ARGUMENT, "page_tokens must be a power of two"};
    s.page_shift = 0;
    while ((1 << s.page_shift) < page_tokens) s.page_shift++;
    s.pages_per_seq = (sh.max_len + page_tokens - 1) / page_tokens;
    s.n_pages = s.pages_per_seq * s.B;

    const size_t d = sh.d_model, F = sh.d_ff(), V = sh.vocab, B = s.B;
    HIP_CHECK(hipStreamCreate(&s.stream));
    for (hipEvent_t& e : s.ev) HIP_CHECK(hipEventCreate(&e));

    // Page table: identity, or a fixed scramble to exercise the indirection.
    std::vector<int> table(static_cast<size_t>(s.n_pages));
    std::iota(table.begin(), table.end(), 0);
    if (o.shuffle_pages) {
        uint64_t x = 0x9E3779B97F4A7C15ull;
        for (size_t i = table.size(); i > 1; i--) {
            x ^= x << 13;
            x ^= x >> 7;
            x ^= x << 17;
            std::swap(table[i - 1], table[x % i]);
        }
    }
    dev_alloc(s.page_table, table.size());
    HIP_CHECK(hipMemcpy(s.page_table, table.data(), table.size() * sizeof(int),
                        hipMemcpyHostToDevice));
    const size_t page_floats = 2ull * sh.heads * page_tokens * sh.head_size();
    dev_alloc(s.kv_pool, static_cast<size_t>(sh.layers) * s.n_pages * page_floats);

    dev_alloc(s.x, B * d);
    dev_alloc(s.h, B * std::max(d, F));
    dev_alloc(s.q, B * d);
    dev_alloc(s.attn, B * d);
    dev_alloc(s.hidden, B * F);
    dev_alloc(s.logits, B * V);
    s.work_stride = static_cast<int>((V + kPickThreads + 3) / 4 * 4);
    dev_alloc(s.work, B * static_cast<size_t>(s.work_stride));
    dev_alloc(s.tok, B);
    s.hist_stride = sh.max_len + 2;
    dev_alloc(s.hist, B * s.hist_stride);
    dev_alloc(s.st, 1);
    HIP_CHECK(hipHostMalloc(&s.host_logits, B * V * sizeof(float)));
    HIP_CHECK(hipHostMalloc(&s.host_ids, B * s.hist_stride * sizeof(int)));
    HIP_CHECK(hipHostMalloc(&s.host_err, sizeof(int)));
    HIP_CHECK(hipHostMalloc(&s.feed, s.hist_stride * sizeof(unsigned long long), hipHostMallocCoherent));
    HIP_CHECK(hipHostMalloc(&s.stop_word, sizeof(unsigned), hipHostMallocCoherent));
    std::memset(s.feed, 0, s.hist_stride * sizeof(unsigned long long));
    *s.stop_word = 0;

    // Attention chunking: a (sequence, head) is split over several workgroups in
    // runs of 512 cache positions, or 256 when that leaves fewer than ~192
    // workgroups at a full context.  Longer runs win even when they leave compute
    // units idle (measured at context 2048 with 2..16 sequences and at context 256
    // with 8..64: every workgroup pays a dependent chain position -> page table ->
    // cache rows -> merge, and a short run does not amortise it).
    int chunk = 512;
    if (static_cast<long>(B) * sh.heads * ((sh.max_len + chunk - 1) / chunk) < 192) chunk = 256;
    if (o.flags & GH_FLAG_SMALL_ATTENTION_CHUNKS) chunk = 16;
    s.attn_chunk = chunk;
    s.attn_max_chunks = (sh.max_len + chunk - 1) / chunk;
    dev_alloc(s.attn_part, B * sh.heads * s.attn_max_chunks * (sh.head_size() + 2));
    dev_alloc(s.attn_tickets, B * sh.heads);

    // The pick keeps its working row in LDS when vocab floats fit there beside the
    // work area and the kernel's static arrays; otherwise the row stays in global
    // memory.
    int dev = 0, lds_bytes = 0;
    HIP_CHECK(hipGetDevice(&dev));
    HIP_CHECK(hipDeviceGetAttribute(&lds_bytes, hipDeviceAttributeMaxSharedMemoryPerBlock, dev));
    const size_t reserve = 8192;
    s.pick_global_scratch = (o.flags & GH_FLAG_PICK_GLOBAL_SCRATCH) != 0;
    s.row_picks_only = (o.flags & GH_FLAG_ROW_PICKS) != 0;
    s.use_prompt_pass = (o.flags & GH_FLAG_STEPWISE_PROMPT) == 0;
    s.pick_row_in_lds = !s.pick_global_scratch
                        && (V + kPickWorkFloats) * sizeof(float) + reserve <= static_cast<size_t>(lds_bytes);
    if (s.pick_row_in_lds) {
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(pick_kernel<true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize,
                                      lds_bytes - static_cast<int>(reserve)));
    }

    {
        hipDeviceProp_t prop;
        HIP_CHECK(hipGetDeviceProperties(&prop, dev));
        const char* why = persist_unavailable(s, lds_bytes, prop.multiProcessorCount);
        if (s.engine == GH_ENGINE_PERSISTENT && why) throw ApiError{GH_ERR_INVALID_ARGUMENT, why};
        if (s.engine == GH_ENGINE_AUTO) s.engine = why ? GH_ENGINE_GRAPH : GH_ENGINE_PERSISTENT;
        if (s.engine == GH_ENGINE_PERSISTENT) {
            const size_t work = d + std::max(d, F) + 192 + kPersistWaves * 4 * 68 + s.pages_per_seq;
            const size_t pick = (s.pick_row_in_lds ? V : 0) + kPickWorkFloats;
            s.persist_lds = std::max(work, pick) * sizeof(float);
            // As many workgroups as give every wavefront exactly one item of the widest phase (the
            // FFN1 row pairs): workgroups beyond that have nothing to do there and still take part
            // in every exchange.  Per token: d512 F2048 (GPT-2) 75.2 us on 256 workgroups, 67.4 on
            // 128; d768 F3072 (GPT-2) 127.0 on 256, 119.0 on 192; the Llama block d768 F2048 (2048
            // items) 116.9 on 256, 129.5 on 192.  Between these sizes every step of 16 either way
            // is slower.
            const int ffn1_items = static_cast<int>(sh.modern() ? F : F / 2);
            const int want = ((ffn1_items + kPersistWaves - 1) / kPersistWaves + 15) / 16 * 16;
            s.persist_grid = std::min(std::min(prop.multiProcessorCount, 256), std::max(32, want));
            // the exchange cells, the token cell (and one of padding), then what the workgroups
            // leave for a pick each of them makes itself: nine planes of one cell per
            // workgroup and a stop word
            s.cells_count = 6 * d + F + 2 + 9 * static_cast<size_t>(s.persist_grid) + 1;
            // and, from an even index, what the workgroups that share a head's long context
            // leave for the head's own: up to fifteen shares of 66 cells for each of up to 16 heads
            s.cells_count = ((s.cells_count + 1) & ~static_cast<size_t>(1)) + 16 * 15 * 66;
            dev_alloc(s.cells, s.cells_count);
            // Rows of the cache written earlier in a launch by other workgroups are read
            // with ordinary loads.  That is sound only because a row is never read before
            // it is written and shares no 128-byte cache line with another row: rows are
            // head_size floats from a base that hipMalloc aligns.
            if ((sh.head_size() * sizeof(float)) % 128 != 0 || reinterpret_cast<uintptr_t>(s.kv_pool) % 256 != 0)
                throw ApiError{GH_ERR_DEVICE, "persistent engine: cache rows are not whole 128-byte lines"};
            dev_alloc(s.ctl, 1);
            if (const char* near = std::getenv("GRADHIP_TEST_NEAR_WRAP")) {
                // Test aid: start the session's two running counts `near` steps before the
                // points where the arrival counters wrap around 2^32 and where the cell tags
                // are re-based, so that a short run crosses both.
                // (a test hook: values outside 1..4096 are ignored, so a stray variable cannot
                // leave the counters inconsistent)
                const long asked = std::strtol(near, nullptr, 10);
                const unsigned n = asked >= 1 && asked <= 4096 ? static_cast<unsigned>(asked) : 0u;
                if (n != 0u) {
                    s.arrive_total = (0u - n * static_cast<unsigned>(s.persist_grid)) / static_cast<unsigned>(s.persist_grid);
                    const unsigned sum = s.arrive_total * static_cast<unsigned>(s.persist_grid);
                    HIP_CHECK(hipMemcpy(&s.ctl->arrive[0], &sum, sizeof(sum), hipMemcpyHostToDevice));
                    s.epoch = static_cast<unsigned>(0xF0000000ull / (static_cast<unsigned long long>(sh.layers + 1) * 8ull)) - n;
                }
            }
            if (std::getenv("GRADHIP_PROF_DUMP")) {
                s.prof_cap = 1 << 16;
                dev_alloc(s.prof, s.prof_cap);
            }
            for (const bool feed : {false, true})
                HIP_CHECK(hipFuncSetAttribute(
                    reinterpret_cast<const void*>(persist_kernel_for(sh, s.pick_row_in_lds, feed)),
                    hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(s.persist_lds)));
            s.launches_per_step = 1;

            // The XCD-sharded form, where the chip and the shape allow it: 8 XCDs of 32
            // compute units, and a ring of a power-of-two size beside the work area
            // (workgroup 0's ring is smaller when the pick keeps its row in LDS).
            XcdGeom gm;
            const bool xcd_wanted = (o.flags & GH_FLAG_XCD_PERSISTENT) != 0;
            if ((o.flags & GH_FLAG_XCD_PERSISTENT) != 0 && (o.flags & GH_FLAG_CLASSIC_PERSISTENT) != 0)
                throw ApiError{GH_ERR_INVALID_ARGUMENT, "GH_FLAG_CLASSIC_PERSISTENT and GH_FLAG_XCD_PERSISTENT exclude each other"};
            if (xcd_wanted && prop.multiProcessorCount == kXcds * kWgPerXcd && xcd_geometry(sh, gm)
                && s.pages_per_seq <= 1024) {
                const size_t statics = 4096;  // the kernel's static LDS (control words, the pick's scratch), rounded up
                const size_t work = (2 * d + kWgPerXcd * kApCells + 512 + kXcdRowWaves * (128 + 32) + 192 + s.pages_per_seq)
                                    * sizeof(float);
                const size_t pick_small = kPickWorkFloats * sizeof(float);
                const size_t pick_row = (V + kPickWorkFloats) * sizeof(float);
                size_t ring = 128 * 1024;
                while (ring + std::max(work, pick_small) + statics > static_cast<size_t>(lds_bytes)) ring /= 2;
                size_t ring0 = ring;
                s.xcd_row_lds = false;
                if (!s.pick_global_scratch) {
                    size_t rr = ring;
                    while (rr >= 32 * 1024 && rr + std::max(work, pick_row) + statics > static_cast<size_t>(lds_bytes)) rr /= 2;
                    if (rr >= 32 * 1024) {
                        ring0 = rr;
                        s.xcd_row_lds = true;
                    }
                }
                if (ring >= 64 * 1024) {
                    xcd_build_stream(m);
                    s.xcd = true;
                    s.xcd_all_slices = (o.flags & GH_FLAG_SMALL_ATTENTION_CHUNKS) != 0;
                    s.xcd_ring_units = static_cast<unsigned>(ring / kXcdUnit);
                    s.xcd_ring_units_wg0 = static_cast<unsigned>(ring0 / kXcdUnit);
                    s.xcd_lds = std::max(ring + work, ring0 + std::max(work, s.xcd_row_lds ? pick_row : pick_small));
                    const XcdCells cl = xcd_cells(m.xcd_geom);
                    s.xcd_cells_count = cl.total;
                    dev_alloc(s.xcells, cl.total);
                    for (const bool feed : {false, true})
                        HIP_CHECK(hipFuncSetAttribute(
                            reinterpret_cast<const void*>(xcd_kernel_for(sh, s.xcd_row_lds, feed)),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(s.xcd_lds)));
                }
            }
        }
    }

    reset_session(s);
    HIP_CHECK(hipStreamSynchronize(s.stream));

    // The matrix-core logits launch can leave what a greedy pick needs (a batch of at
    // least two sequences takes it; the wide form and the tiled form both can).
    if (s.engine != GH_ENGINE_PERSISTENT && s.B >= kMinGemmBatch && gemm_shape_ok(sh.d_model, sh.d_model)) {
        s.best_stride = (sh.vocab + 15) / 16;
        dev_alloc(s.best, static_cast<size_t>(s.B) * s.best_stride);
    }

    if (s.engine == GH_ENGINE_PERSISTENT) {
        // nothing to record: one launch runs any number of steps
    } else if (s.engine == GH_ENGINE_GRAPH) {
        HIP_CHECK(hipStreamBeginCapture(s.stream, hipStreamCaptureModeThreadLocal));
        try {
            s.launches_per_step = enqueue_step(s);
        } catch (...) {
            hipGraph_t g = nullptr;
            (void)hipStreamEndCapture(s.stream, &g);
            if (g) (void)hipGraphDestroy(g);
            throw;
        }
        HIP_CHECK(hipStreamEndCapture(s.stream, &s.graph));
        HIP_CHECK(hipGraphInstantiate(&s.exec, s.graph, nullptr, nullptr, 0));
        if (s.best) {
            HIP_CHECK(hipStreamBeginCapture(s.stream, hipStreamCaptureModeThreadLocal));
            try {
                enqueue_step(s, true);
            } catch (...) {
                hipGraph_t g = nullptr;
                (void)hipStreamEndCapture(s.stream, &g);
                if (g) (void)hipGraphDestroy(g);
                throw;
            }
            HIP_CHECK(hipStreamEndCapture(s.stream, &s.graph_fused));
            HIP_CHECK(hipGraphInstantiate(&s.exec_fused, s.graph_fused, nullptr, nullptr, 0));
        }
    } else {
        // Count the launches of one step without running it twice: a dry capture.
        HIP_CHECK(hipStreamBeginCapture(s.stream, hipStreamCaptureModeThreadLocal));
        hipGraph_t g = nullptr;
        try {
            s.launches_per_step = enqueue_step(s);
        } catch (...) {
            (void)hipStreamEndCapture(s.stream, &g);
            if (g) (void)hipGraphDestroy(g);
            throw;
        }
        HIP_CHECK(hipStreamEndCapture(s.stream, &g));
        if (g) (void)hipGraphDestroy(g);
    }
    return sp;
}

// commit: the pick becomes part of the token history right away (the generate
// loop steps it next); otherwise the caller's following step() records it.
static void launch_pick(Session& s, const gh_sampling& o, const float* dev_uniforms, int u_stride,
                        uint64_t seed, bool commit) {
    PickParams p{};
    p.logits = s.logits;
    p.work = s.work;
    p.V = s.m->shape.vocab;
    p.hist = s.hist;
    p.hist_stride = s.hist_stride;
    p.n_hist = s.n_hist;
    p.pick_idx = s.picks;
    p.tok = s.tok;
    p.temperature = o.temperature;
    p.top_k = o.top_k;
    p.top_p = o.top_p;
    p.penalty = o.repetition_penalty;
    p.greedy = o.greedy;
    p.uniforms = dev_uniforms;
    p.u_stride = u_stride;
    p.seed_lo = static_cast<unsigned>(seed & 0xFFFFFFFFu);
    p.seed_hi = static_cast<unsigned>(seed >> 32);
    p.work_stride = s.work_stride;
    p.sort_cap = kPickWorkFloats;
    if (s.pick_row_in_lds) {
        hipLaunchKernelGGL(pick_kernel<true>, dim3(s.B), dim3(kPickThreads),
                           static_cast<size_t>(p.V + kPickWorkFloats) * sizeof(float), s.stream, p);
    } else {
        hipLaunchKernelGGL(pick_kernel<false>, dim3(s.B), dim3(kPickThreads), kPickWorkFloats * sizeof(float),
                           s.stream, p);
    }
    HIP_CHECK(hipGetLastError());
    if (commit) s.n_hist++;
    s.picks++;
}

static void check_sampling(const gh_sampling& o) {
    if (!o.greedy && !(o.temperature > 0.0f))
        throw ApiError{GH_ERR_INVALID_ARGUMENT, "temperature must be positive"};
    if (!(o.repetition_penalty > 0.0f))
        throw ApiError{GH_ERR_INVALID_ARGUMENT, "repetition_penalty must be positive"};
}

// ---- prompt pass: every prompt token of every sequence through each layer at once

constexpr int kPromptPassMin = 8;         // shorter prompts go token by token
constexpr size_t kPromptPassRows = 32768; // rows per pass; longer prompts run in slices

static bool prompt_pass_ok(const Session& s, int len) {
    const Shape& sh = s.m->shape;
    return len >= kPromptPassMin && sh.head_size() == 64 && sh.d_model % 128 == 0 && sh.d_ff() % 128 == 0;
}

// One projection over M rows (norm folded in for RMSNorm, a norm kernel for LayerNorm).
// Long row blocks take the compute-bound 128 x 128 tiling, short ones the
// latency-bound small tiles.
template <int EPI, bool RMS>
static void launch_rows_gemm(const GemvParams& g, int M, hipStream_t st) {
    if (gemm128_ok(g, M)) {
        // per instantiation, once: the tile needs more than the default 64 KB of LDS
        static std::once_flag lds_raised;
        std::call_once(lds_raised, [] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm128_kernel<EPI, RMS>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          static_cast<int>(kBigLdsBytes)));
        });
        launch_gemm128<EPI, RMS>(g, M, st);
    } else {
        launch_gemm16<EPI, RMS>(g, M, st);
    }
}

template <int PRO, int EPI>
static void project_rows(Session& s, GemvParams g, int M) {
    hipStream_t st = s.stream;
    if (PRO == PRO_RMSNORM) {
        launch_rows_gemm<EPI, true>(g, M, st);
    } else {
        if (PRO == PRO_LAYERNORM) {
            hipLaunchKernelGGL(norm_rows_kernel, dim3((M + 3) / 4), dim3(256), 0, st, g.in, g.gamma, g.beta,
                               s.pp_norm, M, g.K, static_cast<int>(PRO));
            HIP_CHECK(hipGetLastError());
            g.in = s.pp_norm;
            g.in_stride = g.K;
        }
        launch_rows_gemm<EPI, false>(g, M, st);
    }
    HIP_CHECK(hipGetLastError());
}

// Where a scored pass leaves its result: targets and nll are device arrays
// [batch][len] indexed like the ids of the pass.
struct ScoreSink {
    const int* targets;
    float* nll;
};

// Final norm, logits and the target's negative log-likelihood for rows
// pp_x[0 .. M) of a slice (row m = seq * n + t, position t0 + t), a block of rows
// at a time so that the logits of a block stay a modest buffer.
static void score_rows(Session& s, const ScoreSink& sink, int M, int n, int t0, int len) {
    const Model& m = *s.m;
    const Shape& sh = m.shape;
    const size_t V = sh.vocab;
    const size_t want = std::min<size_t>(static_cast<size_t>(M),
                                         std::max<size_t>(128, ((size_t{64} << 20) / V) / 128 * 128));
    if (s.score_rows < want) {
        if (s.score_logits) HIP_CHECK(hipFree(s.score_logits));
        s.score_logits = nullptr;
        dev_alloc(s.score_logits, want * V);
        s.score_rows = want;
    }
    for (int r0 = 0; r0 < M; r0 += static_cast<int>(s.score_rows)) {
        const int rows = std::min<int>(static_cast<int>(s.score_rows), M - r0);
        GemvParams g{};
        g.W = m.E;
        g.N = sh.vocab;
        g.K = sh.d_model;
        g.in = s.pp_x + static_cast<size_t>(r0) * sh.d_model;
        g.in_stride = sh.d_model;
        g.gamma = m.gf;
        g.beta = m.bf;
        g.out = s.score_logits;
        g.out_stride = sh.vocab;
        if (sh.modern()) project_rows<PRO_RMSNORM, EPI_STORE>(s, g, rows);
        else project_rows<PRO_LAYERNORM, EPI_STORE>(s, g, rows);
        hipLaunchKernelGGL(nll_rows_kernel, dim3(rows), dim3(256), 0, s.stream, s.score_logits, sh.vocab, r0, n, t0,
                           len, sink.targets, sink.nll);
        HIP_CHECK(hipGetLastError());
    }
}

// Tokens hist[n_hist .. n_hist + len) of every sequence, positions pos .. pos + len.
// Equivalent to len step() calls (text_gen.cpp:44-46); only the last logits are
// formed unless a sink asks for the likelihood of a target at every position.
static void prompt_pass(Session& s, int len, const ScoreSink* sink = nullptr) {
    const Model& m = *s.m;
    const Shape& sh = m.shape;
    const int d = sh.d_model, F = sh.d_ff(), B = s.B;
    const bool modern = sh.modern();
    hipStream_t st = s.stream;
    const int slice = static_cast<int>(std::max<size_t>(1, std::min<size_t>(len, kPromptPassRows / B)));
    const size_t rows_cap = static_cast<size_t>(slice) * B;
    if (s.pp_rows < rows_cap) {
        for (float** b : {&s.pp_x, &s.pp_q, &s.pp_attn, &s.pp_norm, &s.pp_hidden}) {
            if (*b) HIP_CHECK(hipFree(*b));
            *b = nullptr;
        }
        dev_alloc(s.pp_x, rows_cap * d);
        dev_alloc(s.pp_q, rows_cap * d);
        dev_alloc(s.pp_attn, rows_cap * d);
        dev_alloc(s.pp_norm, rows_cap * d);
        dev_alloc(s.pp_hidden, rows_cap * F);
        s.pp_rows = rows_cap;
    }
    for (int t0 = 0; t0 < len; t0 += slice) {
        const int n = std::min(slice, len - t0);
        const int M = n * B;
        const int pos_base = s.pos + t0;
        hipLaunchKernelGGL(embed_rows_kernel, dim3((d + 255) / 256, M), dim3(256), 0, st, m.E, m.P, s.hist,
                           s.hist_stride, s.n_hist + t0, n, pos_base, s.pp_x, d);
        HIP_CHECK(hipGetLastError());
        for (int l = 0; l < sh.layers; l++) {
            const LayerWeights& w = m.layers[l];
            GemvParams g{};
            g.kv = kv_layout(s);
            g.layer = l;
            g.d_model = d;
            g.st = s.st;
            g.rows_per_seq = n;
            g.pos_base = pos_base;
            g.W = w.wqkv;
            g.bias = w.bqkv;
            g.N = 3 * d;
            g.K = d;
            g.in = s.pp_x;
            g.in_stride = d;
            g.gamma = w.g1;
            g.beta = w.be1;
            g.out = s.pp_q;
            g.out_stride = d;
            g.rope = modern;
            g.rope_cos = m.rope_cos;
            g.rope_sin = m.rope_sin;
            if (modern) project_rows<PRO_RMSNORM, EPI_QKV>(s, g, M);
            else project_rows<PRO_LAYERNORM, EPI_QKV>(s, g, M);

            PrefillAttnParams a{};
            a.q = s.pp_q;
            a.out = s.pp_attn;
            a.kv = g.kv;
            a.layer = l;
            a.d_model = d;
            a.len = n;
            a.pos_base = pos_base;
            a.scale = 1.0f / std::sqrt(static_cast<float>(sh.head_size()));
            // from 512 tokens on, 128 queries per workgroup (16 sequences: 1000 tokens 512 against
            // 585 us, 1536 tokens 860 against 977; at 300 tokens 76 against 60: too few workgroups)
            if (n >= 512)
                hipLaunchKernelGGL(attn_prefill128_kernel, dim3((n + 127) / 128, sh.heads, B), dim3(256), 0, st, a);
            else
                hipLaunchKernelGGL(attn_prefill64_kernel, dim3((n + 63) / 64, sh.heads, B), dim3(256), 0, st, a);
            HIP_CHECK(hipGetLastError());

            g.W = w.wo;
            g.bias = w.bo;
            g.N = d;
            g.K = d;
            g.in = s.pp_attn;
            g.in_stride = d;
            g.out = s.pp_x;
            g.out_stride = d;
            project_rows<PRO_PLAIN, EPI_RESID>(s, g, M);

            g.in = s.pp_x;
            g.in_stride = d;
            g.gamma = w.g2;
            g.beta = w.be2;
            g.out = s.pp_hidden;
            g.out_stride = F;
            g.W = w.w1;
            g.K = d;
            if (modern) {
                g.bias = nullptr;
                g.N = 2 * F;
                project_rows<PRO_RMSNORM, EPI_SWIGLU>(s, g, M);
            } else {
                g.bias = w.b1;
                g.N = F;
                project_rows<PRO_LAYERNORM, EPI_GELU>(s, g, M);
            }
            g.W = w.w2;
            g.bias = modern ? nullptr : w.b2;
            g.N = d;
            g.K = F;
            g.in = s.pp_hidden;
            g.in_stride = F;
            g.out = s.pp_x;
            g.out_stride = d;
            project_rows<PRO_PLAIN, EPI_RESID>(s, g, M);
        }
        if (sink) score_rows(s, *sink, M, n, t0, len);
        if (t0 + n == len) {
            hipLaunchKernelGGL(take_last_rows_kernel, dim3((d + 255) / 256, B), dim3(256), 0, st, s.pp_x, n,
                               s.x, d);
            HIP_CHECK(hipGetLastError());
        }
    }
    s.pos += len;
    s.n_hist += len;
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, st, s.st, s.pos, s.n_hist, s.picks);
    HIP_CHECK(hipGetLastError());
    // logits of the last position, through the decode-size projection
    enqueue_logits(s, /*advance=*/false);
}

// Steps through `len` tokens already staged in the history at n_hist.. (the
// prompt loop of text_gen.cpp:44-46).  log: per-step logits destination or null.
static void run_prompt(Session& s, int len, float* log, size_t* steps_logged) {
    const size_t BV = static_cast<size_t>(s.B) * s.m->shape.vocab;
    if (!log && s.use_prompt_pass && prompt_pass_ok(s, len)) {
        prompt_pass(s, len);
        if (steps_logged) *steps_logged += len;
        return;
    }
    if (s.engine == GH_ENGINE_PERSISTENT) {
        persist_run(s, len, len, 0, false, nullptr, nullptr, 0, 0,
                    log ? log + *steps_logged * BV : nullptr);
        if (steps_logged) *steps_logged += len;
        return;
    }
    const int base = s.n_hist;
    for (int t = 0; t < len; t++) {
        hipLaunchKernelGGL(load_tok_kernel, dim3((s.B + 63) / 64), dim3(64), 0, s.stream, s.hist,
                           s.hist_stride, base + t, s.tok, s.B);
        HIP_CHECK(hipGetLastError());
        run_step(s);
        if (log) {
            HIP_CHECK(hipMemcpyAsync(log + *steps_logged * BV, s.logits, BV * sizeof(float),
                                     hipMemcpyDeviceToDevice, s.stream));
        }
        if (steps_logged) (*steps_logged)++;
    }
    s.n_hist += len;
}

// The decode loop of text_gen.cpp:48-64 from the current context: pick, push,
// stop at capacity, else step.  Returns {picks made, steps run}.
static std::pair<int, int> run_decode(Session& s, int max_tokens, const gh_sampling& o,
                                      const float* du, int u_stride, uint64_t seed, float* log,
                                      size_t* steps_logged) {
    const int C = s.m->shape.max_len;
    const size_t BV = static_cast<size_t>(s.B) * s.m->shape.vocab;
    if (s.engine == GH_ENGINE_PERSISTENT) {
        int picks = 0, steps = 0, pos = s.pos, nh = s.n_hist;
        for (int i = 0; i < max_tokens; i++) {
            if (nh >= s.hist_stride) break;
            picks++;
            nh++;
            if (pos >= C) break;
            steps++;
            pos++;
        }
        persist_run(s, 0, steps, picks, true, &o, du, u_stride, seed,
                    log ? log + *steps_logged * BV : nullptr);
        if (steps_logged) *steps_logged += steps;
        return {picks, steps};
    }
    // Greedy without a penalty on the matrix-core path: after the first step of the call
    // the pick rides at the head of the next step (the logits launch left what it needs).
    const bool pick_rides = s.best && o.greedy && o.repetition_penalty == 1.0f;
    if (pick_rides) {
        hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, s.stream, s.st, s.pos, s.n_hist, s.picks);
        HIP_CHECK(hipGetLastError());
    }
    int picks = 0, steps = 0;
    for (int i = 0; i < max_tokens; i++) {
        if (s.n_hist >= s.hist_stride) break;
        const bool riding = pick_rides && steps > 0 && s.pos < C;
        if (riding) {
            s.n_hist++;
            s.picks++;
        } else {
            launch_pick(s, o, du, u_stride, seed, true);
        }
        picks++;
        if (s.pos >= C) break;
        run_step(s, riding);
        steps++;
        if (log) {
            HIP_CHECK(hipMemcpyAsync(log + *steps_logged * BV, s.logits, BV * sizeof(float),
                                     hipMemcpyDeviceToDevice, s.stream));
        }
        if (steps_logged) (*steps_logged)++;
    }
    return {picks, steps};
}

// Copies the caller's uniforms to the device (grown on demand); null for none.
static const float* stage_uniforms(Session& s, const float* uniforms, size_t n) {
    if (!uniforms || n == 0) return nullptr;
    if (s.uniforms_cap < n) {
        if (s.uniforms) HIP_CHECK(hipFree(s.uniforms));
        s.uniforms = nullptr;
        dev_alloc(s.uniforms, n);
        s.uniforms_cap = n;
    }
    HIP_CHECK(hipMemcpyAsync(s.uniforms, uniforms, n * sizeof(float), hipMemcpyHostToDevice, s.stream));
    return s.uniforms;
}

// ---- a pick that allocates nothing (gh_pick_noalloc)

// The sampler's working rows for callers that cannot allocate: one array per
// GPU, held until the process ends.  Host code never uses this name as an
// address; it asks the runtime where the array lives on the current device.
constexpr size_t kNoAllocScratchFloats = size_t{1} << 20;  // 4 MiB
static __device__ __align__(256) float scratch[kNoAllocScratchFloats];

__global__ __launch_bounds__(kPickThreads) void pick_noalloc_kernel(const PickParams p, int* out_ids) {
    extern __shared__ __attribute__((aligned(128))) float lds[];
    const int b = blockIdx.x;
    const int chosen = pick_body<false, kPickThreads>(p, b, p.work + static_cast<size_t>(b) * p.work_stride, lds);
    if (threadIdx.x == 0) out_ids[b] = chosen;
}

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current GPU, looked up once per device.
static float* scratch_on_current_device() {
    int dev = 0;
    HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) throw ApiError{GH_ERR_DEVICE, "device index beyond the scratch table"};
    std::lock_guard<std::mutex> lk(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* ptr = nullptr;
        HIP_CHECK(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
        if (!ptr) throw ApiError{GH_ERR_DEVICE, "the scratch array has no address on this device"};
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

// ---- matrix-core issue probe (gh_device_mfma_issue)

// Wavefronts 0-3 of a workgroup (one per SIMD) run a dependent chain of fp32 matrix
// products, wavefronts 4-7 (the same SIMDs) runs of VPER dependent-free multiply-adds,
// or wavefronts 0-3 both in turn; every wavefront reports its shader-clock cycles.
template <int VPER>
__global__ __launch_bounds__(512) void mfma_issue_probe_kernel(long long* out, int iters, int mode, float a, float b) {
    typedef float v16f __attribute__((ext_vector_type(16)));
    const int wave = threadIdx.x >> 6;
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; i++) x[i] = a + static_cast<float>(i);
    __syncthreads();
    const long long c0 = clock64(), w0 = wall_clock64();
    if (wave < 4) {
        if (mode & 1) {
            for (int i = 0; i < iters; i++) {
#pragma unroll
                for (int u = 0; u < 8; u++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
            }
        } else if (mode & 4) {
            for (int i = 0; i < iters; i++) {
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < VPER; v++) x[v & 7] = x[v & 7] * b + a;
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    } else if (mode & 2) {
        for (int i = 0; i < iters; i++) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
#pragma unroll
                for (int v = 0; v < VPER; v++) x[v & 7] = x[v & 7] * b + a;
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float keep = acc[0];
#pragma unroll
    for (int i = 0; i < 8; i++) keep += x[i];
    if ((threadIdx.x & 63) == 0) {
        long long* o = out + (static_cast<size_t>(blockIdx.x) * 8 + wave) * 3;
        o[0] = c1 - c0;
        o[1] = w1 - w0;
        o[2] = static_cast<long long>(keep);
    }
}

// ---- hand-off latency probe (gh_device_handoff_latency)

// Workgroup 0 and workgroup `peer` bounce a counter: each waits until the other's word
// has reached the round number and then writes its own.  LOAD: cache policy of the
// polling load (buffer aux bits); DEVICE_STORE: device-scope (write-through) store or
// an ordinary one.  Bounded polling: a side that never sees its peer gives up.
template <int LOAD, bool DEVICE_STORE>
__global__ void handoff_probe_kernel(unsigned* cells, int peer, int rounds, unsigned long long* ticks, unsigned* xcds) {
    const int me = blockIdx.x == 0 ? 0 : (static_cast<int>(blockIdx.x) == peer ? 1 : -1);
    if (threadIdx.x == 0) xcds[blockIdx.x] = xcc_id();
    if (me < 0 || threadIdx.x != 0) return;
    unsigned* mine = cells + me * 64;
    const __amdgpu_buffer_rsrc_t rs = make_buffer(cells + (1 - me) * 64, 4);
    auto put = [&](unsigned v) {
        if (DEVICE_STORE) __hip_atomic_store(mine, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else *reinterpret_cast<volatile unsigned*>(mine) = v;
    };
    const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
    for (int i = 1; i <= rounds; i++) {
        if (me == 0) put(static_cast<unsigned>(i));
        unsigned spins = 0;
        while (static_cast<unsigned>(__builtin_amdgcn_raw_buffer_load_b32(rs, 0, 0, LOAD)) < static_cast<unsigned>(i)
               && ++spins < (1u << 20)) {
        }
        if (me == 1) put(static_cast<unsigned>(i));
    }
    ticks[me] = __builtin_amdgcn_s_memrealtime() - t0;  // 100 MHz
}

// Background load for the probe: streams a buffer until told to stop (or 2000 rounds).
__global__ void handoff_probe_hog(const float4* buf, size_t n4, const volatile unsigned* stop, float* sink) {
    float acc = 0.0f;
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (int it = 0; it < 2000 && *stop == 0u; it++)
        for (int k = 0; k < 16; k++) {
            const float4 v = buf[i];
            acc += (v.x + v.y) + (v.z + v.w);
            i += stride;
            if (i >= n4) i -= n4;
        }
    if (acc == 1.2345f) *sink = acc;
}

using HandoffKernel = void (*)(unsigned*, int, int, unsigned long long*, unsigned*);
static HandoffKernel handoff_kernel_for(int load_policy, bool device_store) {
    switch (load_policy) {
    case 0: return device_store ? handoff_probe_kernel<0, true> : handoff_probe_kernel<0, false>;
    case 1: return device_store ? handoff_probe_kernel<kAuxNonTemporal, true> : handoff_probe_kernel<kAuxNonTemporal, false>;
    case 2: return device_store ? handoff_probe_kernel<kAuxDeviceScope, true> : handoff_probe_kernel<kAuxDeviceScope, false>;
    default: return nullptr;
    }
}

}  // namespace gh

// ====================================================================== C ABI

using namespace gh;

struct gh_model {
    std::unique_ptr<Model> impl;
};
struct gh_session {
    std::unique_ptr<Session> impl;
};

// A plain streaming read (eight 16-byte loads in flight per thread): what a
// bandwidth-bound kernel can reach on this device.
__global__ __launch_bounds__(256) void stream_read_kernel(const float4* __restrict__ a, size_t n4, float* sink) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    for (; i + 7 * stride < n4; i += 8 * stride) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = a[i + u * stride];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            acc.x += v[u].x;
            acc.y += v[u].y;
            acc.z += v[u].z;
            acc.w += v[u].w;
        }
    }
    for (; i < n4; i += stride) {  // what is left (all of a buffer below 256 MiB)
        const float4 v = a[i];
        acc.x += v.x;
        acc.y += v.y;
        acc.z += v.z;
        acc.w += v.w;
    }
    if (acc.x + acc.y + acc.z + acc.w == 12345.0f) *sink = 1.0f;  // keeps the loads alive
}

extern "C" {

const char* gh_last_error(void) { return g_last_error.c_str(); }

// ---- tokenizer (host only)

// Exactly one of the two is set.
struct gh_tokenizer {
    std::optional<gh::ByteBpe> v2;
    std::optional<gh::BpeV1> v1;
};

gh_status gh_tokenizer_load(const char* path, gh_tokenizer** out) {
    return guard([&] {
        if (!path || !out) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        *out = nullptr;
        // anything that does not start with "GTOK" is taken for a v1 cache (tokenizer.cpp:107-117)
        if (is_gtok_file(path)) *out = new gh_tokenizer{ByteBpe::load(path), std::nullopt};
        else *out = new gh_tokenizer{std::nullopt, BpeV1::load(path)};
    });
}

gh_status gh_tokenizer_from_merges(const int32_t* merges, int32_t n_merges, const char* const* specials,
                                   const int32_t* special_lens, int32_t n_specials, gh_tokenizer** out) {
    return guard([&] {
        if (!out || n_merges < 0 || n_specials < 0 || (n_merges > 0 && !merges)
            || (n_specials > 0 && (!specials || !special_lens)))
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        *out = nullptr;
        std::vector<ByteBpe::Merge> m;
        m.reserve(static_cast<size_t>(n_merges));
        for (int32_t r = 0; r < n_merges; r++) m.emplace_back(merges[2 * r], merges[2 * r + 1]);
        std::vector<std::string> sp;
        for (int32_t i = 0; i < n_specials; i++)
            sp.emplace_back(specials[i], static_cast<size_t>(std::max(special_lens[i], 0)));
        *out = new gh_tokenizer{ByteBpe(std::move(m), std::move(sp)), std::nullopt};
    });
}

gh_status gh_tokenizer_save(const gh_tokenizer* t, const char* path) {
    return guard([&] {
        if (!t || !path) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        if (t->v2) t->v2->save(path);
        else t->v1->save(path);
    });
}

void gh_tokenizer_free(gh_tokenizer* t) { delete t; }

gh_status gh_tokenizer_get_info(const gh_tokenizer* t, gh_tokenizer_info* out) {
    return guard([&] {
        if (!t || !out) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        if (t->v2) {
            out->kind = ByteBpe::kKind;
            out->vocab_size = t->v2->vocab_size();
            out->eos_id = t->v2->special_id("<|endoftext|>");  // byte_bpe.h:78
            out->n_merges = static_cast<int32_t>(t->v2->merges().size());
            out->n_specials = static_cast<int32_t>(t->v2->specials().size());
            out->fingerprint = t->v2->fingerprint();
        } else {
            out->kind = BpeV1::kKind;
            out->vocab_size = t->v1->vocab_size();
            out->eos_id = t->v1->special_id("<eos>");  // tokenizer.cpp:95-97
            out->n_merges = static_cast<int32_t>(t->v1->merge_count());
            out->n_specials = 0;
            for (const char* sp : {"<pad>", "<eos>", "<unk>"}) out->n_specials += t->v1->special_id(sp) >= 0;
            out->fingerprint = t->v1->fingerprint();
        }
    });
}

gh_status gh_tokenizer_special_id(const gh_tokenizer* t, const char* token, size_t len, int32_t* id) {
    return guard([&] {
        if (!t || !id || (len > 0 && !token)) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        const std::string_view tv(token, len);
        *id = t->v2 ? t->v2->special_id(tv) : t->v1->special_id(tv);
    });
}

gh_status gh_tokenizer_encode(const gh_tokenizer* t, const char* text, size_t len, int32_t with_specials,
                              int32_t* ids, size_t cap, size_t* n) {
    return guard([&] {
        if (!t || !n || (len > 0 && !text) || (cap > 0 && !ids))
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        const std::string_view tv(text, len);
        const std::vector<int> got = t->v2 ? t->v2->encode(tv, with_specials != 0) : t->v1->encode(tv);
        *n = got.size();
        std::copy_n(got.begin(), std::min(cap, got.size()), ids);
    });
}

gh_status gh_tokenizer_decode(const gh_tokenizer* t, const int32_t* ids, size_t n, char* out, size_t cap,
                              size_t* len) {
    return guard([&] {
        if (!t || !len || (n > 0 && !ids) || (cap > 0 && !out))
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        const std::string got = t->v2 ? t->v2->decode(ids, n) : t->v1->decode(ids, n);
        *len = got.size();
        std::copy_n(got.begin(), std::min(cap, got.size()), out);
    });
}

gh_status gh_pretokenize(const char* text, size_t len, size_t* ends, size_t cap, size_t* n) {
    return guard([&] {
        if (!n || (len > 0 && !text) || (cap > 0 && !ends)) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        const std::string_view v(text, len);
        size_t pieces = 0;
        for (size_t pos = 0; pos < len;) {
            pos = pretok::piece_end(v, pos);
            if (pieces < cap) ends[pieces] = pos;
            pieces++;
        }
        *n = pieces;
    });
}

int32_t gh_codepoint_class(uint32_t codepoint) { return pretok::classify(codepoint); }

static Shape shape_of(const gh_config& c) {
    Shape s;
    s.arch = c.arch;
    s.vocab = c.vocab;
    s.d_model = c.d_model;
    s.layers = c.layers;
    s.heads = c.heads;
    s.max_len = c.max_len;
    s.dropout = c.dropout;
    return s;
}

static void check_config(const gh_config* cfg) {
    if (!cfg) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null config"};
    if (cfg->arch != GH_ARCH_GPT2 && cfg->arch != GH_ARCH_MODERN)
        throw ApiError{GH_ERR_RUNTIME, "unknown architecture tag " + std::to_string(cfg->arch)};
    validate_shape(shape_of(*cfg));
}

gh_status gh_model_load(const char* path, gh_model** out) {
    return guard([&] {
        if (!path || !out) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        *out = nullptr;
        HostModel hm = read_checkpoint(path);
        std::vector<const float*> ptrs;
        for (const auto& t : hm.tensors) ptrs.push_back(t.data());
        try {
            auto m = upload_model(hm.shape, ptrs, hm.tokenizer);
            *out = new gh_model{std::move(m)};
        } catch (const ApiError& e) {
            throw ApiError{e.code, std::string("Failed to load model from ") + path + ": " + e.msg};
        }
    });
}

gh_status gh_model_from_host(const gh_config* cfg, const float* const* tensors, int32_t n_tensors,
                             gh_model** out) {
    return guard([&] {
        if (!tensors || !out) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        *out = nullptr;
        check_config(cfg);
        const Shape s = shape_of(*cfg);
        if (static_cast<size_t>(n_tensors) != tensor_specs(s).size())
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "tensor count does not match the model shape"};
        std::vector<const float*> ptrs(tensors, tensors + n_tensors);
        for (const float* p : ptrs)
            if (!p) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null tensor"};
        std::optional<Fingerprint> fp;
        if (cfg->has_fingerprint) fp = Fingerprint{cfg->tokenizer_kind, cfg->tokenizer_hash};
        *out = new gh_model{upload_model(s, ptrs, fp)};
    });
}

int32_t gh_config_num_tensors(const gh_config* cfg) {
    int32_t n = -1;
    (void)guard([&] {
        check_config(cfg);
        n = static_cast<int32_t>(tensor_specs(shape_of(*cfg)).size());
    });
    return n;
}

gh_status gh_config_tensor_shape(const gh_config* cfg, int32_t index, int32_t* rows, int32_t* cols) {
    return guard([&] {
        check_config(cfg);
        const auto specs = tensor_specs(shape_of(*cfg));
        if (index < 0 || static_cast<size_t>(index) >= specs.size())
            throw ApiError{GH_ERR_OUT_OF_RANGE, "tensor index out of range"};
        if (rows) *rows = specs[index].rows;
        if (cols) *cols = specs[index].cols;
    });
}

gh_status gh_model_save(const gh_model* m, const char* path) {
    return guard([&] {
        if (!m || !path) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        const auto host = download_model(*m->impl);
        std::vector<const float*> ptrs;
        for (const auto& t : host) ptrs.push_back(t.data());
        std::string why;
        if (!write_checkpoint(path, m->impl->shape, ptrs, m->impl->tokenizer, why))
            throw ApiError{GH_ERR_RUNTIME, why};
    });
}

void gh_model_free(gh_model* m) { delete m; }

gh_status gh_model_get_config(const gh_model* m, gh_config* out) {
    return guard([&] {
        if (!m || !out) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        const Shape& s = m->impl->shape;
        *out = gh_config{};
        out->arch = s.arch;
        out->vocab = s.vocab;
        out->d_model = s.d_model;
        out->layers = s.layers;
        out->heads = s.heads;
        out->max_len = s.max_len;
        out->d_ff = s.d_ff();
        out->dropout = s.dropout;
        if (m->impl->tokenizer) {
            out->has_fingerprint = 1;
            out->tokenizer_kind = m->impl->tokenizer->kind;
            out->tokenizer_hash = m->impl->tokenizer->hash;
        }
    });
}

gh_status gh_session_create(const gh_model* m, const gh_session_opts* opts, gh_session** out) {
    return guard([&] {
        if (!m || !out) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        *out = nullptr;
        gh_session_opts o{};
        o.batch = 1;
        if (opts) o = *opts;
        *out = new gh_session{create_session(*m->impl, o)};
    });
}

void gh_session_free(gh_session* s) { delete s; }

gh_status gh_session_reset(gh_session* s) {
    return guard([&] {
        if (!s) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null session"};
        reset_session(*s->impl);
        HIP_CHECK(hipStreamSynchronize(s->impl->stream));
    });
}

gh_status gh_session_step(gh_session* sess, const int32_t* ids, float* logits_host) {
    return guard([&] {
        if (!sess || !ids) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        const PersistGate gate(s);  // held until this call has synchronised its launches
        check_capacity(s);
        check_ids(s, ids, s.B);
        const size_t V = s.m->shape.vocab;
        const bool one_launch = s.engine == GH_ENGINE_PERSISTENT && s.n_hist == s.pos;
        if (one_launch) {
            // One launch, one copy back and one wait per call: the token travels in the
            // kernel's arguments (the kernel records it in the history, whose index is the
            // position), and the kernel's "gave up" word comes back with the logits.
            persist_run(s, 1, 1, 0, false, nullptr, nullptr, 0, 0, nullptr, false, -1, ids[0]);
            HIP_CHECK(hipMemcpyAsync(s.host_err, &s.ctl->abort, sizeof(int), hipMemcpyDeviceToHost, s.stream));
        } else {
            std::memcpy(s.host_ids, ids, s.B * sizeof(int));
            HIP_CHECK(hipMemcpyAsync(s.tok, s.host_ids, s.B * sizeof(int), hipMemcpyHostToDevice,
                                     s.stream));
            // The history (index == position) feeds the repetition penalty of later picks.
            hipLaunchKernelGGL(store_hist_kernel, dim3((s.B + 63) / 64), dim3(64), 0, s.stream, s.hist,
                               s.hist_stride, s.n_hist, s.tok, s.B);
            HIP_CHECK(hipGetLastError());
            if (s.engine == GH_ENGINE_PERSISTENT) {
                persist_run(s, 1, 1, 0, false, nullptr, nullptr, 0, 0, nullptr);
            } else {
                s.n_hist++;
                run_step(s);
            }
        }
        HIP_CHECK(hipMemcpyAsync(s.host_logits, s.logits, s.B * V * sizeof(float),
                                 hipMemcpyDeviceToHost, s.stream));
        HIP_CHECK(hipStreamSynchronize(s.stream));
        // (the word read back with the logits says whether the kernel finished its waits)
        if (!one_launch || *s.host_err != 0) check_persist_abort(s);
        if (logits_host) std::memcpy(logits_host, s.host_logits, s.B * V * sizeof(float));
    });
}

gh_status gh_session_logits(gh_session* s, const float** logits) {
    return guard([&] {
        if (!s || !logits) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        *logits = s->impl->host_logits;
    });
}

gh_status gh_session_prefill(gh_session* sess, const int32_t* ids, int32_t len,
                             float* last_logits_host) {
    return guard([&] {
        if (!sess || !ids) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        const PersistGate gate(s);  // held until this call has synchronised its launches
        if (len < 0) throw ApiError{GH_ERR_INVALID_ARGUMENT, "negative length"};
        if (len == 0) return;
        if (s.pos + len > s.m->shape.max_len)
            throw ApiError{GH_ERR_RUNTIME, "InferenceSession: context exceeds max_len"};
        check_ids(s, ids, static_cast<size_t>(s.B) * len);
        const size_t V = s.m->shape.vocab;
        // Stage the ids into the history, then step through them.
        const int base = s.n_hist;
        for (int b = 0; b < s.B; b++) {
            std::memcpy(s.host_ids + static_cast<size_t>(b) * s.hist_stride,
                        ids + static_cast<size_t>(b) * len, len * sizeof(int));
            HIP_CHECK(hipMemcpyAsync(s.hist + static_cast<size_t>(b) * s.hist_stride + base,
                                     s.host_ids + static_cast<size_t>(b) * s.hist_stride,
                                     len * sizeof(int), hipMemcpyHostToDevice, s.stream));
        }
        run_prompt(s, len, nullptr, nullptr);
        HIP_CHECK(hipMemcpyAsync(s.host_logits, s.logits, s.B * V * sizeof(float),
                                 hipMemcpyDeviceToHost, s.stream));
        HIP_CHECK(hipStreamSynchronize(s.stream));
        check_persist_abort(s);
        if (last_logits_host) std::memcpy(last_logits_host, s.host_logits, s.B * V * sizeof(float));
    });
}

gh_status gh_session_score(gh_session* sess, const int32_t* ids, const int32_t* targets, int32_t len,
                           float* nll_host) {
    return guard([&] {
        if (!sess || !ids || !targets || !nll_host) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        const PersistGate gate(s);  // held until this call has synchronised its launches
        if (len < 0) throw ApiError{GH_ERR_INVALID_ARGUMENT, "negative length"};
        if (len == 0) return;
        if (s.pos + len > s.m->shape.max_len)
            throw ApiError{GH_ERR_RUNTIME, "InferenceSession: context exceeds max_len"};
        const size_t n = static_cast<size_t>(s.B) * len;
        check_ids(s, ids, n);
        check_ids(s, targets, n);
        const int base = s.n_hist;
        for (int b = 0; b < s.B; b++) {
            std::memcpy(s.host_ids + static_cast<size_t>(b) * s.hist_stride,
                        ids + static_cast<size_t>(b) * len, len * sizeof(int));
            HIP_CHECK(hipMemcpyAsync(s.hist + static_cast<size_t>(b) * s.hist_stride + base,
                                     s.host_ids + static_cast<size_t>(b) * s.hist_stride,
                                     len * sizeof(int), hipMemcpyHostToDevice, s.stream));
        }
        // targets and results live for this call only
        struct Scratch {
            int* targets = nullptr;
            float* nll = nullptr;
            ~Scratch() {
                if (targets) (void)hipFree(targets);
                if (nll) (void)hipFree(nll);
            }
        } tmp;
        dev_alloc(tmp.targets, n);
        dev_alloc(tmp.nll, n);
        HIP_CHECK(hipMemcpyAsync(tmp.targets, targets, n * sizeof(int), hipMemcpyHostToDevice, s.stream));
        const ScoreSink sink{tmp.targets, tmp.nll};
        if (s.use_prompt_pass && prompt_pass_ok(s, len)) {
            prompt_pass(s, len, &sink);
        } else {
            // token by token: every step leaves the logits of its position
            const int V = s.m->shape.vocab;
            for (int t = 0; t < len; t++) {
                if (s.engine == GH_ENGINE_PERSISTENT) {
                    persist_run(s, 1, 1, 0, false, nullptr, nullptr, 0, 0, nullptr);  // token from the history
                } else {
                    hipLaunchKernelGGL(load_tok_kernel, dim3((s.B + 63) / 64), dim3(64), 0, s.stream, s.hist,
                                       s.hist_stride, base + t, s.tok, s.B);
                    HIP_CHECK(hipGetLastError());
                    run_step(s);
                }
                hipLaunchKernelGGL(nll_rows_kernel, dim3(s.B), dim3(256), 0, s.stream, s.logits, V, 0, 1, t, len,
                                   sink.targets, sink.nll);
                HIP_CHECK(hipGetLastError());
            }
            if (s.engine != GH_ENGINE_PERSISTENT) s.n_hist += len;
        }
        HIP_CHECK(hipMemcpyAsync(nll_host, tmp.nll, n * sizeof(float), hipMemcpyDeviceToHost, s.stream));
        HIP_CHECK(hipStreamSynchronize(s.stream));
        check_persist_abort(s);
    });
}

int32_t gh_session_position(const gh_session* s) { return s ? s->impl->pos : -1; }
int32_t gh_session_capacity(const gh_session* s) { return s ? s->impl->m->shape.max_len : -1; }
int32_t gh_session_vocab(const gh_session* s) { return s ? s->impl->m->shape.vocab : -1; }
int32_t gh_session_batch(const gh_session* s) { return s ? s->impl->B : -1; }

gh_status gh_session_read_kv(gh_session* sess, int32_t seq, int32_t layer, int32_t kv, int32_t pos,
                             float* out_host) {
    return guard([&] {
        if (!sess || !out_host) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        const Shape& sh = s.m->shape;
        if (seq < 0 || seq >= s.B || layer < 0 || layer >= sh.layers || kv < 0 || kv > 1 || pos < 0
            || pos >= s.pos)
            throw ApiError{GH_ERR_OUT_OF_RANGE, "cache row out of range"};
        HIP_CHECK(hipStreamSynchronize(s.stream));
        std::vector<int> table(static_cast<size_t>(s.n_pages));
        HIP_CHECK(hipMemcpy(table.data(), s.page_table, table.size() * sizeof(int),
                            hipMemcpyDeviceToHost));
        const int hs = sh.head_size();
        const int page = table[static_cast<size_t>(seq) * s.pages_per_seq + (pos >> s.page_shift)];
        const int slot = pos & ((1 << s.page_shift) - 1);
        for (int h = 0; h < sh.heads; h++) {
            const size_t run = ((static_cast<size_t>(layer) * s.n_pages + page) * 2 + kv) * sh.heads + h;
            const size_t off = ((run << s.page_shift) + slot) * hs;
            HIP_CHECK(hipMemcpy(out_host + static_cast<size_t>(h) * hs, s.kv_pool + off,
                                hs * sizeof(float), hipMemcpyDeviceToHost));
        }
    });
}

gh_status gh_session_pick(gh_session* sess, const gh_sampling* opt, const float* uniforms,
                          uint64_t seed, int32_t* out_ids) {
    return guard([&] {
        if (!sess || !opt) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        check_sampling(*opt);
        if (s.pos == 0) throw ApiError{GH_ERR_RUNTIME, "no logits yet: step or prefill first"};
        if (s.n_hist >= s.hist_stride)
            throw ApiError{GH_ERR_RUNTIME, "token history is full"};
        const float* du = nullptr;
        if (uniforms) {
            if (s.uniforms_cap < static_cast<size_t>(s.B)) {
                if (s.uniforms) HIP_CHECK(hipFree(s.uniforms));
                s.uniforms = nullptr;
                dev_alloc(s.uniforms, s.B);
                s.uniforms_cap = s.B;
            }
            HIP_CHECK(hipMemcpyAsync(s.uniforms, uniforms, s.B * sizeof(float),
                                     hipMemcpyHostToDevice, s.stream));
            du = s.uniforms;
        }
        // The draw index is folded into the pointer: one uniform per sequence here.
        const int saved = s.picks;
        if (du) s.picks = 0;
        launch_pick(s, *opt, du, 1, seed, false);  // the stand-alone pick kernel serves every engine
        if (du) s.picks = saved + 1;
        HIP_CHECK(hipMemcpyAsync(s.host_ids, s.tok, s.B * sizeof(int), hipMemcpyDeviceToHost,
                                 s.stream));
        HIP_CHECK(hipStreamSynchronize(s.stream));
        if (out_ids) std::memcpy(out_ids, s.host_ids, s.B * sizeof(int));
    });
}

gh_status gh_session_decode(gh_session* sess, int32_t max_tokens, const gh_sampling* opt,
                            const float* uniforms, uint64_t seed, int32_t* out_ids,
                            int32_t* out_count) {
    return guard([&] {
        if (!sess || !opt || !out_count) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        const PersistGate gate(s);  // held until this call has synchronised its launches
        check_sampling(*opt);
        *out_count = 0;
        s.timing = gh_timing{};
        s.timing.launches_per_step = s.launches_per_step;
        if (max_tokens <= 0) return;
        if (s.pos == 0) throw ApiError{GH_ERR_RUNTIME, "no logits yet: step or prefill first"};
        const size_t B = s.B;
        const float* du = opt->greedy ? nullptr : stage_uniforms(s, uniforms, B * max_tokens);
        const int first = s.n_hist;
        const int saved_picks = s.picks;
        if (du) s.picks = 0;  // uniforms are indexed from this call's first pick
        HIP_CHECK(hipEventRecord(s.ev[1], s.stream));
        const auto [made, stepped] = run_decode(s, max_tokens, *opt, du, max_tokens, seed, nullptr, nullptr);
        HIP_CHECK(hipEventRecord(s.ev[2], s.stream));
        if (du) s.picks = saved_picks + made;
        for (size_t b = 0; b < B; b++)
            HIP_CHECK(hipMemcpyAsync(s.host_ids + b * s.hist_stride,
                                     s.hist + b * s.hist_stride + first, made * sizeof(int),
                                     hipMemcpyDeviceToHost, s.stream));
        HIP_CHECK(hipStreamSynchronize(s.stream));
        check_persist_abort(s);
        if (out_ids)
            for (size_t b = 0; b < B; b++)
                std::memcpy(out_ids + b * max_tokens, s.host_ids + b * s.hist_stride,
                            made * sizeof(int));
        *out_count = made;
        HIP_CHECK(hipEventElapsedTime(&s.timing.decode_ms, s.ev[1], s.ev[2]));
        s.timing.decode_steps = stepped;
    });
}

gh_status gh_session_decode_stream(gh_session* sess, int32_t max_tokens, const gh_sampling* opt,
                                   const float* uniforms, uint64_t seed, int32_t stop_token,
                                   gh_token_callback on_tokens, void* user, int32_t* out_ids,
                                   int32_t* out_count) {
    return guard([&] {
        if (!sess || !opt || !out_count || !on_tokens) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        const PersistGate gate(s);  // held until this call has synchronised its launches
        check_sampling(*opt);
        *out_count = 0;
        s.timing = gh_timing{};
        s.timing.launches_per_step = s.launches_per_step;
        if (max_tokens <= 0) return;
        if (s.pos == 0) throw ApiError{GH_ERR_RUNTIME, "no logits yet: step or prefill first"};
        const int B = s.B, C = s.m->shape.max_len;
        const float* du = opt->greedy ? nullptr : stage_uniforms(s, uniforms, static_cast<size_t>(B) * max_tokens);
        const int saved_picks = s.picks;
        if (du) s.picks = 0;  // uniforms are indexed from this call's first pick
        int made = 0, stepped = 0;
        HIP_CHECK(hipEventRecord(s.ev[1], s.stream));
        if (s.engine == GH_ENGINE_PERSISTENT) {
            // One launch runs the whole loop; the kernel reports each pick in pinned
            // memory as it is made and this thread hands it on while the kernel goes on.
            int planned_picks = 0, planned_steps = 0, pos = s.pos, nh = s.n_hist;
            for (int i = 0; i < max_tokens; i++) {
                if (nh >= s.hist_stride) break;
                planned_picks++;
                nh++;
                if (pos >= C) break;
                planned_steps++;
                pos++;
            }
            __atomic_store_n(s.stop_word, 0u, __ATOMIC_RELEASE);
            const unsigned base = s.feed_base;
            persist_run(s, 0, planned_steps, planned_picks, true, opt, du, max_tokens, seed, nullptr, true,
                        stop_token);
            HIP_CHECK(hipEventRecord(s.ev[2], s.stream));
            bool kernel_done = false;
            unsigned idle = 0;
            // Whatever ends this loop (the callback, a HIP error), the kernel must have
            // stopped and the host's view must match the device's before control leaves.
            auto settle = [&] {
                stepped = std::min(made, planned_steps);
                s.pos -= planned_steps - stepped;
                s.arrive_total -= static_cast<unsigned>(planned_steps - stepped);
                s.n_hist -= planned_picks - made;
                s.picks -= planned_picks - made;
            };
            try {
                while (made < planned_picks) {
                    const unsigned long long w = __atomic_load_n(s.feed + made, __ATOMIC_ACQUIRE);
                    if (static_cast<unsigned>(w >> 32) == base + static_cast<unsigned>(made) + 1u) {
                        const int32_t tok = static_cast<int32_t>(static_cast<unsigned>(w));
                        if (tok < 0) break;  // the kernel saw the stop word before this pick
                        if (out_ids) out_ids[made] = tok;
                        made++;  // delivered (or thrown out of) below: the round counts either way
                        const int32_t asked = on_tokens(user, &tok, made - 1);
                        idle = 0;
                        if (asked != 0) __atomic_store_n(s.stop_word, 1u, __ATOMIC_RELEASE);
                        if (tok == stop_token) break;  // the kernel ends after this token's step
                        continue;
                    }
                    if (kernel_done) break;  // the launch is over and reported no further pick
                    if ((++idle & 255u) == 0u) {
                        const hipError_t q = hipStreamQuery(s.stream);
                        if (q == hipSuccess) kernel_done = true;  // read the feed once more, then leave
                        else if (q != hipErrorNotReady) HIP_CHECK(q);
                    }
                }
            } catch (...) {
                // stop the kernel at its next pick, wait for it, and take every round it
                // still completed into account before handing the error on
                __atomic_store_n(s.stop_word, 1u, __ATOMIC_RELEASE);
                (void)hipStreamSynchronize(s.stream);
                while (made < planned_picks) {
                    const unsigned long long w = __atomic_load_n(s.feed + made, __ATOMIC_ACQUIRE);
                    if (static_cast<unsigned>(w >> 32) != base + static_cast<unsigned>(made) + 1u
                        || static_cast<int32_t>(static_cast<unsigned>(w)) < 0)
                        break;
                    if (out_ids) out_ids[made] = static_cast<int32_t>(static_cast<unsigned>(w));
                    made++;
                }
                settle();
                if (du) s.picks = saved_picks + made;
                *out_count = made;
                throw;
            }
            HIP_CHECK(hipStreamSynchronize(s.stream));
            check_persist_abort(s);
            // persist_run advanced the host's view by the planned run: take back what was not run
            settle();
        } else {
            std::vector<char> seen(static_cast<size_t>(B), 0);
            int n_seen = 0;
            for (int i = 0; i < max_tokens; i++) {
                if (s.n_hist >= s.hist_stride) break;
                launch_pick(s, *opt, du, max_tokens, seed, true);
                HIP_CHECK(hipMemcpyAsync(s.host_ids, s.tok, B * sizeof(int), hipMemcpyDeviceToHost, s.stream));
                HIP_CHECK(hipStreamSynchronize(s.stream));
                if (out_ids)
                    for (int b = 0; b < B; b++) out_ids[static_cast<size_t>(b) * max_tokens + i] = s.host_ids[b];
                const int32_t asked = on_tokens(user, s.host_ids, i);
                made++;
                for (int b = 0; b < B; b++)
                    if (s.host_ids[b] == stop_token && !seen[b]) {
                        seen[b] = 1;
                        n_seen++;
                    }
                if (s.pos >= C) break;
                run_step(s);
                stepped++;
                if (asked != 0 || n_seen == B) break;
            }
            HIP_CHECK(hipEventRecord(s.ev[2], s.stream));
            HIP_CHECK(hipStreamSynchronize(s.stream));
        }
        if (du) s.picks = saved_picks + made;
        *out_count = made;
        HIP_CHECK(hipEventElapsedTime(&s.timing.decode_ms, s.ev[1], s.ev[2]));
        s.timing.decode_steps = stepped;
    });
}

gh_status gh_session_generate(gh_session* sess, const int32_t* prompts, int32_t prompt_len,
                              int32_t max_tokens, const gh_sampling* opt, const float* uniforms,
                              uint64_t seed, int32_t* out_tokens, int32_t* out_len,
                              float* step_logits_host, int32_t* n_steps) {
    return guard([&] {
        if (!sess || !opt || !out_tokens || !out_len)
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        Session& s = *sess->impl;
        const PersistGate gate(s);  // held until this call has synchronised its launches
        const Shape& sh = s.m->shape;
        check_sampling(*opt);
        *out_len = 0;
        if (n_steps) *n_steps = 0;
        s.timing = gh_timing{};
        s.timing.launches_per_step = s.launches_per_step;
        if (prompt_len <= 0) return;  // text_gen.cpp:40: an empty prompt generates nothing
        if (!prompts) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null prompts"};
        if (max_tokens < 0) max_tokens = 0;
        check_ids(s, prompts, static_cast<size_t>(s.B) * prompt_len);
        if (prompt_len > sh.max_len)
            throw ApiError{GH_ERR_RUNTIME, "InferenceSession: context exceeds max_len"};
        const size_t B = s.B, V = sh.vocab;

        reset_session(s);
        for (size_t b = 0; b < B; b++)
            std::memcpy(s.host_ids + b * s.hist_stride, prompts + b * prompt_len,
                        prompt_len * sizeof(int));
        HIP_CHECK(hipMemcpyAsync(s.hist, s.host_ids, B * s.hist_stride * sizeof(int),
                                 hipMemcpyHostToDevice, s.stream));
        const float* du =
            opt->greedy ? nullptr : stage_uniforms(s, uniforms, B * static_cast<size_t>(max_tokens));
        float* log = nullptr;
        if (step_logits_host) {
            const size_t need = (static_cast<size_t>(prompt_len) + max_tokens) * B * V;
            if (s.logit_log_cap < need) {
                if (s.logit_log) HIP_CHECK(hipFree(s.logit_log));
                s.logit_log = nullptr;
                dev_alloc(s.logit_log, need);
                s.logit_log_cap = need;
            }
            log = s.logit_log;
        }
        size_t steps = 0;
        HIP_CHECK(hipEventRecord(s.ev[0], s.stream));
        run_prompt(s, prompt_len, log, &steps);
        HIP_CHECK(hipEventRecord(s.ev[1], s.stream));
        const auto [made, stepped] = run_decode(s, max_tokens, *opt, du, max_tokens, seed, log, &steps);
        (void)made;
        HIP_CHECK(hipEventRecord(s.ev[2], s.stream));

        const int total = s.n_hist;
        HIP_CHECK(hipMemcpyAsync(s.host_ids, s.hist, B * s.hist_stride * sizeof(int),
                                 hipMemcpyDeviceToHost, s.stream));
        HIP_CHECK(hipStreamSynchronize(s.stream));
        check_persist_abort(s);
        const size_t out_stride = static_cast<size_t>(prompt_len) + max_tokens;
        for (size_t b = 0; b < B; b++)
            std::memcpy(out_tokens + b * out_stride, s.host_ids + b * s.hist_stride,
                        total * sizeof(int));
        *out_len = total;
        if (step_logits_host)
            HIP_CHECK(hipMemcpy(step_logits_host, s.logit_log, steps * B * V * sizeof(float),
                                hipMemcpyDeviceToHost));
        if (n_steps) *n_steps = static_cast<int32_t>(steps);
        HIP_CHECK(hipEventElapsedTime(&s.timing.prompt_ms, s.ev[0], s.ev[1]));
        HIP_CHECK(hipEventElapsedTime(&s.timing.decode_ms, s.ev[1], s.ev[2]));
        s.timing.prompt_steps = prompt_len;
        s.timing.decode_steps = stepped;
    });
}

gh_status gh_pick_noalloc(const float* logits, int32_t batch, int32_t vocab, const int32_t* history,
                          int32_t history_stride, int32_t n_history, const gh_sampling* opt,
                          const float* uniforms, uint64_t seed, int32_t pick_index, int32_t* out_ids,
                          void* hip_stream) {
    return guard([&] {
        if (!logits || !opt || !out_ids) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        if (batch < 1 || vocab < 1 || n_history < 0 || pick_index < 0 || n_history > history_stride
            || (n_history > 0 && !history))
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "gh_pick_noalloc: bad sizes"};
        check_sampling(*opt);
        const size_t work_stride = (static_cast<size_t>(vocab) + kPickThreads + 3) / 4 * 4;
        if (static_cast<size_t>(batch) * work_stride > kNoAllocScratchFloats)
            throw ApiError{GH_ERR_INVALID_ARGUMENT,
                           "gh_pick_noalloc: batch x (vocab + 1024) floats exceed the 4 MiB scratch array ("
                               + std::to_string(kNoAllocScratchFloats) + " floats)"};
        PickParams p{};
        p.logits = logits;
        p.work = scratch_on_current_device();
        p.work_stride = static_cast<int>(work_stride);
        p.V = vocab;
        p.hist = const_cast<int*>(history);  // read only on this path
        p.hist_stride = history_stride;
        p.n_hist = n_history;
        p.pick_idx = uniforms ? 0 : pick_index;
        p.tok = nullptr;
        p.temperature = opt->temperature;
        p.top_k = opt->top_k;
        p.top_p = opt->top_p;
        p.penalty = opt->repetition_penalty;
        p.greedy = opt->greedy;
        p.uniforms = uniforms;
        p.u_stride = 1;
        p.seed_lo = static_cast<unsigned>(seed & 0xFFFFFFFFu);
        p.seed_hi = static_cast<unsigned>(seed >> 32);
        p.sort_cap = kPickWorkFloats;
        hipLaunchKernelGGL(pick_noalloc_kernel, dim3(batch), dim3(kPickThreads), kPickWorkFloats * sizeof(float),
                           static_cast<hipStream_t>(hip_stream), p, out_ids);
        HIP_CHECK(hipGetLastError());
    });
}

gh_status gh_session_last_timing(const gh_session* s, gh_timing* out) {
    return guard([&] {
        if (!s || !out) throw ApiError{GH_ERR_INVALID_ARGUMENT, "null argument"};
        *out = s->impl->timing;
        out->row_picks = 0;
        if (s->impl->ctl) {
            unsigned n = 0;
            HIP_CHECK(hipMemcpy(&n, &s->impl->ctl->row_picks, sizeof(n), hipMemcpyDeviceToHost));
            out->row_picks = static_cast<int32_t>(n);
        }
    });
}

gh_status gh_device_info(char* name, size_t name_len, int32_t* compute_units, int32_t* is_gfx950) {
    return guard([&] {
        require_gpu();
        int dev = 0;
        HIP_CHECK(hipGetDevice(&dev));
        hipDeviceProp_t prop;
        HIP_CHECK(hipGetDeviceProperties(&prop, dev));
        if (name && name_len) {
            std::snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
        }
        if (compute_units) *compute_units = prop.multiProcessorCount;
        if (is_gfx950) *is_gfx950 = std::strstr(prop.gcnArchName, "gfx950") != nullptr;
        (void)scratch_on_current_device();  // set-up for gh_pick_noalloc on this device
    });
}

gh_status gh_device_read_bandwidth(size_t bytes, int32_t repeats, double* gb_per_s) {
    return guard([&] {
        require_gpu();
        if (!gb_per_s || bytes < (1u << 20) || repeats < 1)
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "read bandwidth probe: need >= 1 MiB, >= 1 repeat"};
        const size_t n4 = bytes / sizeof(float4);
        struct Scratch {  // released on every path out of this function
            float4* buf = nullptr;
            float* sink = nullptr;
            hipEvent_t e0 = nullptr, e1 = nullptr;
            ~Scratch() {
                if (e0) (void)hipEventDestroy(e0);
                if (e1) (void)hipEventDestroy(e1);
                if (buf) (void)hipFree(buf);
                if (sink) (void)hipFree(sink);
            }
        } t;
        HIP_CHECK(hipMalloc(&t.buf, n4 * sizeof(float4)));
        HIP_CHECK(hipMalloc(&t.sink, sizeof(float)));
        HIP_CHECK(hipMemset(t.buf, 0x3c, n4 * sizeof(float4)));  // finite floats, not zeros
        HIP_CHECK(hipEventCreate(&t.e0));
        HIP_CHECK(hipEventCreate(&t.e1));
        double best = 0.0;
        for (int r = 0; r < repeats + 1; r++) {  // the first pass warms up
            HIP_CHECK(hipEventRecord(t.e0, nullptr));
            hipLaunchKernelGGL(stream_read_kernel, dim3(8192), dim3(256), 0, nullptr, t.buf, n4, t.sink);
            HIP_CHECK(hipGetLastError());
            HIP_CHECK(hipEventRecord(t.e1, nullptr));
            HIP_CHECK(hipEventSynchronize(t.e1));
            float ms = 0.0f;
            HIP_CHECK(hipEventElapsedTime(&ms, t.e0, t.e1));
            if (r > 0) best = std::max(best, static_cast<double>(n4) * sizeof(float4) / (ms * 1e-3) / 1e9);
        }
        *gb_per_s = best;
    });
}

gh_status gh_device_handoff_latency(int32_t load_policy, int32_t device_scope_store, int32_t peer, int32_t busy,
                                    double* us_per_round_trip, int32_t* xcd_a, int32_t* xcd_b) {
    return guard([&] {
        require_gpu();
        HandoffKernel kernel = handoff_kernel_for(load_policy, device_scope_store != 0);
        if (!kernel || !us_per_round_trip || peer < 1 || peer > 15)
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "hand-off probe: load policy 0..2, peer workgroup 1..15"};
        struct Scratch {  // released on every path out of this function
            unsigned *cells = nullptr, *xcds = nullptr, *stop = nullptr;
            unsigned long long* ticks = nullptr;
            float4* big = nullptr;
            float* sink = nullptr;
            hipStream_t s1 = nullptr, s2 = nullptr;
            ~Scratch() {
                if (stop) *stop = 1u;
                (void)hipDeviceSynchronize();
                if (s1) (void)hipStreamDestroy(s1);
                if (s2) (void)hipStreamDestroy(s2);
                for (void* p : {static_cast<void*>(cells), static_cast<void*>(xcds), static_cast<void*>(ticks),
                                static_cast<void*>(big), static_cast<void*>(sink)})
                    if (p) (void)hipFree(p);
                if (stop) (void)hipHostFree(stop);
            }
        } t;
        const int rounds = 1000;
        const size_t big_bytes = busy ? (size_t(2) << 30) : sizeof(float4);
        dev_alloc(t.cells, 256);
        dev_alloc(t.xcds, 16);
        dev_alloc(t.ticks, 2);
        HIP_CHECK(hipMalloc(&t.big, big_bytes));
        HIP_CHECK(hipMemset(t.big, 0, big_bytes));
        dev_alloc(t.sink, 1);
        HIP_CHECK(hipHostMalloc(&t.stop, sizeof(unsigned), hipHostMallocCoherent));
        *t.stop = 0u;
        HIP_CHECK(hipStreamCreateWithFlags(&t.s1, hipStreamNonBlocking));
        HIP_CHECK(hipStreamCreateWithFlags(&t.s2, hipStreamNonBlocking));
        HIP_CHECK(hipDeviceSynchronize());
        if (busy) {
            hipLaunchKernelGGL(handoff_probe_hog, dim3(240), dim3(256), 0, t.s2, t.big, big_bytes / sizeof(float4),
                               t.stop, t.sink);
            HIP_CHECK(hipGetLastError());
        }
        hipLaunchKernelGGL(kernel, dim3(16), dim3(64), 0, t.s1, t.cells, peer, rounds, t.ticks, t.xcds);
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(t.s1));
        *t.stop = 1u;
        HIP_CHECK(hipDeviceSynchronize());
        unsigned long long ticks[2];
        unsigned xcds[16];
        HIP_CHECK(hipMemcpy(ticks, t.ticks, sizeof(ticks), hipMemcpyDeviceToHost));
        HIP_CHECK(hipMemcpy(xcds, t.xcds, sizeof(xcds), hipMemcpyDeviceToHost));
        *us_per_round_trip = static_cast<double>(ticks[0]) / 100.0 / rounds;
        if (xcd_a) *xcd_a = static_cast<int32_t>(xcds[0]);
        if (xcd_b) *xcd_b = static_cast<int32_t>(xcds[peer]);
    });
}

gh_status gh_device_mfma_issue(int32_t mode, int32_t valu_per_slot, double* clk_per_product, double* clk_per_valu_slot,
                               double* shader_mhz) {
    return guard([&] {
        require_gpu();
        using Kernel = void (*)(long long*, int, int, float, float);
        Kernel kernel = valu_per_slot == 8    ? mfma_issue_probe_kernel<8>
                        : valu_per_slot == 16 ? mfma_issue_probe_kernel<16>
                        : valu_per_slot == 24 ? mfma_issue_probe_kernel<24>
                                              : nullptr;
        if (!kernel || mode < 1 || mode > 6 || (mode & 1 && mode & 4) || !clk_per_product || !clk_per_valu_slot ||
            !shader_mhz)
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "matrix-core issue probe: mode 1, 2, 3, 4 or 6; 8, 16 or 24 "
                                                    "multiply-adds per slot"};
        const int blocks = 256, iters = 4000;
        struct Scratch {
            long long* out = nullptr;
            ~Scratch() {
                if (out) (void)hipFree(out);
            }
        } t;
        dev_alloc(t.out, static_cast<size_t>(blocks) * 8 * 3);
        for (int rep = 0; rep < 2; rep++) {  // the first run brings the clock up
            hipLaunchKernelGGL(kernel, dim3(blocks), dim3(512), 0, nullptr, t.out, iters, mode, 1.0f, 0.999f);
            HIP_CHECK(hipGetLastError());
            HIP_CHECK(hipDeviceSynchronize());
        }
        std::vector<long long> h(static_cast<size_t>(blocks) * 8 * 3);
        HIP_CHECK(hipMemcpy(h.data(), t.out, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
        double mfma = 0.0, valu = 0.0, cyc = 0.0, wall = 0.0;
        for (int b = 0; b < blocks; b++)
            for (int w = 0; w < 8; w++) {
                const long long* o = &h[(static_cast<size_t>(b) * 8 + w) * 3];
                (w < 4 ? mfma : valu) += static_cast<double>(o[0]);
                const bool busy = w < 4 ? (mode & 5) != 0 : (mode & 2) != 0;
                if (busy) {
                    cyc += static_cast<double>(o[0]);
                    wall += static_cast<double>(o[1]);
                }
            }
        const double slots = static_cast<double>(blocks) * 4 * iters * 8;
        *clk_per_product = (mode & 5) ? mfma / slots : 0.0;
        *clk_per_valu_slot = (mode & 2) ? valu / slots : 0.0;
        *shader_mhz = wall > 0.0 ? cyc / wall * 100.0 : 0.0;  // the constant clock counts at 100 MHz
    });
}

gh_status gh_device_reread_bandwidth(size_t bytes, int32_t passes, double* gb_per_s) {
    return guard([&] {
        require_gpu();
        if (!gb_per_s || bytes < (1u << 20) || passes < 1)
            throw ApiError{GH_ERR_INVALID_ARGUMENT, "re-read bandwidth probe: need >= 1 MiB, >= 1 pass"};
        const size_t n4 = bytes / sizeof(float4);
        struct Scratch {
            float4* buf = nullptr;
            float* sink = nullptr;
            hipEvent_t e0 = nullptr, e1 = nullptr;
            ~Scratch() {
                if (e0) (void)hipEventDestroy(e0);
                if (e1) (void)hipEventDestroy(e1);
                if (buf) (void)hipFree(buf);
                if (sink) (void)hipFree(sink);
            }
        } t;
        HIP_CHECK(hipMalloc(&t.buf, n4 * sizeof(float4)));
        HIP_CHECK(hipMalloc(&t.sink, sizeof(float)));
        HIP_CHECK(hipMemset(t.buf, 0x3c, n4 * sizeof(float4)));  // finite floats, not zeros
        HIP_CHECK(hipEventCreate(&t.e0));
        HIP_CHECK(hipEventCreate(&t.e1));
        // Every pass is a launch of its own that streams the whole buffer (passes inside one
        // launch would only re-read what the resident workgroups hold, which the L2s serve).
        // 2048 x 256 threads with eight loads each cover 64 MiB per round.
        const int grid = static_cast<int>(std::min<size_t>(8192, std::max<size_t>(256, n4 / (256 * 8))));
        for (int r = -2; r < passes; r++) {  // two passes warm up, then one span over the rest
            if (r == 0) HIP_CHECK(hipEventRecord(t.e0, nullptr));
            hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(256), 0, nullptr, t.buf, n4, t.sink);
        }
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipEventRecord(t.e1, nullptr));
        HIP_CHECK(hipEventSynchronize(t.e1));
        float ms = 0.0f;
        HIP_CHECK(hipEventElapsedTime(&ms, t.e0, t.e1));
        *gb_per_s = static_cast<double>(passes) * static_cast<double>(n4) * sizeof(float4) / (ms * 1e-3) / 1e9;
    });
}

}  // extern "C"

// Persistent batch-1 decoder: ONE kernel launch runs a whole run of steps
// (prompt tokens, then pick + step rounds), because at 69M parameters a step is
// ~40 dependent projections of a few microseconds each and a kernel launch per
// projection costs more than the projection.
//
// One workgroup per compute unit stays resident.  Inside a step the phases
//   norm+QKV -> attention -> W_o+residual -> norm+FFN1 -> FFN2+residual  (per layer)
//   -> final norm + logits -> pick
// hand their outputs to the next phase through "cells": 8-byte {value, tag}
// pairs written and read with single device-scope accesses, so a value and the
// tag that says which (step, layer, phase) produced it always travel together.
// A consumer polls the cells it needs until every tag matches; there is no
// separate barrier.  Polling is bounded and watches an abort flag, so every
// wavefront leaves the kernel even if a producer never shows up.
//
// The arithmetic per phase is the same as the one-kernel-per-op path
// (kernels_gemv.h, kernels_attn.h), i.e. src/transformer/inference.cpp:150-258.
#pragma once

#include "kernels_attn.h"
#include "kernels_common.h"
#include "kernels_gemv.h"
#include "kernels_pick.h"

namespace gh {

constexpr int kPersistThreads = 512;
constexpr int kPersistWaves = kPersistThreads / 64;

struct Cell {
    float v;
    unsigned tag;
};

struct LayerPtrs {
    const float *wqkv, *bqkv, *wo, *bo, *w1, *b1, *w2, *b2, *g1, *be1, *g2, *be2;
};

// Floats of one layer when its tensors follow each other in the order of
// LayerPtrs with no gaps (every size is a multiple of 64 floats when d_model
// and the FFN width are multiples of 256): w1 holds gate and up rows for the
// Modern block, b1 has F entries in both.
constexpr size_t layer_floats(size_t D, size_t F, bool modern) {
    return 3 * D * D + 3 * D + D * D + D + (modern ? 2 : 1) * F * D + F + D * F + D + 4 * D;
}

// The tensors of layer l of such a blob.  Plain address arithmetic on a kernel
// argument: no table to fetch before the rows can be requested, and the
// compiler knows the rows are in global memory.
template <int KD, int KF, bool MODERN>
__device__ __forceinline__ LayerPtrs layer_at(const float* layer0, int l) {
    constexpr size_t D = KD * 256, F = KF * 256;
    const float* b = layer0 + static_cast<size_t>(l) * layer_floats(D, F, MODERN);
    asm volatile("" : "+s"(b));
    LayerPtrs w;
    w.wqkv = b, b += 3 * D * D;
    w.bqkv = b, b += 3 * D;
    w.wo = b, b += D * D;
    w.bo = b, b += D;
    w.w1 = b, b += (MODERN ? 2 : 1) * F * D;
    w.b1 = b, b += F;
    w.w2 = b, b += D * F;
    w.b2 = b, b += D;
    w.g1 = b, b += D;
    w.be1 = b, b += D;
    w.g2 = b, b += D;
    w.be2 = b;
    return w;
}

struct PersistCtl {
    unsigned abort;     // set by any workgroup that gave up waiting
    unsigned where;     // phase tag it was waiting for (diagnostics)
    unsigned row_picks;  // picks workgroup 0 made from the whole row (the others: every workgroup, from candidates)
    unsigned pad[29];
    unsigned arrive[16 * 32];  // logits-complete counters, one per 128-byte line
    unsigned xcd_count[8 * 32];  // workgroups that have started on each XCD, one counter per line (kernels_xcd.h)
};

struct PersistParams {
    const float* E;
    const float* P;
    const float* layer0;  // layer 0's first tensor; the layers follow each other as layer_at() says
    const float *gf, *bf, *rope_cos, *rope_sin;
    int d, F, V, L, H;
    KvLayout kv;
    // One block of exchange cells, in this order: x after a layer [d], x after the
    // attention half [d], q [d], new key [d], new value [d], attention output [d],
    // FFN hidden [F], the picked token [1] (+ 1 unused), then what the workgroups leave for
    // a pick that each of them makes itself: planes of one cell per workgroup (greedy:
    // largest logit, its index; top-k: four values, four indices, the fifth value) and
    // the host's stop request as workgroup 0 read it [1]; then, from an even index, the
    // shares of a head's attention that other workgroups computed [16 heads][15][66].  The
    // kernel addresses them from the one
    // base: eight pointers held through the whole token loop are sixteen scalar
    // registers that would otherwise be parked in vector lanes and fetched back.
    Cell* cells;
    float* logits;     // [V]
    float* logit_log;  // [steps][V] or nullptr
    PersistCtl* ctl;
    int* hist;  // token history of the sequence
    int pos0;          // cache positions already filled
    int n_prompt;      // steps whose token is hist[pos0 + s]
    int n_steps;       // step() calls in this launch
    int n_picks;       // picks in this launch
    int start_with_pick;  // the first pick uses the logits already in memory
    int tok0;             // >= 0: the token of step 0 (not yet in the history: the kernel records it)
    int wg_picks;         // picks that follow a step may be made by every workgroup from candidates
    unsigned epoch;    // tag base of this launch; (epoch + s) never repeats in a session
    unsigned arrive_base;  // logits phases completed before this launch
    PickParams pick;
    unsigned spin_limit;
    // Streaming (all optional).  feed: pinned host memory, one 8-byte {token, tag}
    // word per pick of this launch, tag = feed_base + pick number + 1, written as
    // each token is picked so the host can hand it on while the kernel goes on; a
    // token of -1 says the run ended before that pick.  stop_request: a pinned host
    // word the host sets to end the run at the next pick.  stop_token: the run ends
    // after the step that follows a pick of this token (-1: none).
    unsigned long long* feed;
    unsigned feed_base;
    const unsigned* stop_request;
    int stop_token;
    unsigned long long* prof;  // optional: phase-end timestamps of workgroup 0 (100 MHz clock)
    int prof_cap;
};

__device__ __forceinline__ void cell_put(Cell* c, float v, unsigned tag) {
    const unsigned long long w =
        (static_cast<unsigned long long>(tag) << 32) | static_cast<unsigned long long>(__float_as_uint(v));
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(c), w, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bool cell_get(const Cell* c, unsigned tag, float& v) {
    const unsigned long long w = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(c),
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v = __uint_as_float(static_cast<unsigned>(w));
    return static_cast<unsigned>(w >> 32) == tag;
}

__device__ __forceinline__ void coherent_store(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// "Did any thread of the workgroup give up its wait": a barrier and one LDS word
// that stays zero until a wait is abandoned, after which the kernel only exits.
// (__syncthreads_or reads the workgroup's dimensions from the dispatch packet on
// every call: a trip to memory behind every exchange.)  The kernel clears the word
// before its first wait.
__shared__ unsigned g_wait_abandoned;

__device__ __forceinline__ bool any_abandoned(bool failed) {
    if (failed) g_wait_abandoned = 1u;
    __syncthreads();
    return g_wait_abandoned != 0u;
}

// Workgroup-wide: waits until cells [0, n) carry `tag`, copying the values to
// dst (LDS).  Every thread polls only its own cells and stops as soon as they
// have arrived; the workgroup meets once at the end.  Returns false when the wait
// was abandoned (the kernel must exit).
__device__ inline bool gather_cells(const Cell* src, int n, unsigned tag, float* dst,
                                    const PersistParams& p) {
    const __amdgpu_buffer_rsrc_t rs = make_buffer(src, static_cast<unsigned>(n) * 8u);
    const int itag = static_cast<int>(tag);
    unsigned spins = 0;
    bool failed = false;
    for (;;) {
        bool ok = true;
        // Two cells per 16-byte load.  The stride is the compile-time workgroup size:
        // blockDim.x is a load from the dispatch packet, one more trip to memory in
        // front of every poll.
        for (int i = 2 * threadIdx.x; i < n; i += 2 * kPersistThreads) {
            const v4i w = coherent_load16(rs, static_cast<unsigned>(i) * 8u);
            ok = ok && w.y == itag && (i + 1 >= n || w.w == itag);
            dst[i] = __int_as_float(w.x);
            if (i + 1 < n) dst[i + 1] = __int_as_float(w.z);
        }
        if (ok) break;
        ++spins;
        if (spins > p.spin_limit
            || ((spins & 63u) == 0u
                && __hip_atomic_load(&p.ctl->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
            failed = true;
            break;
        }
    }
    if (any_abandoned(failed)) {
        if (threadIdx.x == 0) {
            __hip_atomic_store(&p.ctl->where, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&p.ctl->abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return false;
    }
    return true;
}

// Reports pick number i_pick of this launch to the host: one 8-byte word in pinned memory.
__device__ __forceinline__ void feed_put(const PersistParams& p, int i_pick, int token) {
    const unsigned long long w =
        (static_cast<unsigned long long>(p.feed_base + static_cast<unsigned>(i_pick) + 1u) << 32)
        | static_cast<unsigned long long>(static_cast<unsigned>(token));
    __hip_atomic_store(p.feed + i_pick, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// One pick by workgroup 0 (text_gen.cpp:48-61 / :80-86): waits until every
// workgroup's logits rows have landed, picks, records the token in the history
// and publishes it in the token cell.  The other workgroups return at once and
// learn the token from the cell.  False: the wait was abandoned.
// NT: threads of the workgroup (all of them call).  tok_cell: where the token is
// published.  chosen_out: the pick, for every thread of workgroup 0.
template <bool ROW_LDS, bool FEED, int NT = kPersistThreads>
__device__ __forceinline__ bool persist_pick(const PersistParams& p, float* lds, int i_pick,
                                    unsigned arrive_gen, unsigned tok_tag, bool wait_logits, int grid,
                                    Cell* tok_cell, int* chosen_out = nullptr) {
    if (blockIdx.x != 0) return true;
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));  // nothing of the pick is computed ahead of the token loop
    if (p.prof && i_pick < 1024 && tid == 0) p.prof[p.prof_cap / 2 + 4 * i_pick + 2] = __builtin_amdgcn_s_memrealtime();
    PickParams pk = p.pick;
    pk.n_hist = p.pick.n_hist + i_pick;
    pk.pick_idx = p.pick.pick_idx + i_pick;
    // the draw needs no logits: form it while they arrive
    const float u = pk.greedy ? 0.0f : pick_draw(pk, 0);
    // The host's stop request (one trip over the bus while the other workgroups'
    // logits arrive): no pick; every workgroup leaves when it reads the token cell.
    if constexpr (FEED) {
        const unsigned stop = __hip_atomic_load(p.stop_request, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        if (__builtin_amdgcn_readfirstlane(stop) != 0u) {
            if (tid == 0) {
                cell_put(tok_cell, __int_as_float(-1), tok_tag);
                feed_put(p, i_pick, -1);
            }
            return false;
        }
    }
    if (wait_logits) {
        // one wavefront watches the 16 arrival counters; the workgroup meets once
        bool failed = false;
        if (tid < 64) {
            const unsigned target = arrive_gen * static_cast<unsigned>(grid);
            unsigned spins = 0;
            for (;;) {
                unsigned v = 0;
                if (tid < 16)
                    v = __hip_atomic_load(&p.ctl->arrive[tid * 32], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
                // wrap-safe: the counters run on for the life of the session
                if (static_cast<int>(__builtin_amdgcn_readfirstlane(v) - target) >= 0) break;
                ++spins;
                if (spins > p.spin_limit
                    || ((spins & 63u) == 63u
                        && __hip_atomic_load(&p.ctl->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
                    failed = true;
                    break;
                }
            }
        }
        if (any_abandoned(failed)) {
            if (tid == 0) {
                __hip_atomic_store(&p.ctl->where, 0xFFFFFFFEu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&p.ctl->abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            return false;
        }
    }
    unsigned long long* pp = (p.prof && i_pick < 1024) ? p.prof + p.prof_cap / 2 + 4 * i_pick : nullptr;
    if (pp && tid == 0) pp[0] = __builtin_amdgcn_s_memrealtime();
    const int chosen = ROW_LDS ? pick_body<true, NT>(pk, 0, lds, lds + pk.V, u)
                               : pick_body<true, NT>(pk, 0, pk.work, lds, u);
    if (chosen_out) *chosen_out = chosen;
    if (tid == 0) {
        __hip_atomic_store(&p.hist[pk.n_hist], chosen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        cell_put(tok_cell, __int_as_float(chosen), tok_tag);
        if constexpr (FEED) feed_put(p, i_pick, chosen);
        __hip_atomic_fetch_add(&p.ctl->row_picks, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (pp) pp[1] = __builtin_amdgcn_s_memrealtime();
    }
    return true;
}

template <int KV>
__device__ __forceinline__ void load_row(const float* W, int row, int K, int lane, float4 (&w)[KV]) {
    const float4* wr = reinterpret_cast<const float4*>(W + static_cast<size_t>(row) * K);
#pragma unroll
    for (int i = 0; i < KV; i++) w[i] = wr[i * 64 + lane];
}

template <int KV>
__device__ __forceinline__ float dot_row(const float4 (&w)[KV], const float4 (&h)[KV]) {
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < KV; i++) a += dot4(w[i], h[i]);
    return wave_sum(a);
}

// The same dot product with the input vector read from LDS as it is consumed.
template <int KV>
__device__ __forceinline__ float dot_row_lds(const float4 (&w)[KV], const float* x, int lane) {
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < KV; i++) a += dot4(w[i], reinterpret_cast<const float4*>(x)[i * 64 + lane]);
    return wave_sum(a);
}

// Register-resident norm parameters of one lane: the gamma (and beta) float4s
// that line up with its slice of the row.
template <int KV>
struct NormRegs {
    float4 g[KV];
    float4 b[KV];
};

template <int KV, int PRO>
__device__ __forceinline__ void load_norm(const float* gamma, const float* beta, int lane, NormRegs<KV>& n) {
    if constexpr (PRO != PRO_PLAIN) {
#pragma unroll
        for (int i = 0; i < KV; i++) n.g[i] = reinterpret_cast<const float4*>(gamma)[i * 64 + lane];
    }
    if constexpr (PRO == PRO_LAYERNORM) {
#pragma unroll
        for (int i = 0; i < KV; i++) n.b[i] = reinterpret_cast<const float4*>(beta)[i * 64 + lane];
    }
}

// This lane's slice of the input vector held in LDS, normalised with preloaded
// gamma / beta (layer_norm_row, inference.cpp:30-58).
template <int KV, int PRO>
__device__ __forceinline__ void load_input(const float* xs, const NormRegs<KV>& n, int lane, float4 (&h)[KV]) {
    constexpr int K = KV * 256;
#pragma unroll
    for (int i = 0; i < KV; i++) h[i] = reinterpret_cast<const float4*>(xs)[i * 64 + lane];
    if constexpr (PRO == PRO_RMSNORM) {
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < KV; i++) ss += dot4(h[i], h[i]);
        const float r = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(K) + kNormEps);
#pragma unroll
        for (int i = 0; i < KV; i++)
            h[i] = make_float4(n.g[i].x * h[i].x * r, n.g[i].y * h[i].y * r, n.g[i].z * h[i].z * r,
                               n.g[i].w * h[i].w * r);
    } else if constexpr (PRO == PRO_LAYERNORM) {
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < KV; i++) sum += (h[i].x + h[i].y) + (h[i].z + h[i].w);
        const float mean = wave_sum(sum) / static_cast<float>(K);
        float var = 0.0f;
#pragma unroll
        for (int i = 0; i < KV; i++) {
            h[i] = make_float4(h[i].x - mean, h[i].y - mean, h[i].z - mean, h[i].w - mean);
            var += dot4(h[i], h[i]);
        }
        const float inv_std = 1.0f / sqrtf(wave_sum(var) / static_cast<float>(K) + kNormEps);
#pragma unroll
        for (int i = 0; i < KV; i++)
            h[i] = make_float4(n.g[i].x * h[i].x * inv_std + n.b[i].x, n.g[i].y * h[i].y * inv_std + n.b[i].y,
                               n.g[i].z * h[i].z * inv_std + n.b[i].z, n.g[i].w * h[i].w * inv_std + n.b[i].w);
    }
}

// Everything phase A (norm1 + QKV) needs that does not depend on the
// activations: two weight rows, the norm parameters, the biases and the
// rotation of this position.  Loaded one exchange ahead of its use.
template <int KD, int PRO>
struct QkvOperands {
    float4 w0[KD], w1[KD];
    NormRegs<KD> n;
    float b0, b1, cs, sn;
};

template <int KD, int PRO, bool MODERN>
__device__ __forceinline__ void load_qkv_operands(const PersistParams& p, const LayerPtrs& w, int item,
                                                  int pos, int lane, QkvOperands<KD, PRO>& o) {
    constexpr int D = KD * 256, HS = 64;
    const int row = 2 * item;
    load_row<KD>(w.wqkv, row, D, lane, o.w0);
    load_row<KD>(w.wqkv, row + 1, D, lane, o.w1);
    load_norm<KD, PRO>(w.g1, w.be1, lane, o.n);
    o.b0 = w.bqkv[row];
    o.b1 = w.bqkv[row + 1];
    o.cs = 1.0f;
    o.sn = 0.0f;
    if (MODERN && row < 2 * D) {
        const int j = ((row % D) % HS) >> 1;
        o.cs = p.rope_cos[pos * (HS / 2) + j];
        o.sn = p.rope_sin[pos * (HS / 2) + j];
    }
}

// KD = d_model / 256, KF = FFN width / 256; head size 64.  FEED: the streaming
// variant (feed, stop word, stop token); the plain one carries none of it.
template <int KD, int KF, bool MODERN, bool ROW_LDS, bool FEED>
__global__ __launch_bounds__(kPersistThreads) void persist_decode_kernel(const PersistParams p) {
    extern __shared__ __attribute__((aligned(128))) float lds[];
    constexpr int D = KD * 256, F = KF * 256, HS = 64;
    constexpr int PRO = MODERN ? PRO_RMSNORM : PRO_LAYERNORM;
    constexpr int RL = 8;  // logits rows per wavefront item
    // Beyond kAttnShareFrom positions a head's attention is shared by several workgroups,
    // kAttnShare positions each: what a workgroup's eight wavefronts take in one batch of 32.
    // (One workgroup up to 512 positions: 256..512 ran at 132 us per token alone and 138 in two shares.)
    constexpr int kAttnShareFrom = 512, kAttnShare = 256, kAttnMaxShares = 16;
    float* xs = lds;                      // [D] residual stream of this step
    float* vin = lds + D;                 // [max(D, F)] attention output / FFN hidden
    float* ascr = vin + (F > D ? F : D);  // attention scratch: q, k, v of the head + wave partials
    int* ptab = reinterpret_cast<int*>(ascr + 192 + kPersistWaves * 4 * 68);  // [pages_per_seq]
    int tid = threadIdx.x, wave = tid >> 6;
    int lane = tid & 63;
    const int wg = blockIdx.x, G = gridDim.x;
    const int V = p.V, L = p.L, H = p.H;
    const int stride = G * kPersistWaves;  // wavefronts in the grid
    int first = wg + G * wave;             // item i of a phase goes to workgroup i % G
    int i_pick = 0;
    unsigned arrive_gen = p.arrive_base;
    int n_stamp = 0;
    bool ended = false;  // a picked token was the stop token
    // Greedy picks of this launch are made by every workgroup from per-workgroup maxima
    // (the pick that opens a launch on logits of an earlier one is workgroup 0's).
    const bool fast_greedy = p.wg_picks != 0 && p.pick.greedy != 0;
    // Top-k picks likewise, when a workgroup's rows are one item per wavefront (64 values)
    // and every workgroup has an item (at least eight values).
    const bool fast_topk = p.wg_picks != 0 && p.pick.greedy == 0 && p.pick.top_k > 0 && p.pick.top_k <= 64 && p.pick.top_k < V
                           && (V + RL - 1) / RL <= G * kPersistWaves && V >= G * RL;
    bool pairs_out = false;  // the last logits phase left the planes for the pick that follows
    auto stamp = [&]() {
        if (p.prof && wg == 0 && tid == 0 && n_stamp < p.prof_cap) p.prof[n_stamp] = __builtin_amdgcn_s_memrealtime();
        n_stamp++;
    };
    stamp();

    // The sequence's page table never changes while the kernel runs.
    for (int i = tid; i < p.kv.pages_per_seq; i += kPersistThreads) ptab[i] = p.kv.page_table[i];
    if (tid == 0) g_wait_abandoned = 0u;
    __syncthreads();
    auto kv_at = [&](int layer, int which, int head, int t) -> size_t {
        const int page = ptab[t >> p.kv.page_shift];
        const int slot = t & ((1 << p.kv.page_shift) - 1);
        const size_t run = ((static_cast<size_t>(layer) * p.kv.n_pages + page) * 2 + which) * H + head;
        return ((run << p.kv.page_shift) + slot) * HS;
    };

    constexpr int NQKV = 3 * D / 2;  // phase A items: pairs of rows
    const bool has_qkv = wg + G * wave < NQKV;

    for (int s = 0;; s++) {
        // ===== pick before step s (text_gen.cpp:48-61): the first one of a launch may
        // use logits that are already in memory, later ones follow step s - 1.  One call
        // site: the sampler is the largest piece of code in the kernel.
        const bool pick_here =
            (!FEED || !ended) && i_pick < p.n_picks && s >= p.n_prompt && (s > 0 || p.start_with_pick);
        // Layer 0's QKV operands are fetched while the token is on its way.
        QkvOperands<KD, PRO> qo;
        auto load_qo0 = [&]() {
            const LayerPtrs w0l = layer_at<KD, KF, MODERN>(p.layer0, 0);
            if (has_qkv) load_qkv_operands<KD, PRO, MODERN>(p, w0l, first, p.pos0 + s, lane, qo);
            else qo = QkvOperands<KD, PRO>{};  // nothing to keep alive across steps
        };
        int tok_fast = 0;
        bool tok_known = false;
        if (pick_here && pairs_out) {
            // ===== a pick without a picker (text_gen.cpp:48-61, :135-209).  The logits phase
            // of step s - 1 left, per workgroup, its largest penalised logit and first index
            // (greedy), or its four largest scaled ones and the fifth's value (top-k of at most
            // 64).  Every workgroup reads all of them and makes the same pick itself: the
            // token needs one exchange and no row is read back.
            asm volatile("" : "+v"(tid));
            wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            lane = tid & 63;
            first = wg + G * wave;
            unsigned long long* pp =
                (p.prof && wg == 0 && tid == 0 && i_pick < 1024) ? p.prof + p.prof_cap / 2 + 4 * i_pick : nullptr;
            if (pp) pp[2] = __builtin_amdgcn_s_memrealtime();
            if (s < p.n_steps) load_qo0();
            const unsigned tt = ((p.epoch + static_cast<unsigned>(s)) * static_cast<unsigned>(L + 1)
                                 + static_cast<unsigned>(L)) * 8u + 7u;
            const Cell* pc = p.cells + 6 * D + F + 2;
            float* g = lds;  // the gathered planes; xs and vin hold nothing between steps
            bool stop = false;
            if (fast_greedy) {
                if (!gather_cells(pc, 2 * G + 1, tt, g, p)) return;
                if (pp) pp[0] = __builtin_amdgcn_s_memrealtime();
                float best = -INFINITY;
                int bi = 0x7FFFFFFF;
                for (int j = lane; j < G; j += 64) {
                    const float v = g[j];
                    const int i = __float_as_int(g[G + j]);
                    if (v > best || (v == best && i < bi)) {
                        best = v;
                        bi = i;
                    }
                }
                wave_first_max(best, bi);
                tok_fast = bi == 0x7FFFFFFF ? 0 : bi;
                stop = FEED && __float_as_int(g[2 * G]) != 0;
                tok_known = true;
            } else {
                PickParams pk = p.pick;
                pk.pick_idx = p.pick.pick_idx + i_pick;
                const float u = pick_draw(pk, 0);  // needs no logits
                PTICK_BEGIN();
                if (!gather_cells(pc, 9 * G + 1, tt, g, p)) return;
                PTICK(9);
                if (pp) pp[0] = __builtin_amdgcn_s_memrealtime();
                // The four planes hold every value that can survive the cut when the largest
                // value a workgroup kept back is below the k-th largest of the planes; the
                // sampler checks that and declines otherwise (workgroup 0 then picks from the row).
                float kept_back = -INFINITY;
                for (int j = lane; j < G; j += 64) kept_back = fmaxf(kept_back, g[8 * G + j]);
                kept_back = wave_max(kept_back);
                PTICK(10);
                float* red = g + 9 * G + 8;
                int* ishare = reinterpret_cast<int*>(red + 8);
                float* work = g + 9 * G + 64;
                const int c = sample_topk_fast<kPersistThreads, 2>(g, 4 * G, 1.0f, pk.top_k, pk.top_p, u, work, red, ishare,
                                                                   reinterpret_cast<const int*>(g + 4 * G), kept_back, V - 1);
                stop = FEED && __float_as_int(g[9 * G]) != 0;
                __syncthreads();
                tok_fast = c;
                tok_known = c >= 0 || stop;
#ifdef GH_PICK_TICKS
                if (wg == 0 && tid == 0) g_pick_ticks[c >= 0 ? 12 : 13] += 1;
#endif
            }
            if (stop) tok_fast = -1;  // the host asked for the run to end here
            if (tok_known) {
                if (wg == 0 && tid == 0) {
                    if (tok_fast >= 0)
                        __hip_atomic_store(&p.hist[p.pick.n_hist + i_pick], tok_fast, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                    if constexpr (FEED) feed_put(p, i_pick, tok_fast);
                }
                if (pp) pp[1] = __builtin_amdgcn_s_memrealtime();
                i_pick++;
            }
        }
        if (pick_here && !tok_known) {
            const unsigned tt = ((p.epoch + static_cast<unsigned>(s)) * static_cast<unsigned>(L + 1)
                                 + static_cast<unsigned>(L)) * 8u + (s == 0 ? 6u : 7u);
            if (!persist_pick<ROW_LDS, FEED>(p, lds, i_pick, arrive_gen, tt, s > 0, G, p.cells + 6 * p.d + p.F)) return;
            i_pick++;
            if (wg == 0) {
                // the pick used the whole LDS; restore the page table
                __syncthreads();
                for (int i = tid; i < p.kv.pages_per_seq; i += kPersistThreads) ptab[i] = p.kv.page_table[i];
                __syncthreads();
            }
        }
        pairs_out = false;
        stamp();
        if ((FEED && ended) || s >= p.n_steps) break;
        if (FEED && tok_known && tok_fast < 0) return;
        asm volatile("" : "+v"(tid));  // as in the layer loop below
        wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        lane = tid & 63;
        first = wg + G * wave;
        const int pos = p.pos0 + s;
        const unsigned sb = (p.epoch + 1u + static_cast<unsigned>(s)) * static_cast<unsigned>(L + 1);
        auto tag_of = [&](int layer, int ph) {
            return (sb + static_cast<unsigned>(layer)) * 8u + static_cast<unsigned>(ph) + 1u;
        };
        const bool want_logits = (s >= p.n_prompt - 1) || p.logit_log != nullptr || s == p.n_steps - 1;

        if (!tok_known) load_qo0();

        // ---- token and embedding (inference.cpp:159-182)
        int tok;
        if (s < p.n_prompt) {
            if (s == 0 && p.tok0 >= 0) {
                // handed over in the launch's arguments: no copy and no launch in front of a single step
                tok = p.tok0;
                if (wg == 0 && tid == 0)
                    __hip_atomic_store(&p.hist[pos], tok, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                tok = p.hist[pos];
            }
        } else if (tok_known) {
            tok = tok_fast;
            if constexpr (FEED) ended = tok == p.stop_token;  // this step is the last one
        } else {
            // the pick that followed step s-1 (or opened the launch)
            const unsigned tt = ((p.epoch + static_cast<unsigned>(s)) * static_cast<unsigned>(L + 1)
                                 + static_cast<unsigned>(L)) * 8u + (s == 0 ? 6u : 7u);
            if (!gather_cells((p.cells + 6 * D + F), 1, tt, ascr, p)) return;
            tok = __float_as_int(ascr[0]);
            __syncthreads();
            if constexpr (FEED) {
                if (tok < 0) return;          // the host asked for the run to end here
                ended = tok == p.stop_token;  // this step is the last one
            }
        }
        for (int j = tid; j < D; j += kPersistThreads) {
            float v = p.E[static_cast<size_t>(tok) * D + j];
            if (!MODERN) v += p.P[static_cast<size_t>(pos) * D + j];
            xs[j] = v;
        }
        __syncthreads();

        for (int l = 0; l < L; l++) {
            const LayerPtrs w = layer_at<KD, KF, MODERN>(p.layer0, l);
            // Keep the compiler from hoisting every lane- and item-derived address of
            // every phase out of the layer loop (they would not fit in registers and
            // would be spilled to scratch memory): re-derive them per layer.
            asm volatile("" : "+v"(tid));
            wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            lane = tid & 63;
            first = wg + G * wave;

            // ===== phase A: norm1 + QKV (+bias, RoPE) -> q / new k / new v cells and the cache
            for (int item = first; item < NQKV; ) {
                const int row = 2 * item;
                float4 h[KD];
                load_input<KD, PRO>(xs, qo.n, lane, h);
                float a = dot_row<KD>(qo.w0, h) + qo.b0;
                float c = dot_row<KD>(qo.w1, h) + qo.b1;
                if (lane == 0) {
                    const int sec = row / D, col = row - sec * D;
                    if (MODERN && sec < 2) {
                        const float ra = a * qo.cs - c * qo.sn;
                        const float rc = a * qo.sn + c * qo.cs;
                        a = ra;
                        c = rc;
                    }
                    const unsigned t = tag_of(l, 0);
                    if (sec == 0) {
                        cell_put((p.cells + 2 * D) + col, a, t);
                        cell_put((p.cells + 2 * D) + col + 1, c, t);
                    } else {
                        Cell* dst = (sec == 1 ? (p.cells + 3 * D) : (p.cells + 4 * D)) + col;
                        cell_put(dst, a, t);
                        cell_put(dst + 1, c, t);
                        const int head = col / HS, jj = col - head * HS;
                        float* cr = p.kv.pool + kv_at(l, sec - 1, head, pos) + jj;
                        coherent_store(cr, a);
                        coherent_store(cr + 1, c);
                    }
                }
                item += stride;
                if (item < NQKV) load_qkv_operands<KD, PRO, MODERN>(p, w, item, pos, lane, qo);
            }
            stamp();

            // ===== phase B: attention of one head per workgroup (inference.cpp:211-225).
            // One compute unit fetches a head's cached rows at about 100 GB/s, which is what
            // a long context costs: beyond kAttnShareFrom positions the context of a head is
            // cut into shares of at most kAttnShare positions, the last (with the new position)
            // for the head's own workgroup and the others for the workgroups 16, 32, ... places
            // further on, which are idle in this phase.  They need q only, leave (maximum, sum,
            // 64 weighted sums) in cells, and the head's workgroup folds the shares in a fixed order.
            const int ctx = pos + 1;
            // (no more shares than the grid has groups of 16 workgroups: the head's own and G / 16 - 1 others)
            const int n_shares =
                ctx <= kAttnShareFrom ? 1 : min(min(kAttnMaxShares, G >> 4), (ctx + kAttnShare - 1) / kAttnShare);  // uniform
            const bool head_wg = wg < H;
            const bool share_wg = !head_wg && (wg & 15) < H && (wg >> 4) < n_shares;
            if (head_wg || share_wg) {
                const int hd = wg & 15;
                const int share = head_wg ? n_shares - 1 : (wg >> 4) - 1;
                float* qkv = ascr;         // [3][64]: q, key and value of the current position
                float* part = ascr + 192;  // [waves][4 lane groups][68]: m, l, pad, pad, acc[64]
                // this workgroup's positions [lo, hi); they are dealt to the wavefronts in
                // runs of `chunk` (a multiple of 4), walked 32 at a time
                const int span = (((ctx + n_shares - 1) / n_shares) + 3) & ~3;
                const int lo = share * span, hi = min(ctx, lo + span);
                const int chunk = (((hi - lo + kPersistWaves - 1) / kPersistWaves) + 3) & ~3;
                const int sub = lane >> 4, dl = lane & 15;
                const int t0 = lo + wave * chunk;
                Cell* share_cells = p.cells + ((6 * D + F + 2 + 9 * G + 2) & ~1);  // [H][15][66]
                // Cached rows do not depend on this step's q: the first 32 positions of
                // the run are fetched before waiting for q (all of it for contexts <= 256).
                const float* pool = p.kv.pool;
                float4 k4[8], v4[8];
#pragma unroll
                for (int it = 0; it < 8; it++) {
                    const int tt = t0 + it * 4 + sub;
                    k4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
                    v4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (it * 4 < chunk && tt < min(pos, hi)) {
                        const unsigned ko = static_cast<unsigned>(kv_at(l, 0, hd, tt)) + dl * 4;
                        const unsigned vo = static_cast<unsigned>(kv_at(l, 1, hd, tt)) + dl * 4;
                        k4[it] = *reinterpret_cast<const float4*>(pool + ko);
                        v4[it] = *reinterpret_cast<const float4*>(pool + vo);
                    }
                }
                // q, new key, new value of this head: one wait for all three (a workgroup with
                // a share of older positions needs q alone)
                {
                    const unsigned t = tag_of(l, 0);
                    unsigned spins = 0;
                    bool failed = false;
                    if (tid < (head_wg ? 96 : 32)) {
                        const int seg = tid >> 5, j = (tid & 31) * 2;
                        const Cell* src = (seg == 0 ? (p.cells + 2 * D) : seg == 1 ? (p.cells + 3 * D) : (p.cells + 4 * D)) + hd * HS;
                        const __amdgpu_buffer_rsrc_t rs = make_buffer(src, HS * 8u);
                        for (;;) {
                            const v4i w = coherent_load16(rs, static_cast<unsigned>(j) * 8u);
                            qkv[seg * 64 + j] = __int_as_float(w.x);
                            qkv[seg * 64 + j + 1] = __int_as_float(w.z);
                            if (w.y == static_cast<int>(t) && w.w == static_cast<int>(t)) break;
                            ++spins;
                            if (spins > p.spin_limit
                                || ((spins & 63u) == 0u
                                    && __hip_atomic_load(&p.ctl->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
                                failed = true;
                                break;
                            }
                        }
                    }
                    if (any_abandoned(failed)) {
                        if (tid == 0) {
                            __hip_atomic_store(&p.ctl->where, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            __hip_atomic_store(&p.ctl->abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                        return;
                    }
                }
                const float4 q4 = reinterpret_cast<const float4*>(qkv)[dl];
                float m = -INFINITY, lsum = 0.0f;
                float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
                // Batches of 8 iterations (32 positions); softmax state is merged online.
                for (int batch = 0; batch * 32 < chunk; batch++) {
                    if (batch >= 1) {
#pragma unroll
                        for (int it = 0; it < 8; it++) {
                            const int tt = t0 + batch * 32 + it * 4 + sub;
                            k4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
                            v4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
                            if (batch * 32 + it * 4 < chunk && tt < min(pos, hi)) {
                                const unsigned ko = static_cast<unsigned>(kv_at(l, 0, hd, tt)) + dl * 4;
                                const unsigned vo = static_cast<unsigned>(kv_at(l, 1, hd, tt)) + dl * 4;
                                k4[it] = *reinterpret_cast<const float4*>(pool + ko);
                                v4[it] = *reinterpret_cast<const float4*>(pool + vo);
                            }
                        }
                    }
                    float sc[8];
#pragma unroll
                    for (int it = 0; it < 8; it++) {
                        const int rel = batch * 32 + it * 4 + sub;
                        const int tt = t0 + rel;
                        const bool in_run = rel < chunk;
                        if (in_run && tt == pos) {
                            k4[it] = reinterpret_cast<const float4*>(qkv + 64)[dl];
                            v4[it] = reinterpret_cast<const float4*>(qkv + 128)[dl];
                        }
                        const float sdot = row16_sum(dot4(q4, k4[it]));
                        sc[it] = (in_run && tt < hi) ? sdot * 0.125f : -INFINITY;  // 1/sqrt(64)
                    }
                    float mb = sc[0];
#pragma unroll
                    for (int it = 1; it < 8; it++) mb = fmaxf(mb, sc[it]);
                    // the four position groups of the wavefront share one running maximum
                    mb = fmaxf(mb, dpp_move<0x142, 0xA>(mb, mb));
                    mb = fmaxf(mb, dpp_move<0x143, 0xC>(mb, mb));
                    mb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mb), 63));
                    const float mn = fmaxf(m, mb);
                    if (mn > -INFINITY) {
                        // The 16 lanes of a position group hold the same eight scores and the
                        // same running maximum.  Lane dl forms one exponential, that of score
                        // dl (lane 8: of the old maximum, the rescaling factor), and the group
                        // shares them by row broadcasts: one exponential per lane and batch
                        // instead of nine, with the same values.
                        float arg = sc[0];
#pragma unroll
                        for (int it = 1; it < 8; it++) arg = (dl == it) ? sc[it] : arg;
                        arg = (dl == 8) ? m : arg;
                        const float em = expf(arg - mn);  // exp(-inf) = 0: unused slots, first batch
                        const float f = row_lane<8>(em);
                        lsum *= f;
                        acc.x *= f;
                        acc.y *= f;
                        acc.z *= f;
                        acc.w *= f;
                        const float e[8] = {row_lane<0>(em), row_lane<1>(em), row_lane<2>(em), row_lane<3>(em),
                                            row_lane<4>(em), row_lane<5>(em), row_lane<6>(em), row_lane<7>(em)};
#pragma unroll
                        for (int it = 0; it < 8; it++) {
                            lsum += e[it];
                            acc.x += e[it] * v4[it].x;
                            acc.y += e[it] * v4[it].y;
                            acc.z += e[it] * v4[it].z;
                            acc.w += e[it] * v4[it].w;
                        }
                        m = mn;
                    }
                }
                // The four lane groups of a wavefront (16 lanes = one position slot each)
                // share its running maximum: their sums are added across the groups, and
                // the wavefront leaves one share.
                lsum += __shfl_xor(lsum, 16, kWave);
                acc.x += __shfl_xor(acc.x, 16, kWave);
                acc.y += __shfl_xor(acc.y, 16, kWave);
                acc.z += __shfl_xor(acc.z, 16, kWave);
                acc.w += __shfl_xor(acc.w, 16, kWave);
                lsum += __shfl_xor(lsum, 32, kWave);
                acc.x += __shfl_xor(acc.x, 32, kWave);
                acc.y += __shfl_xor(acc.y, 32, kWave);
                acc.z += __shfl_xor(acc.z, 32, kWave);
                acc.w += __shfl_xor(acc.w, 32, kWave);
                float* mine = part + wave * 68;  // m, l, pad, pad, acc[64]
                if (sub == 0) {
                    reinterpret_cast<float4*>(mine + 4)[dl] = acc;
                    if (dl == 0) {
                        mine[0] = m;
                        mine[1] = lsum;
                    }
                }
                __syncthreads();
                float M = -INFINITY, Lsum = 0.0f, o = 0.0f;
                if (tid < HS) {
#pragma unroll
                    for (int w8 = 0; w8 < kPersistWaves; w8++) M = fmaxf(M, part[w8 * 68]);
                    // one exponential per lane (wavefront lane % 8's), read across by all
                    static_assert(kPersistWaves == 8, "lane % 8 picks a wavefront");
                    const float fmine = expf(part[(tid & 7) * 68] - M);  // 0 for wavefronts without positions
#pragma unroll
                    for (int w8 = 0; w8 < kPersistWaves; w8++) {
                        const float f = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fmine), w8));
                        Lsum += part[w8 * 68 + 1] * f;
                        o += part[w8 * 68 + 4 + tid] * f;
                    }
                }
                if (share_wg) {
                    // this share's maximum, sum and weighted sums, for the head's workgroup
                    if (tid < HS) {
                        Cell* mine_c = share_cells + (hd * (kAttnMaxShares - 1) + share) * 66;
                        const unsigned t = tag_of(l, 5);
                        cell_put(mine_c + 2 + tid, o, t);
                        if (tid == 0) {
                            cell_put(mine_c, M, t);
                            cell_put(mine_c + 1, Lsum, t);
                        }
                    }
                } else if (n_shares > 1) {
                    // the other shares, then the fold in share order with this one last
                    __syncthreads();  // part[] is read; it takes the shares now
                    if (!gather_cells(share_cells + hd * (kAttnMaxShares - 1) * 66, (n_shares - 1) * 66, tag_of(l, 5), part, p)) return;
                    if (tid < HS) {
                        float Mall = M;
                        for (int j = 0; j < n_shares - 1; j++) Mall = fmaxf(Mall, part[j * 66]);
                        float Lall = 0.0f, oall = 0.0f;
                        for (int j = 0; j < n_shares - 1; j++) {
                            const float f = expf(part[j * 66] - Mall);
                            Lall += part[j * 66 + 1] * f;
                            oall += part[j * 66 + 2 + tid] * f;
                        }
                        const float f = expf(M - Mall);
                        Lall += Lsum * f;
                        oall += o * f;
                        cell_put((p.cells + 5 * D) + hd * HS + tid, oall * (1.0f / Lall), tag_of(l, 1));
                    }
                } else if (tid < HS) {
                    cell_put((p.cells + 5 * D) + hd * HS + tid, o * (1.0f / Lsum), tag_of(l, 1));
                }
                __syncthreads();
            }
            stamp();

            // FFN1's operands (phase D).  Workgroups without a head spend phase C waiting
            // for the attention of the others while HBM idles: their wavefronts that have no
            // W_o row request the FFN1 rows now.  (The loads of a wavefront return in
            // order, so its polls of phase C queue behind these rows; that wait is the
            // long one anyway.  Workgroups with a head are late already and fetch as before.)
            constexpr int NIT = MODERN ? F : F / 2;  // pairs of weight rows
            float4 fw0[KD], fw1[KD];
            NormRegs<KD> n2;
            float fb0 = 0.0f, fb1 = 0.0f;
#pragma unroll
            for (int i = 0; i < KD; i++) {
                fw0[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                fw1[i] = fw0[i];
                n2.g[i] = fw0[i];
                n2.b[i] = fw0[i];
            }
            auto load_ffn1 = [&]() {
                if (first < NIT) {
                    load_row<KD>(w.w1, 2 * first, D, lane, fw0);
                    load_row<KD>(w.w1, 2 * first + 1, D, lane, fw1);
                    load_norm<KD, PRO>(w.g2, w.be2, lane, n2);
                    if (!MODERN) {
                        fb0 = w.b1[2 * first];
                        fb1 = w.b1[2 * first + 1];
                    }
                }
            };
            const bool early_ffn1 = wave >= (D + G - 1) / G && wg >= H;
            if (early_ffn1) load_ffn1();
            // With FFN2 rows of more than 8 KB (hidden widths above 2048) the same idle
            // wavefronts also bring the FFN2 rows of this workgroup's first three wavefronts
            // into this XCD's L2 (one float per 128-byte line touches a whole row), and those
            // of a workgroup with a head on the same XCD, which has no idle time of its own:
            // the rows are then a trip to the L2, not to HBM, when the FFN2 phase asks for
            // them two exchanges later.  Measured on one box, us per token: hidden 3072
            // (d768 GPT-2) 131.9 -> 124.7; at hidden 2048 it does not pay (Modern d768
            // 115.9 -> 117.7, GPT-2 d512 77.6 -> 77.5), so those shapes go without.
            // A workgroup with a head comes out of the attention phase last and then has its
            // W_o, FFN1 and FFN2 rows still to fetch from HBM, while every other workgroup
            // waits for its outputs.  The workgroup 16 places further on (same XCD: workgroups
            // go round-robin over 8) spends the attention phase idle; its wavefronts without a
            // W_o row touch one float per 128-byte line of those rows, which brings them into
            // the L2 the head workgroup will ask.  Measured on one box, us per token: Modern
            // d768 119.4 -> 118.0, GPT-2 d512 77.6 -> 76.6; with a hidden width of 3072 the
            // helpers' own polls come too late behind all this and a token took 9.6 us longer,
            // so wide shapes only get the touch below.
            if (F <= 2048 && early_ffn1 && wg - 16 >= 0 && wg - 16 < H) {
                const int other = wg - 16;
                const int hw = wave - (D + G - 1) / G;  // 0 .. 4
                float touched = 0.0f;
                constexpr int kLinesD = D / 32;          // 128-byte lines of a row of D floats
                const int ld = lane < kLinesD ? lane : 0;
                // W_o: up to three rows, one per helper wavefront
                {
                    const int row = other + G * hw;
                    if (hw < (D + G - 1) / G && row < D) touched += w.wo[static_cast<size_t>(row) * D + ld * 32];
                }
                // FFN1: the head workgroup's eight items of two rows each, dealt to the five helpers
                for (int wv = hw; wv < kPersistWaves; wv += kPersistWaves - (D + G - 1) / G) {
                    const int item = other + G * wv;
                    if (item < NIT) {
                        touched += w.w1[static_cast<size_t>(2 * item) * D + ld * 32];
                        touched += w.w1[static_cast<size_t>(2 * item + 1) * D + ld * 32];
                    }
                }
                // FFN2: up to three rows of F floats
                {
                    const int row = other + G * hw;
                    if (hw < (D + G - 1) / G && row < D) {
#pragma unroll
                        for (int part = 0; part < (F + 2047) / 2048; part++)
                            touched += w.w2[static_cast<size_t>(row) * F + (part * 2048 + lane * 32) % F];
                    }
                }
                asm volatile("" ::"v"(touched));
            }
            if constexpr (F > 2048) {
                if (early_ffn1 && wave < 2 * ((D + G - 1) / G)) {
                    const int w3 = wave - (D + G - 1) / G;  // the wavefront whose row this one touches
                    const int row = wg + G * w3;
                    float touched = 0.0f;
                    if (row < D) {
                        touched += w.w2[static_cast<size_t>(row) * F + lane * 32];
                        touched += w.w2[static_cast<size_t>(row) * F + (2048 + lane * 32) % F];
                    }
                    const int other = wg - 16;  // same XCD (workgroups go round-robin over 8)
                    if (other >= 0 && other < H) {
                        const int row2 = other + G * w3;
                        if (row2 < D) {
                            touched += w.w2[static_cast<size_t>(row2) * F + lane * 32];
                            touched += w.w2[static_cast<size_t>(row2) * F + (2048 + lane * 32) % F];
                        }
                    }
                    asm volatile("" ::"v"(touched));
                }
            }

            // ===== phase C: x += b_o + attn @ W_o
            {
                float4 w0[KD];
                float bo = 0.0f;
                // idle wavefronts get defined (zero) operands: values left undefined on
                // one path make the register allocator spill them on the other
                if (first < D) {
                    load_row<KD>(w.wo, first, D, lane, w0);
                    bo = w.bo[first];
                } else {
#pragma unroll
                    for (int i = 0; i < KD; i++) w0[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
                if (!gather_cells((p.cells + 5 * D), D, tag_of(l, 1), vin, p)) return;
                for (int row = first; row < D; ) {
                    const float a = dot_row_lds<KD>(w0, vin, lane);
                    if (lane == 0) cell_put((p.cells + D) + row, (xs[row] + bo) + a, tag_of(l, 2));
                    row += stride;
                    if (row < D) {
                        load_row<KD>(w.wo, row, D, lane, w0);
                        bo = w.bo[row];
                    }
                }
            }
            stamp();

            // ===== phase D: norm2 + FFN1 (SwiGLU or GELU) -> hidden cells
            {
                if (!early_ffn1) load_ffn1();
                __syncthreads();  // every wave is done reading xs (phase C)
                if (!gather_cells((p.cells + D), D, tag_of(l, 2), xs, p)) return;
                for (int item = first; item < NIT; ) {
                    float4 h[KD];
                    load_input<KD, PRO>(xs, n2, lane, h);
                    const float a = dot_row<KD>(fw0, h);
                    const float c = dot_row<KD>(fw1, h);
                    if (lane == 0) {
                        const unsigned t = tag_of(l, 3);
                        if (MODERN) {
                            cell_put((p.cells + 6 * D) + item, c * silu(a), t);
                        } else {
                            cell_put((p.cells + 6 * D) + 2 * item, gelu_tanh(a + fb0), t);
                            cell_put((p.cells + 6 * D) + 2 * item + 1, gelu_tanh(c + fb1), t);
                        }
                    }
                    item += stride;
                    if (item < NIT) {
                        load_row<KD>(w.w1, 2 * item, D, lane, fw0);
                        load_row<KD>(w.w1, 2 * item + 1, D, lane, fw1);
                        if (!MODERN) {
                            fb0 = w.b1[2 * item];
                            fb1 = w.b1[2 * item + 1];
                        }
                    }
                }
            }
            stamp();

            // ===== phase E: x += (b2 +) hidden @ W2 -> next layer's input cells
            {
                float4 w0[KF];
                float b2 = 0.0f;
                if (first < D) {
                    load_row<KF>(w.w2, first, F, lane, w0);
                    if (!MODERN) b2 = w.b2[first];
                } else {
#pragma unroll
                    for (int i = 0; i < KF; i++) w0[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
                if (!gather_cells((p.cells + 6 * D), F, tag_of(l, 3), vin, p)) return;
                for (int row = first; row < D; ) {
                    const float a = dot_row_lds<KF>(w0, vin, lane);
                    if (lane == 0) cell_put(p.cells + row, (xs[row] + b2) + a, tag_of(l, 4));
                    row += stride;
                    if (row < D) {
                        load_row<KF>(w.w2, row, F, lane, w0);
                        if (!MODERN) b2 = w.b2[row];
                    }
                }
            }
            stamp();

            // ===== the next consumer of x is layer l+1's QKV: its operands are
            // fetched while x is still being exchanged.
            if (l + 1 < L) {
                const LayerPtrs wn = layer_at<KD, KF, MODERN>(p.layer0, l + 1);
                if (has_qkv) load_qkv_operands<KD, PRO, MODERN>(p, wn, first, pos, lane, qo);
                else qo = QkvOperands<KD, PRO>{};
                __syncthreads();  // xs is overwritten next
                if (!gather_cells(p.cells, D, tag_of(l, 4), xs, p)) return;
            }
        }

        if (want_logits) {
            // ===== final norm + logits = h @ E^T (inference.cpp:251-254); the rows of
            // E are fetched while the last layer's x is still being exchanged.
            const int nitems = (V + RL - 1) / RL;
            float4 wr[RL][KD];
            NormRegs<KD> nf;
            load_norm<KD, PRO>(p.gf, p.bf, lane, nf);
            // every wavefront fetches: rows past the end are clamped here and skipped on
            // store (a conditional fetch makes the compiler spill the rows to scratch)
#pragma unroll
            for (int r = 0; r < RL; r++) load_row<KD>(p.E, min(first * RL + r, V - 1), D, lane, wr[r]);
            // A pick every workgroup makes itself follows: beside the rows go this workgroup's
            // largest penalised logit and its first index (greedy) or its four largest
            // penalised, scaled logits with their indices and the value of the fifth (top-k).
            // logits_with_penalty (text_gen.cpp:14-33) counts once per occurrence in the last
            // 50 tokens, which every wavefront holds a lane each.
            const bool pick_next = (!FEED || !ended) && i_pick < p.n_picks && s + 1 >= p.n_prompt;
            const bool publish = (fast_greedy || fast_topk) && pick_next;
            int window = 0;
            int* win = reinterpret_cast<int*>(ascr) + 2 * kPersistWaves;  // [64] the window's tokens, in LDS
            float* mine8 = ascr + 2 * kPersistWaves + 64;                 // [64] the workgroup's values (top-k)
            unsigned stop_word = 0u;
            if (publish) {
                if (p.pick.penalty != 1.0f) {
                    const int n_hist = p.pick.n_hist + i_pick;
                    window = min(kPenaltyWindow, n_hist);
                    if (tid < window)
                        win[tid] = __hip_atomic_load(&p.hist[n_hist - window + tid], __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);
                }
                if constexpr (FEED) {
                    // the host's stop request: one trip over the bus behind the rows of E
                    if (wg == 0 && tid == 0)
                        stop_word = __hip_atomic_load(p.stop_request, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                }
            }
            const float inv_t = 1.0f / p.pick.temperature;
            float best = -INFINITY;
            int best_row = 0x7FFFFFFF;
            __syncthreads();
            if (!gather_cells(p.cells, D, tag_of(L - 1, 4), xs, p)) return;
            stamp();
            float4 h[KD];
            load_input<KD, PRO>(xs, nf, lane, h);
            auto emit = [&](int item, const float4 (&rows)[RL][KD]) {
                float out[RL];
#pragma unroll
                for (int r = 0; r < RL; r++) out[r] = dot_row<KD>(rows[r], h);
                if (publish) {
                    const int win_tok = lane < window ? win[lane] : -1;
#pragma unroll
                    for (int r = 0; r < RL; r++) {
                        const int row = item * RL + r;
                        float v = out[r];
                        if (window > 0) {
                            const int times = __popcll(__ballot(win_tok == row));
                            for (int c = 0; c < times; c++) v = (v > 0.0f) ? v / p.pick.penalty : v * p.pick.penalty;
                        }
                        if (fast_greedy) {
                            if (row < V && v > best) {  // rows ascend: the first maximum stays
                                best = v;
                                best_row = row;
                            }
                        } else if (lane == 0) {
                            v *= inv_t;  // text_gen.cpp:140-143
                            mine8[wave * RL + r] = (row < V && v == v) ? v : -INFINITY;
                        }
                    }
                }
                if (lane == 0) {
#pragma unroll
                    for (int r = 0; r < RL; r++) {
                        const int row = item * RL + r;
                        if (row < V) {
                            coherent_store(p.logits + row, out[r]);
                            if (p.logit_log) p.logit_log[static_cast<size_t>(s) * V + row] = out[r];
                        }
                    }
                }
            };
            // The first item uses the rows fetched ahead; later ones (vocabularies
            // beyond 8 rows per wavefront of the grid) fetch their own.
            emit(first, wr);  // rows past the end are clamped on load and skipped on store
            for (int item = first + stride; item < nitems; item += stride) {
                float4 wl[RL][KD];
#pragma unroll
                for (int r = 0; r < RL; r++) load_row<KD>(p.E, min(item * RL + r, V - 1), D, lane, wl[r]);
                emit(item, wl);
            }
            PTICK_BEGIN();
            if (publish) {
                const unsigned tt = ((p.epoch + static_cast<unsigned>(s + 1)) * static_cast<unsigned>(L + 1)
                                     + static_cast<unsigned>(L)) * 8u + 7u;
                Cell* pc = p.cells + 6 * D + F + 2;
                if (fast_greedy) {
                    if (lane == 0) {
                        ascr[wave] = best;
                        ascr[kPersistWaves + wave] = __int_as_float(best_row);
                    }
                    __syncthreads();
                    if (wave == 0) {
                        best = lane < kPersistWaves ? ascr[lane] : -INFINITY;
                        best_row = lane < kPersistWaves ? __float_as_int(ascr[kPersistWaves + lane]) : 0x7FFFFFFF;
                        first_max_step<0xB1, 0xF>(best, best_row);
                        first_max_step<0x4E, 0xF>(best, best_row);
                        first_max_step<0x141, 0xF>(best, best_row);  // lanes 0..7 hold the workgroup's pair
                    }
                    if (tid == 0) {
                        cell_put(pc + wg, best, tt);
                        cell_put(pc + G + wg, __int_as_float(best_row), tt);
                        if (wg == 0) cell_put(pc + 2 * G, __int_as_float(stop_word != 0u ? 1 : 0), tt);
                    }
                } else {
                    // Values [4 G], indices [4 G], the fifth value [G], the stop word.  A
                    // workgroup's j-th largest sits at (j / 2) * 2 G + 2 wg + j % 2: read as a row
                    // of 4 G by 2 G threads, two elements each, every second thread of every
                    // wavefront then holds a workgroup's maximum, which is what keeps the
                    // sampler's first threshold close to the k-th largest.  Wavefront 0 takes
                    // the largest five times (equal values: the lower row, which is the lower lane).
                    __syncthreads();
                    if (wave == 0) {
                        float rest = mine8[lane];
                        const int row = (wg + G * (lane >> 3)) * RL + (lane & 7);
#pragma unroll
                        for (int j = 0; j < 5; j++) {
                            const float sel = wave_max(rest);
                            const unsigned long long at = __ballot(rest == sel);
                            if (lane == __ffsll(static_cast<long long>(at)) - 1) {
                                if (j < 4) {
                                    Cell* c = pc + (j >> 1) * 2 * G + 2 * wg + (j & 1);
                                    cell_put(c, sel, tt);
                                    cell_put(c + 4 * G, __int_as_float(row), tt);
                                } else {
                                    cell_put(pc + 8 * G + wg, sel, tt);
                                }
                                rest = -INFINITY;
                            }
                        }
                        if (wg == 0 && lane == 0) cell_put(pc + 9 * G, __int_as_float(stop_word != 0u ? 1 : 0), tt);
                    }
                }
                pairs_out = true;
                PTICK(8);
            }
            // This workgroup's rows are out: signal.  The count follows the rows for the
            // picker that reads them back; in a launch of greedy picks nobody does.
            if (!fast_greedy) {
                __builtin_amdgcn_s_waitcnt(0);
                __syncthreads();
            }
            arrive_gen++;
            if (tid == 0)
                __hip_atomic_fetch_add(&p.ctl->arrive[(wg & 15) * 32], 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        } else {
            // nobody needs this step's logits: the last x stays in its cells
            stamp();
        }
        stamp();
    }
}

}  // namespace gh

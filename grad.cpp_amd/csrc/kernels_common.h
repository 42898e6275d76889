// Shared device-side definitions for the gfx950 decode kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace gh {

constexpr int kWave = 64;
constexpr float kNormEps = 1e-5f;  // include/grad/transformer/layer_norm.h:18

// Per-session counters that live in device memory so that a recorded step
// graph can be replayed without changing kernel arguments.
struct DevState {
    int pos;     // positions already in the cache (shared by all sequences)
    int n_hist;  // tokens in each sequence's history (prompt + picks)
    int picks;   // picks made so far (index of the next uniform draw)
    int pad;
};

// Paged KV cache.  pool is [layers][n_pages][2 (K,V)][heads][page_tokens][head_size];
// page_table is [batch][pages_per_seq] physical page numbers.  One (page, K|V,
// head) run is page_tokens * head_size contiguous floats, so a head's keys for
// consecutive positions stream as whole cache lines.
struct KvLayout {
    float* pool;
    const int* page_table;
    int n_pages;
    int pages_per_seq;
    int heads;
    int head_size;
    int page_shift;  // page_tokens == 1 << page_shift
};

__device__ __forceinline__ size_t kv_offset(const KvLayout& kv, int layer, int seq, int which,
                                            int head, int t) {
    const int page = kv.page_table[seq * kv.pages_per_seq + (t >> kv.page_shift)];
    const int slot = t & ((1 << kv.page_shift) - 1);
    const size_t run = (((static_cast<size_t>(layer) * kv.n_pages + page) * 2 + which) * kv.heads
                        + head);
    return ((run << kv.page_shift) + slot) * kv.head_size;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Block-wide reductions through a small LDS scratch (one float per wave).
// Every thread of the block must call them; all threads get the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = 0.0f;
    for (int w = 0; w < nw; w++) r += scratch[w];
    return r;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = scratch[0];
    for (int w = 1; w < nw; w++) r = fmaxf(r, scratch[w]);
    return r;
}

__device__ __forceinline__ float dot4(const float4& a, const float4& b) {
    return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}

// inference.cpp:69-80
__device__ __forceinline__ float gelu_tanh(float x) {
    const float t = tanhf(0.79788456f * (x + 0.044715f * x * x * x));
    return 0.5f * x * (1.0f + t);
}

// inference.cpp:82-91
__device__ __forceinline__ float silu(float x) { return x / (1.0f + expf(-x)); }

}  // namespace gh

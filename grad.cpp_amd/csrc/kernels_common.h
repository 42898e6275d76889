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
    int hist_lead;  // n_hist - pos when the next pick is made (0 in a decode loop: the pick lands at hist[pos])
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

// Device-scope ("sc1") vector loads through a buffer descriptor.  They see data
// other workgroups of a running kernel wrote with device-scope stores, like an
// atomic load does, but several can be in flight at once.  Reads past the end
// of the buffer return zero.
typedef int v4i __attribute__((ext_vector_type(4)));
constexpr int kAuxDeviceScope = 16;  // sc1 on gfx94x / gfx950 buffer instructions

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

__device__ __forceinline__ v4i coherent_load16(__amdgpu_buffer_rsrc_t rs, unsigned byte_offset) {
    return __builtin_amdgcn_raw_buffer_load_b128(rs, byte_offset, 0, kAuxDeviceScope);
}

// Wavefront reductions on the data-parallel-primitive (DPP) path: lane
// permutations inside the ALU instead of trips through the LDS crossbar.
// Four steps fold each row of 16 lanes, two row broadcasts fold the four rows
// into lane 63, and a scalar read hands the result to every lane.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v, float fill) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), CTRL,
                                                      ROW_MASK, 0xF, false));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1, 0xF>(v, 0.0f);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xF>(v, 0.0f);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xF>(v, 0.0f);  // row_half_mirror
    v += dpp_move<0x140, 0xF>(v, 0.0f);  // row_mirror
    v += dpp_move<0x142, 0xA>(v, 0.0f);  // row_bcast:15 into rows 1 and 3
    v += dpp_move<0x143, 0xC>(v, 0.0f);  // row_bcast:31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1, 0xF>(v, v));
    v = fmaxf(v, dpp_move<0x4E, 0xF>(v, v));
    v = fmaxf(v, dpp_move<0x141, 0xF>(v, v));
    v = fmaxf(v, dpp_move<0x140, 0xF>(v, v));
    v = fmaxf(v, dpp_move<0x142, 0xA>(v, v));
    v = fmaxf(v, dpp_move<0x143, 0xC>(v, v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// The largest value of a wavefront and, among equal ones, the lowest index that came
// with it: the same six steps on a (value, index) pair.  Every lane returns the result.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void first_max_step(float& v, int& i) {
    const float ov = dpp_move<CTRL, ROW_MASK>(v, v);
    const int oi = __builtin_amdgcn_update_dpp(i, i, CTRL, ROW_MASK, 0xF, false);
    if (ov > v || (ov == v && oi < i)) {
        v = ov;
        i = oi;
    }
}

__device__ __forceinline__ void wave_first_max(float& v, int& i) {
    first_max_step<0xB1, 0xF>(v, i);
    first_max_step<0x4E, 0xF>(v, i);
    first_max_step<0x141, 0xF>(v, i);
    first_max_step<0x140, 0xF>(v, i);
    first_max_step<0x142, 0xA>(v, i);
    first_max_step<0x143, 0xC>(v, i);
    v = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
    i = __builtin_amdgcn_readlane(i, 63);
}

// Running total over the lanes of a wavefront, this lane's own value included:
// shifts inside each row of 16, then the totals of the rows before.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_move_int(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xF, false);  // lanes without a source get 0
}

__device__ __forceinline__ int wave_inclusive_scan(int v) {
    v += dpp_move_int<0x111, 0xF>(v);  // row_shr:1
    v += dpp_move_int<0x112, 0xF>(v);  // row_shr:2
    v += dpp_move_int<0x114, 0xF>(v);  // row_shr:4
    v += dpp_move_int<0x118, 0xF>(v);  // row_shr:8
    v += dpp_move_int<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_move_int<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

// Lane N of every row of 16 lanes, handed to all lanes of that row.
template <int N>
__device__ __forceinline__ float row_lane(float v) {
    static_assert(N >= 0 && N < 16, "a row has 16 lanes");
    return dpp_move<0x150 + N, 0xF>(v, 0.0f);  // row_newbcast:N
}

// Block-wide reductions through a small LDS scratch (one float per wave).
// Every thread of the block must call them; all threads get the result.
// nt: threads of the workgroup; a caller that knows it at compile time passes it
// (blockDim.x is a load from the dispatch packet).
__device__ __forceinline__ float block_sum(float v, float* scratch, int nt = blockDim.x) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (nt + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = 0.0f;
    for (int w = 0; w < nw; w++) r += scratch[w];
    return r;
}

__device__ __forceinline__ float block_max(float v, float* scratch, int nt = blockDim.x) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (nt + 63) >> 6;
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

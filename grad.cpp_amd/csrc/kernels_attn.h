// Decode attention for one new position per sequence over the paged KV cache:
// scores, softmax and the weighted sum of V for one (sequence, head, chunk of
// positions) per workgroup.  Long contexts are cut into chunks; the last
// workgroup to finish a (sequence, head) merges the chunk results.
//
// Restates the per-head loop of src/transformer/inference.cpp:211-225 and
// softmax_row (:60-67).
#pragma once

#include "kernels_common.h"

namespace gh {

struct AttnParams {
    const float* q;  // [batch][d_model], already rotated
    float* out;      // [batch][d_model]
    KvLayout kv;
    int layer;
    int d_model;
    const DevState* st;
    int chunk;       // positions per workgroup
    int max_chunks;  // grid.x
    float scale;     // 1 / sqrt(head_size)
    float* part;     // [batch][heads][max_chunks][head_size + 2]: m, l, acc
    unsigned* tickets;  // [batch][heads], zero between launches
};

// Merges chunk partials (running max m, sum l, unnormalised acc) of one head.
__device__ __forceinline__ void attn_merge(const AttnParams& p, int b, int h, int nchunk, int hs) {
    const float* base = p.part + (static_cast<size_t>(b) * p.kv.heads + h) * p.max_chunks * (hs + 2);
    float M = -INFINITY;
    for (int s = 0; s < nchunk; s++) M = fmaxf(M, base[s * (hs + 2)]);
    float L = 0.0f;
    for (int s = 0; s < nchunk; s++) L += base[s * (hs + 2) + 1] * expf(base[s * (hs + 2)] - M);
    const float inv = 1.0f / L;
    for (int j = threadIdx.x; j < hs; j += blockDim.x) {
        float o = 0.0f;
        for (int s = 0; s < nchunk; s++)
            o += base[s * (hs + 2) + 2 + j] * expf(base[s * (hs + 2)] - M);
        p.out[static_cast<size_t>(b) * p.d_model + h * hs + j] = o * inv;
    }
}

// HS: head size, a power of two in [4, 256].  HS/4 lanes hold one position's
// row as float4s, so a wavefront reads 64*4 consecutive floats of the page.
// HS == 0 is the any-head-size path (one lane per position, one lane per output).
template <int HS>
__global__ __launch_bounds__(256) void attn_decode_kernel(const AttnParams p) {
    extern __shared__ float smem[];
    float* sc = smem;                 // [chunk] scores -> probabilities
    float* red = smem + p.chunk;      // [waves * head_size] + 8 reduction scratch
    const int hs = HS > 0 ? HS : p.kv.head_size;
    const int ck = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int ctx = p.st->pos + 1;
    const int nchunk = (ctx + p.chunk - 1) / p.chunk;
    if (ck >= nchunk) return;
    const int t0 = ck * p.chunk;
    const int n = min(ctx, t0 + p.chunk) - t0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    float* scratch = red + nw * hs;
    const float* qh = p.q + static_cast<size_t>(b) * p.d_model + h * hs;

    // ---- scores: s_t = dot(q_h, K[t,h]) * scale (inference.cpp:215-217)
    if constexpr (HS > 0) {
        constexpr int LPP = HS / 4, PPW = 64 / LPP;
        const int sub = lane / LPP, dl = lane % LPP;
        const float4 q4 = reinterpret_cast<const float4*>(qh)[dl];
        for (int base = wave * PPW; base < n; base += nw * PPW) {
            const int i = base + sub;
            float s = 0.0f;
            if (i < n) {
                const float4 k4 = *reinterpret_cast<const float4*>(
                    p.kv.pool + kv_offset(p.kv, p.layer, b, 0, h, t0 + i) + dl * 4);
                s = dot4(q4, k4);
            }
#pragma unroll
            for (int o = LPP / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
            if (dl == 0 && i < n) sc[i] = s * p.scale;
        }
    } else {
        for (int i = tid; i < n; i += blockDim.x) {
            const float* kr = p.kv.pool + kv_offset(p.kv, p.layer, b, 0, h, t0 + i);
            float s = 0.0f;
            for (int j = 0; j < hs; j++) s += qh[j] * kr[j];
            sc[i] = s * p.scale;
        }
    }
    __syncthreads();

    // ---- softmax over the chunk (softmax_row, inference.cpp:60-67)
    float m = -INFINITY;
    for (int i = tid; i < n; i += blockDim.x) m = fmaxf(m, sc[i]);
    m = block_max(m, scratch);
    float l = 0.0f;
    for (int i = tid; i < n; i += blockDim.x) {
        const float e = expf(sc[i] - m);
        sc[i] = e;
        l += e;
    }
    l = block_sum(l, scratch);
    const bool single = nchunk == 1;
    if (single) {
        const float inv = 1.0f / l;
        for (int i = tid; i < n; i += blockDim.x) sc[i] *= inv;
    }
    __syncthreads();

    // ---- out_h = sum_t p_t * V[t,h] (inference.cpp:220-224)
    if constexpr (HS > 0) {
        constexpr int LPP = HS / 4, PPW = 64 / LPP;
        const int sub = lane / LPP, dl = lane % LPP;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int i = wave * PPW + sub; i < n; i += nw * PPW) {
            const float pt = sc[i];
            const float4 v4 = *reinterpret_cast<const float4*>(
                p.kv.pool + kv_offset(p.kv, p.layer, b, 1, h, t0 + i) + dl * 4);
            acc.x += pt * v4.x;
            acc.y += pt * v4.y;
            acc.z += pt * v4.z;
            acc.w += pt * v4.w;
        }
#pragma unroll
        for (int o = LPP; o < 64; o <<= 1) {
            acc.x += __shfl_xor(acc.x, o, kWave);
            acc.y += __shfl_xor(acc.y, o, kWave);
            acc.z += __shfl_xor(acc.z, o, kWave);
            acc.w += __shfl_xor(acc.w, o, kWave);
        }
        if (sub == 0) reinterpret_cast<float4*>(red + wave * HS)[dl] = acc;
    } else {
        // one thread per output dim, all positions of the chunk; waves are not split.
        for (int j = tid; j < hs; j += blockDim.x) {
            float a = 0.0f;
            for (int i = 0; i < n; i++)
                a += sc[i] * p.kv.pool[kv_offset(p.kv, p.layer, b, 1, h, t0 + i) + j];
            red[j] = a;
        }
    }
    __syncthreads();

    const int nred = HS > 0 ? nw : 1;
    if (single) {
        for (int j = tid; j < hs; j += blockDim.x) {
            float o = 0.0f;
            for (int w = 0; w < nred; w++) o += red[w * hs + j];
            p.out[static_cast<size_t>(b) * p.d_model + h * hs + j] = o;
        }
        return;
    }

    float* mine = p.part
                  + ((static_cast<size_t>(b) * p.kv.heads + h) * p.max_chunks + ck) * (hs + 2);
    for (int j = tid; j < hs; j += blockDim.x) {
        float o = 0.0f;
        for (int w = 0; w < nred; w++) o += red[w * hs + j];
        mine[2 + j] = o;
    }
    if (tid == 0) {
        mine[0] = m;
        mine[1] = l;
    }
    // Publish the partial, then take a ticket; the last chunk to arrive merges.
    __threadfence();
    __syncthreads();
    __shared__ unsigned ticket;
    if (tid == 0) ticket = atomicAdd(&p.tickets[b * p.kv.heads + h], 1u);
    __syncthreads();
    if (ticket != static_cast<unsigned>(nchunk - 1)) return;
    __threadfence();
    attn_merge(p, b, h, nchunk, hs);
    if (tid == 0) p.tickets[b * p.kv.heads + h] = 0u;
}

}  // namespace gh

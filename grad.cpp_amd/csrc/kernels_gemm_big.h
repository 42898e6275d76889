// Projections over many rows (a prompt pass: hundreds to tens of thousands of
// token rows): C[M,N] = A[M,K] . Wt[N,K]^T on the fp32 matrix cores with the
// classic compute-bound tiling — one workgroup owns a 128 x 128 tile of C, its
// four wavefronts 64 x 64 each (four accumulator tiles of 32 x 32, products
// v_mfma_f32_32x32x2_f32: 730 k tok/s on the 16 x 1536-token prompt pass against
// 711 k with sixteen 16 x 16 tiles and the 16x16x4 product, same LDS reads, half
// the product instructions), and A and W travel through LDS in K-steps of 16,
// double buffered, fetched with row-contiguous 16-byte loads.  The 64-row decode kernel (gemm16_kernel) is
// bound by latency and wants many small tiles; here the arithmetic is the bound
// and every fetched element is reused 64 times from LDS.
//
// The same prologue and epilogues as the other projection kernels: RMSNorm is
// folded in (gamma on the way into LDS, the row's sum of squares from the same
// loads, 1/rms on the finished dot product; layer_norm_row, inference.cpp:33-43)
// and gemv_epilogue<EPI> consumes column pairs of a row.
#pragma once

#include "kernels_gemm.h"

namespace gh {

constexpr int kBigTile = 128;       // rows and columns of C per workgroup
constexpr int kBigK = 16;           // K-step
constexpr int kBigLd = kBigK + 4;   // LDS row stride of a staged tile (floats): conflict-free float4 access
constexpr int kBigCLd = kBigTile + 4;  // LDS row stride of the finished tile
constexpr int kBigThreads = 256;
constexpr size_t kBigLdsBytes = static_cast<size_t>(kBigTile) * kBigCLd * sizeof(float) + kBigTile * sizeof(float);

template <int EPI, bool RMS>
__global__ __launch_bounds__(kBigThreads) void gemm128_kernel(const GemvParams p, int M, int n_tiles) {
    extern __shared__ __attribute__((aligned(128))) float lds_big[];
    // staging: [2 buffers][A | W][128][kBigLd]; after the K loop the same memory
    // holds the finished tile [128][kBigCLd] and the row scales [128]
    float* stage = lds_big;
    float* ctile = lds_big;
    float* row_scale = lds_big + kBigTile * kBigCLd;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // 64 x 64 quadrant of the tile
    const int m_tile = blockIdx.x / n_tiles, n_tile = blockIdx.x - m_tile * n_tiles;
    const int m0 = m_tile * kBigTile, n0 = n_tile * kBigTile;
    const int K = p.K;

    // fetch assignment: thread t brings rows t/4 and t/4 + 64, 16-byte chunk t%4 of each
    const int fr = tid >> 2, fc = tid & 3;
    const float* a_src0 = p.in + static_cast<size_t>(min(m0 + fr, M - 1)) * p.in_stride + fc * 4;
    const float* a_src1 = p.in + static_cast<size_t>(min(m0 + fr + 64, M - 1)) * p.in_stride + fc * 4;
    const float* w_src0 = p.W + static_cast<size_t>(min(n0 + fr, p.N - 1)) * K + fc * 4;
    const float* w_src1 = p.W + static_cast<size_t>(min(n0 + fr + 64, p.N - 1)) * K + fc * 4;
    const float* g_src = RMS ? p.gamma + fc * 4 : nullptr;
    const int stash_at = fr * kBigLd + fc * 4;  // this thread's float4 slot in a staged tile (second row: + 64 rows)

    typedef float v16f __attribute__((ext_vector_type(16)));
    v16f acc32[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc32[a][b][r] = 0.0f;
    const int i32 = lane & 31, h32 = lane >> 5;
    float ss0 = 0.0f, ss1 = 0.0f;

    float4 ra0, ra1, rw0, rw1, rg = make_float4(1.f, 1.f, 1.f, 1.f);
#define GH_BIG_FETCH(k)                                                  \
    ra0 = *reinterpret_cast<const float4*>(a_src0 + (k));               \
    ra1 = *reinterpret_cast<const float4*>(a_src1 + (k));               \
    rw0 = *reinterpret_cast<const float4*>(w_src0 + (k));               \
    rw1 = *reinterpret_cast<const float4*>(w_src1 + (k));               \
    if (RMS) rg = *reinterpret_cast<const float4*>(g_src + (k));
#define GH_BIG_STASH(buf)                                                                          \
    {                                                                                              \
        float* as_ = stage + (buf) * (2 * kBigTile * kBigLd);                                      \
        float* ws_ = as_ + kBigTile * kBigLd;                                                      \
        if (RMS) {                                                                                 \
            ss0 += dot4(ra0, ra0);                                                                 \
            ss1 += dot4(ra1, ra1);                                                                 \
            ra0 = make_float4(ra0.x * rg.x, ra0.y * rg.y, ra0.z * rg.z, ra0.w * rg.w);             \
            ra1 = make_float4(ra1.x * rg.x, ra1.y * rg.y, ra1.z * rg.z, ra1.w * rg.w);             \
        }                                                                                          \
        *reinterpret_cast<float4*>(as_ + stash_at) = ra0;                                          \
        *reinterpret_cast<float4*>(as_ + stash_at + 64 * kBigLd) = ra1;                            \
        *reinterpret_cast<float4*>(ws_ + stash_at) = rw0;                                          \
        *reinterpret_cast<float4*>(ws_ + stash_at + 64 * kBigLd) = rw1;                            \
    }

    GH_BIG_FETCH(0)
    GH_BIG_STASH(0)
    __syncthreads();
    const int steps = K / kBigK;
    for (int s = 0; s < steps; s++) {
        const int buf = s & 1;
        if (s + 1 < steps) {  // in flight while this step multiplies
            GH_BIG_FETCH((s + 1) * kBigK)
        }
        const float* as = stage + buf * (2 * kBigTile * kBigLd) + (wm * 64) * kBigLd;
        const float* ws = stage + buf * (2 * kBigTile * kBigLd) + kBigTile * kBigLd + (wn * 64) * kBigLd;
        // 32 x 32 x 2 products: lane (row i32, half h32) brings k = 4 h32 + e (+ 8 q) to product e of
        // round q, for A and W alike, so every k of the step is multiplied once
#pragma unroll
        for (int q = 0; q < 2; q++) {
            float4 fa[2], fb[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                fa[t] = *reinterpret_cast<const float4*>(as + (t * 32 + i32) * kBigLd + q * 8 + h32 * 4);
                fb[t] = *reinterpret_cast<const float4*>(ws + (t * 32 + i32) * kBigLd + q * 8 + h32 * 4);
            }
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++) {
                    acc32[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a].x, fb[b].x, acc32[a][b], 0, 0, 0);
                    acc32[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a].y, fb[b].y, acc32[a][b], 0, 0, 0);
                    acc32[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a].z, fb[b].z, acc32[a][b], 0, 0, 0);
                    acc32[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a].w, fb[b].w, acc32[a][b], 0, 0, 0);
                }
        }
        if (s + 1 < steps) GH_BIG_STASH(buf ^ 1)
        __syncthreads();
    }
#undef GH_BIG_FETCH
#undef GH_BIG_STASH

    // finished tile -> LDS (accumulator layout: lane holds column i32, rows 8 (r / 4) + 4 h32 + r % 4)
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                ctile[(wm * 64 + a * 32 + 8 * (r >> 2) + 4 * h32 + (r & 3)) * kBigCLd + wn * 64 + b * 32 + i32] =
                    acc32[a][b][r];
    if (RMS) {
        // the four threads that fetched a row hold its partial sums of squares
        float v0 = ss0, v1 = ss1;
        v0 += dpp_move<0xB1, 0xF>(v0, 0.0f);  // quad_perm [1,0,3,2]
        v1 += dpp_move<0xB1, 0xF>(v1, 0.0f);
        v0 += dpp_move<0x4E, 0xF>(v0, 0.0f);  // quad_perm [2,3,0,1]
        v1 += dpp_move<0x4E, 0xF>(v1, 0.0f);
        if (fc == 0) {
            row_scale[fr] = 1.0f / sqrtf(v0 / static_cast<float>(K) + kNormEps);
            row_scale[fr + 64] = 1.0f / sqrtf(v1 / static_cast<float>(K) + kNormEps);
        }
    }
    __syncthreads();
    // column pairs (n, n + 1) of one row go through the shared epilogue
    for (int e = tid; e < kBigTile * (kBigTile / 2); e += kBigThreads) {
        const int i = e >> 6, jp = (e & 63) * 2;
        const int m = m0 + i, n = n0 + jp;
        if (m >= M || n >= p.N) continue;
        const float2 c = *reinterpret_cast<const float2*>(ctile + i * kBigCLd + jp);
        float v0 = c.x, v1 = c.y;
        if (RMS) {
            const float r = row_scale[i];
            v0 *= r;
            v1 *= r;
        }
        gemv_epilogue<EPI>(p, m, n, v0, v1, n + 1 < p.N);
    }
}

// True when the big-tile kernel applies: enough rows to fill the GPU with
// 128-row tiles and K a multiple of the K-step.
inline bool gemm128_ok(const GemvParams& p, int M) {
    return M >= 4 * kBigTile && p.K % kBigK == 0 && p.in_stride % 4 == 0;
}

template <int EPI, bool RMS>
inline void launch_gemm128(const GemvParams& p, int M, hipStream_t st) {
    const int m_tiles = (M + kBigTile - 1) / kBigTile, n_tiles = (p.N + kBigTile - 1) / kBigTile;
    hipLaunchKernelGGL((gemm128_kernel<EPI, RMS>), dim3(m_tiles * n_tiles), dim3(kBigThreads), kBigLdsBytes, st, p,
                       M, n_tiles);
}

}  // namespace gh

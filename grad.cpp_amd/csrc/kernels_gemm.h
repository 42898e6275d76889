// Batched projections for several sequences per step: C[M,N] = A[M,K] . Wt[N,K]^T
// on the fp32 matrix cores (v_mfma_f32_16x16x4_f32), fed by a row-norm kernel.
// The same epilogues as the batch-1 path run on the accumulator tile.
//
// The reference has no batch dimension (inference.h:23); M rows here are M
// independent InferenceSession::step calls sharing one pass over the weights.
#pragma once

#include "kernels_gemv.h"

namespace gh {

typedef float v4f __attribute__((ext_vector_type(4)));

// h[m] = norm(x[m]) for every row (layer_norm_row, inference.cpp:30-58).
// One wavefront per row; kind is PRO_LAYERNORM or PRO_RMSNORM.
__global__ __launch_bounds__(256) void norm_rows_kernel(const float* __restrict__ x,
                                                        const float* __restrict__ gamma,
                                                        const float* __restrict__ beta, float* h,
                                                        int M, int d, int kind) {
    const int lane = threadIdx.x & 63;
    const int m = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (m >= M) return;
    const float* xr = x + static_cast<size_t>(m) * d;
    float* hr = h + static_cast<size_t>(m) * d;
    if (kind == PRO_RMSNORM) {
        float ss = 0.0f;
        for (int k = lane; k < d; k += 64) ss += xr[k] * xr[k];
        const float r = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(d) + kNormEps);
        for (int k = lane; k < d; k += 64) hr[k] = gamma[k] * xr[k] * r;
    } else {
        float s = 0.0f;
        for (int k = lane; k < d; k += 64) s += xr[k];
        const float mean = wave_sum(s) / static_cast<float>(d);
        float var = 0.0f;
        for (int k = lane; k < d; k += 64) var += (xr[k] - mean) * (xr[k] - mean);
        const float inv_std = 1.0f / sqrtf(wave_sum(var) / static_cast<float>(d) + kNormEps);
        for (int k = lane; k < d; k += 64) hr[k] = gamma[k] * (xr[k] - mean) * inv_std + beta[k];
    }
}

// One workgroup = one 16 x 16 tile of C (16 rows of A against 16 weight rows);
// its four wavefronts split K and meet in LDS, and every wavefront keeps four
// K-steps of loads in flight.  The A and W fragments are read as float4 along K:
// lane group g = lane/16 holds k = 16*it + 4*g .. +3, and MFMA step s multiplies
// element s of every group, so one float4 per lane feeds four MFMA steps.  K must
// be a multiple of 64.  Small tiles are deliberate: with at most a few dozen rows
// of A the projections are bound by streaming the weights, and the narrow ones
// (N = d_model) need many workgroups to cover the GPU.
//
// Workgroups that share a weight tile are placed on the same XCD (hardware
// deals consecutive workgroup ids round-robin over the 8 XCDs), so a weight
// tile crosses HBM once and is re-read from that XCD's L2.
//
// RMS: the RMSNorm that precedes the projection is folded in.  A holds the raw
// residual rows; gamma scales A as it is loaded, the row's sum of squares is
// accumulated from the same fragments, and 1/rms multiplies the finished dot
// product (layer_norm_row, inference.cpp:33-43, distributes over the sum).
template <int EPI, bool RMS>
__global__ __launch_bounds__(256) void gemm16_kernel(const GemvParams p, int M, int m_tiles) {
    __shared__ float red[4][16 * 16];
    __shared__ float ssq[4][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // id -> (weight tile, row tile): ids with the same id % 8 and consecutive id / 8 share a weight tile
    const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
    const int n_tile = xcd + 8 * (slot / m_tiles), m_tile = slot % m_tiles;
    const int n0 = n_tile * 16, m0 = m_tile * 16;
    if (n0 >= p.N) return;
    const int K = p.K, kq = K / 4;
    const int j = lane & 15, g = lane >> 4;
    const int wrow = min(n0 + j, p.N - 1), arow = min(m0 + j, M - 1);
    const float* wp = p.W + static_cast<size_t>(wrow) * K + wave * kq + g * 4;
    const float* ap = p.in + static_cast<size_t>(arow) * p.in_stride + wave * kq + g * 4;
    const float* gp = RMS ? p.gamma + wave * kq + g * 4 : nullptr;
    v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
    float ss = 0.0f;

    auto step = [&](const float4& a_raw, const float4& b4, const float4& g4) {
        float4 a4 = a_raw;
        if (RMS) {
            ss += dot4(a_raw, a_raw);
            a4 = make_float4(a_raw.x * g4.x, a_raw.y * g4.y, a_raw.z * g4.z, a_raw.w * g4.w);
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4.x, b4.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4.y, b4.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4.z, b4.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4.w, b4.w, acc, 0, 0, 0);
    };
    int k = 0;
    for (; k + 64 <= kq; k += 64) {
        float4 a[4], b[4], gm[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            b[u] = *reinterpret_cast<const float4*>(wp + k + 16 * u);
            a[u] = *reinterpret_cast<const float4*>(ap + k + 16 * u);
            gm[u] = RMS ? *reinterpret_cast<const float4*>(gp + k + 16 * u) : make_float4(1.f, 1.f, 1.f, 1.f);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) step(a[u], b[u], gm[u]);
    }
    for (; k < kq; k += 16) {
        const float4 b4 = *reinterpret_cast<const float4*>(wp + k);
        const float4 a4 = *reinterpret_cast<const float4*>(ap + k);
        const float4 g4 = RMS ? *reinterpret_cast<const float4*>(gp + k) : make_float4(1.f, 1.f, 1.f, 1.f);
        step(a4, b4, g4);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) red[wave][(4 * g + r) * 16 + j] = acc[r];
    if (RMS) {
        // lanes j, j+16, j+32, j+48 hold the same row's partial sums of squares
        ss += __shfl_xor(ss, 16, kWave);
        ss += __shfl_xor(ss, 32, kWave);
        if (lane < 16) ssq[wave][lane] = ss;
    }
    __syncthreads();
    if (threadIdx.x < 128) {
        const int i = threadIdx.x >> 3, jp = (threadIdx.x & 7) * 2;
        const int m = m0 + i, n = n0 + jp;
        if (m < M && n < p.N) {
            const int at = i * 16 + jp;
            float v0 = (red[0][at] + red[1][at]) + (red[2][at] + red[3][at]);
            float v1 = (red[0][at + 1] + red[1][at + 1]) + (red[2][at + 1] + red[3][at + 1]);
            if (RMS) {
                const float ms = (ssq[0][i] + ssq[1][i]) + (ssq[2][i] + ssq[3][i]);
                const float r = 1.0f / sqrtf(ms / static_cast<float>(K) + kNormEps);
                v0 *= r;
                v1 *= r;
            }
            gemv_epilogue<EPI>(p, m, n, v0, v1, n + 1 < p.N);
        }
    }
}

template <int EPI, bool RMS>
inline void launch_gemm16(const GemvParams& p, int M, hipStream_t st) {
    const int m_tiles = (M + 15) / 16;
    const int n_tiles = (p.N + 15) / 16;
    const int n_tiles8 = (n_tiles + 7) / 8 * 8;  // whole rounds of the 8 XCDs
    hipLaunchKernelGGL((gemm16_kernel<EPI, RMS>), dim3(n_tiles8 * m_tiles), dim3(256), 0, st, p, M, m_tiles);
}

// The MFMA path needs K % 64 == 0 and 16-byte aligned rows; other shapes walk
// the batch with the batch-1 kernels.
inline bool gemm_shape_ok(int K, int in_stride) { return K % 64 == 0 && in_stride % 4 == 0; }

}  // namespace gh

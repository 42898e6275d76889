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

// One workgroup = one 16-wide slab of output columns (weight rows) for up to
// 16*MT rows of A; its four wavefronts split K and meet in LDS.  The A and W
// fragments are read as float4 along K: lane group g = lane/16 holds
// k = 16*it + 4*g .. +3, and MFMA step s multiplies element s of every group,
// so one float4 per lane feeds four MFMA steps.  K must be a multiple of 64.
template <int MT, int EPI>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const GemvParams p, int M) {
    __shared__ float red[4][MT][16 * 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 16;
    const int m0 = blockIdx.y * (16 * MT);
    const int K = p.K;
    const int kq = K / 4;  // K range of this wavefront
    const int j = lane & 15, g = lane >> 4;

    const int wrow = min(n0 + j, p.N - 1);
    const float* wp = p.W + static_cast<size_t>(wrow) * K + wave * kq + g * 4;
    const float* ap[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const int arow = min(m0 + t * 16 + j, M - 1);
        ap[t] = p.in + static_cast<size_t>(arow) * p.in_stride + wave * kq + g * 4;
    }
    v4f acc[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};

    for (int k = 0; k < kq; k += 16) {
        const float4 b4 = *reinterpret_cast<const float4*>(wp + k);
        float4 a4[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) a4[t] = *reinterpret_cast<const float4*>(ap[t] + k);
#pragma unroll
        for (int t = 0; t < MT; t++) {
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[t].x, b4.x, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[t].y, b4.y, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[t].z, b4.z, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[t].w, b4.w, acc[t], 0, 0, 0);
        }
    }
    // Accumulator layout: lane holds column j, rows 4*g + r.
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) red[wave][t][(4 * g + r) * 16 + j] = acc[t][r];
    __syncthreads();

    // Column pairs (n, n+1) of one row go through the shared epilogue.
    for (int e = threadIdx.x; e < MT * 16 * 8; e += 256) {
        const int t = e / 128, rem = e % 128;
        const int i = rem / 8, jp = (rem % 8) * 2;
        const int m = m0 + t * 16 + i, n = n0 + jp;
        if (m >= M || n >= p.N) continue;
        const int at = i * 16 + jp;
        const float v0 = (red[0][t][at] + red[1][t][at]) + (red[2][t][at] + red[3][t][at]);
        const float v1 = (red[0][t][at + 1] + red[1][t][at + 1])
                         + (red[2][t][at + 1] + red[3][t][at + 1]);
        gemv_epilogue<EPI>(p, m, n, v0, v1, n + 1 < p.N);
    }
}

// The MFMA path needs K % 64 == 0 and 16-byte aligned rows; other shapes walk
// the batch with the batch-1 kernels.
inline bool gemm_shape_ok(int K, int in_stride) { return K % 64 == 0 && in_stride % 4 == 0; }

template <int EPI>
inline void launch_gemm_mfma(const GemvParams& p, int M, hipStream_t st) {
    const int mt = M > 32 ? 4 : (M > 16 ? 2 : 1);
    const dim3 grid((p.N + 15) / 16, (M + 16 * mt - 1) / (16 * mt));
    switch (mt) {
        case 1: hipLaunchKernelGGL((gemm_mfma_kernel<1, EPI>), grid, dim3(256), 0, st, p, M); break;
        case 2: hipLaunchKernelGGL((gemm_mfma_kernel<2, EPI>), grid, dim3(256), 0, st, p, M); break;
        default: hipLaunchKernelGGL((gemm_mfma_kernel<4, EPI>), grid, dim3(256), 0, st, p, M); break;
    }
}

}  // namespace gh

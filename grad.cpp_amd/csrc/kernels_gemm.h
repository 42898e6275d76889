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
// product (layer_norm_row, inference.cpp:33-43, distributes over the sum).//
// MT x NT: 16-row tiles of A and 16-row tiles of W per workgroup.  Narrow
// projections run 1 x 1 (most workgroups); wide ones take the whole batch
// (MT = 4) so each weight row is fetched once, and the widest also several
// weight tiles per fetch of A (NT = 4).
template <int EPI, bool RMS, int MT, int NT, int KW>
__global__ __launch_bounds__(64 * KW) void gemm16_kernel(const GemvParams p, int M, int m_groups) {
    __shared__ float red[KW][MT][NT][16 * 16];
    __shared__ float ssq[KW][MT][16];
    // Every scalar argument the kernel reads is named here, at its start: the
    // compiler fetches an argument in the block that first uses it, and with the
    // uses spread behind the early exit and the epilogue's conditions that made four
    // fetches from the argument segment, each waited for before the next, in front
    // of the first weight load.  Named together they are one batch and one wait.
    asm volatile("" ::"s"(p.W), "s"(p.in), "s"(p.out), "s"(p.bias), "s"(p.gamma), "s"(p.N), "s"(p.K),
                 "s"(p.in_stride), "s"(p.out_stride), "s"(M), "s"(m_groups));
    if constexpr (EPI == EPI_QKV)
        asm volatile("" ::"s"(p.st), "s"(p.rope_cos), "s"(p.rope_sin), "s"(p.kv.page_table), "s"(p.kv.pool),
                     "s"(p.d_model), "s"(p.rows_per_seq), "s"(p.kv.pages_per_seq), "s"(p.kv.page_shift));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // id -> (weight group, row group): ids with the same id % 8 and consecutive id / 8 share weights
    const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
    {
        // workgroups past the tiles only touch the next launch's weights into their XCD's L2
        const int main_blocks = (((p.N + 16 * NT - 1) / (16 * NT) + 7) & ~7) * m_groups;
        if (id >= main_blocks) {
            touch_next_weights(p.next, id - main_blocks, 64 * KW);
            return;
        }
    }
    const int n_group = xcd + 8 * (slot / m_groups), m_group = slot % m_groups;
    const int n0 = n_group * 16 * NT, m0 = m_group * 16 * MT;
    if (n0 >= p.N) return;
    const int K = p.K, kq = K / KW;  // this wavefront's share of K
    const int j = lane & 15, g = lane >> 4;
    // Fetch layout: four neighbouring lanes read 64 contiguous bytes of one row
    // (lane = 4 * row + chunk), which the memory pipeline serves far faster than
    // the MFMA operand layout (lane = 16 * chunk + row) where neighbouring lanes
    // sit in different rows.  to_operand() moves a fetched float4 to the lane that
    // feeds it to the matrix core.
    const int fr = lane >> 2, fc = lane & 3;
    const int from_lane = (j * 4 + g) * 4;  // byte address of the source lane for ds_bpermute
    auto to_operand = [&](const float4& v) {
        return make_float4(
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.x))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.y))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.z))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.w))));
    };
    const float* wp[NT];
    const float* ap[MT];
#pragma unroll
    for (int t = 0; t < NT; t++)
        wp[t] = p.W + static_cast<size_t>(min(n0 + t * 16 + fr, p.N - 1)) * K + wave * kq + fc * 4;
#pragma unroll
    for (int t = 0; t < MT; t++)
        ap[t] = p.in + static_cast<size_t>(min(m0 + t * 16 + fr, M - 1)) * p.in_stride + wave * kq + fc * 4;
    const float* gp = RMS ? p.gamma + wave * kq + g * 4 : nullptr;
    // The first pair of outputs this thread will finish: what its epilogue reads
    // (bias, residual, position, page, rotation) is requested now, not after the
    // products, where it would be one or two more trips to memory on the tail.
    constexpr int kEpiElems = MT * NT * 128;
    const auto epi_at = [&](int e, int& m, int& n, int& tile_t, int& tile_u, int& at) {
        const int tile = e >> 7, rem = e & 127;
        tile_t = tile / NT;
        tile_u = tile % NT;
        const int i = rem >> 3, jp = (rem & 7) * 2;
        m = m0 + tile_t * 16 + i;
        n = n0 + tile_u * 16 + jp;
        at = i * 16 + jp;
    };
    EpiOperands first_epi;
    {
        int m, n, t, u, at;
        epi_at(static_cast<int>(threadIdx.x), m, n, t, u, at);
        if (static_cast<int>(threadIdx.x) < kEpiElems && m < M && n < p.N)
            first_epi = epi_fetch<EPI>(p, m, n, n + 1 < p.N);
    }
    v4f acc[MT][NT];
    float ss[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) {
        ss[t] = 0.0f;
#pragma unroll
        for (int u = 0; u < NT; u++) acc[t][u] = v4f{0.f, 0.f, 0.f, 0.f};
    }
    // K-steps of loads in flight per round.  Four, not as many as the registers would hold: with
    // eight (16 x 16 tiles: 90-124 vector registers) fewer workgroups fit a compute unit, and a
    // launch of these tiles lives on the number of loads the whole chip has in flight, not on
    // one wavefront's (measured at 64 rows, 0.4385 -> 0.4345 ms per step, and at 16 rows,
    // 0.568 -> 0.553 ms; two, three, five and six were all slower than four).
    constexpr int UNROLL = (MT + NT + 1) <= 6 ? 4 : 2;

    // One K-step in two halves.  prepare(): the fetched float4s go to the lanes that feed
    // them to the matrix core (ds_bpermute, a trip through the LDS crossbar each), with
    // the norm's share of the work.  multiply(): the products.  The halves of
    // neighbouring steps are interleaved below, the permutes of step u + 1 going out
    // before the products of step u, so that the crossbar's latency is paid beside the
    // products instead of in front of every one of them; sched_barrier keeps the
    // compiler from folding the two back into permute, wait, multiply, permute, ...
    // Only for one tile per workgroup: with more tiles (64 rows against wide
    // projections) the operands held for two steps cost registers and occupancy, and a
    // step measured slower that way (c3 421.5 -> 434.8 us; c4, all 1 x 1, 547.7 -> 544.8).
    constexpr bool kInterleave = MT * NT == 1;
    struct Operands {
        float4 a[MT], b[NT];
    };
    auto prepare = [&](const float4 (&a_in)[MT], const float4 (&b_in)[NT], const float4& g4, Operands& o) {
#pragma unroll
        for (int u = 0; u < NT; u++) o.b[u] = to_operand(b_in[u]);
#pragma unroll
        for (int t = 0; t < MT; t++) o.a[t] = to_operand(a_in[t]);
        if (RMS) {
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const float4 a = o.a[t];
                ss[t] += dot4(a, a);
                o.a[t] = make_float4(a.x * g4.x, a.y * g4.y, a.z * g4.z, a.w * g4.w);
            }
        }
    };
    auto multiply = [&](const Operands& o) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int u = 0; u < NT; u++) {
                acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x4f32(o.a[t].x, o.b[u].x, acc[t][u], 0, 0, 0);
                acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x4f32(o.a[t].y, o.b[u].y, acc[t][u], 0, 0, 0);
                acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x4f32(o.a[t].z, o.b[u].z, acc[t][u], 0, 0, 0);
                acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x4f32(o.a[t].w, o.b[u].w, acc[t][u], 0, 0, 0);
            }
    };
    int k = 0;
    for (; k + 16 * UNROLL <= kq; k += 16 * UNROLL) {
        float4 a[UNROLL][MT], b[UNROLL][NT], gm[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
#pragma unroll
            for (int t = 0; t < NT; t++) b[u][t] = *reinterpret_cast<const float4*>(wp[t] + k + 16 * u);
#pragma unroll
            for (int t = 0; t < MT; t++) a[u][t] = *reinterpret_cast<const float4*>(ap[t] + k + 16 * u);
            gm[u] = RMS ? *reinterpret_cast<const float4*>(gp + k + 16 * u) : make_float4(1.f, 1.f, 1.f, 1.f);
        }
        if constexpr (kInterleave) {
            Operands o[2];
            prepare(a[0], b[0], gm[0], o[0]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                if (u + 1 < UNROLL) prepare(a[u + 1], b[u + 1], gm[u + 1], o[(u + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
                multiply(o[u & 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                Operands o;
                prepare(a[u], b[u], gm[u], o);
                multiply(o);
            }
        }
    }
    if (k < kq) {
        // The steps left over go out as one more round with every load in flight: a
        // step past the end re-reads the last one (a cache hit) and is not consumed.
        float4 a[UNROLL][MT], b[UNROLL][NT], gm[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL - 1; u++) {
            const int kk = min(k + 16 * u, kq - 16);
#pragma unroll
            for (int t = 0; t < NT; t++) b[u][t] = *reinterpret_cast<const float4*>(wp[t] + kk);
#pragma unroll
            for (int t = 0; t < MT; t++) a[u][t] = *reinterpret_cast<const float4*>(ap[t] + kk);
            gm[u] = RMS ? *reinterpret_cast<const float4*>(gp + kk) : make_float4(1.f, 1.f, 1.f, 1.f);
        }
        if constexpr (kInterleave) {
            Operands o[UNROLL - 1];
#pragma unroll
            for (int u = 0; u < UNROLL - 1; u++)
                if (k + 16 * u < kq) prepare(a[u], b[u], gm[u], o[u]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < UNROLL - 1; u++)
                if (k + 16 * u < kq) multiply(o[u]);
        } else {
#pragma unroll
            for (int u = 0; u < UNROLL - 1; u++)
                if (k + 16 * u < kq) {
                    Operands o;
                    prepare(a[u], b[u], gm[u], o);
                    multiply(o);
                }
        }
    }
    // Accumulator layout: lane holds column j, rows 4*g + r.
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int u = 0; u < NT; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[wave][t][u][(4 * g + r) * 16 + j] = acc[t][u][r];
    if (RMS) {
        // lanes j, j+16, j+32, j+48 hold the same row's partial sums of squares
#pragma unroll
        for (int t = 0; t < MT; t++) {
            float v = ss[t];
            v += __shfl_xor(v, 16, kWave);
            v += __shfl_xor(v, 32, kWave);
            if (lane < 16) ssq[wave][t][lane] = v;
        }
    }
    __syncthreads();
    // Column pairs (n, n+1) of one row go through the shared epilogue.
    for (int e = threadIdx.x; e < kEpiElems; e += 64 * KW) {
        int m, n, t, u, at;
        epi_at(e, m, n, t, u, at);
        if (m >= M || n >= p.N) continue;
        const int i = at >> 4;
        float v0 = 0.0f, v1 = 0.0f;
#pragma unroll
        for (int w = 0; w < KW; w++) {
            v0 += red[w][t][u][at];
            v1 += red[w][t][u][at + 1];
        }
        if (RMS) {
            float ms = 0.0f;
#pragma unroll
            for (int w = 0; w < KW; w++) ms += ssq[w][t][i];
            const float r = 1.0f / sqrtf(ms / static_cast<float>(K) + kNormEps);
            v0 *= r;
            v1 *= r;
        }
        const bool has1 = n + 1 < p.N;
        if (e == static_cast<int>(threadIdx.x)) epi_apply<EPI>(p, m, n, v0, v1, has1, first_epi);
        else gemv_epilogue<EPI>(p, m, n, v0, v1, has1);
        if constexpr (EPI == EPI_STORE) {
            if (p.best) {
                // eight neighbouring lanes hold the 16 columns of one row of one tile, in
                // column order: fold them (an inactive lane's value is never taken)
                float bv = (has1 && v1 > v0) ? v1 : v0;
                int bn = (has1 && v1 > v0) ? n + 1 : n;
                first_max_step<0xB1, 0xF>(bv, bn);
                first_max_step<0x4E, 0xF>(bv, bn);
                first_max_step<0x141, 0xF>(bv, bn);
                if ((e & 7) == 0) p.best[static_cast<size_t>(m) * p.best_stride + (n >> 4)] = make_float2(bv, __int_as_float(bn));
            }
        }
    }
}

template <int EPI, bool RMS, int MT, int NT, int KW>
inline void launch_gemm16_as(const GemvParams& p, int M, hipStream_t st) {
    const int m_groups = (M + 16 * MT - 1) / (16 * MT);
    const int n_groups = (p.N + 16 * NT - 1) / (16 * NT);
    const int n_groups8 = (n_groups + 7) / 8 * 8;  // whole rounds of the 8 XCDs
    hipLaunchKernelGGL((gemm16_kernel<EPI, RMS, MT, NT, KW>), dim3(n_groups8 * m_groups + p.next.blocks),
                       dim3(64 * KW), 0, st, p, M, m_groups);
}

// Weight tiles per workgroup of the wide kernel: 16000 rows = 250 workgroups.
constexpr int kWideTiles = 4;

// Wide projections of a few rows (the tied logits of a decode step: N = vocab,
// M <= 32 sequences).  With 16 x 16 tiles every workgroup fetches its rows of A
// again, and for N in the thousands that traffic (M x K per tile) is several
// times the weights.  Here A is stationary: K is split over the 8 wavefronts of
// a workgroup, each keeps its K / 8 slice of all M rows in registers in the MFMA
// operand layout (RMSNorm gain already applied), and the workgroup walks
// kWideTiles consecutive 16-row weight tiles, all requested at the start, so
// every weight row crosses the chip once and A once per four tiles.
// KS = K / 128 K-steps of 16 per wavefront; MT 16-row tiles of A.
template <bool RMS, int MT, int KS>
__global__ __launch_bounds__(512) void gemm_wide_kernel(const GemvParams p, int M) {
    constexpr int KW = 8, NTILE = kWideTiles;
    __shared__ float red[KW][MT][16 * 16];
    __shared__ float ssq[KW][MT][16];
    __shared__ float rinv[MT][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int K = p.K, kq = KS * 16;
    const int j = lane & 15, g = lane >> 4;
    const int fr = lane >> 2, fc = lane & 3;  // fetch layout: 4 lanes read 64 B of one row
    const int from_lane = (j * 4 + g) * 4;
    auto to_operand = [&](const float4& v) {
        return make_float4(
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.x))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.y))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.z))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from_lane, __float_as_int(v.w))));
    };
    const int n_tiles = (p.N + 15) >> 4;
    const int tile0 = blockIdx.x * NTILE;
    const int tile_end = min(tile0 + NTILE, n_tiles);
    if (tile0 >= n_tiles) return;
    // Weights and outputs go through bounded buffer descriptors: an access past the
    // end reads zero / is dropped, so no load or store of the tile loop sits under
    // a branch and the waits between them count exactly the operations in flight
    // (a conditional one makes the compiler wait for everything, and a wavefront's
    // loads return in order, so the tile being waited for would be the last).
    constexpr unsigned kPastEnd = 0x80000000u;  // beyond any matrix this kernel is given
    const __amdgpu_buffer_rsrc_t rs_w = make_buffer(p.W, static_cast<unsigned>(p.N) * K * 4u);
    const __amdgpu_buffer_rsrc_t rs_o =
        make_buffer(p.out, (static_cast<unsigned>(M - 1) * p.out_stride + p.N) * 4u);
    auto fetch_tile = [&](int tile, float4 (&w)[KS]) {
        const int row = tile * 16 + fr;
        const unsigned off = (tile < tile_end && row < p.N)
                                 ? (static_cast<unsigned>(row) * K + wave * kq + fc * 4) * 4u
                                 : kPastEnd;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs_w, off, 64 * s, 0);
            w[s] = make_float4(__int_as_float(v.x), __int_as_float(v.y), __int_as_float(v.z), __int_as_float(v.w));
        }
    };
    // A first: a wavefront's loads return in the order they were issued, so the
    // (cached) rows of A must not queue behind the weight tiles coming from HBM.
    float4 as[MT][KS];  // this wavefront's K slice of every row
    float4 gm[KS];
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const float* ap = p.in + static_cast<size_t>(min(t * 16 + fr, M - 1)) * p.in_stride + wave * kq + fc * 4;
#pragma unroll
        for (int s = 0; s < KS; s++) as[t][s] = *reinterpret_cast<const float4*>(ap + 16 * s);
    }
#pragma unroll
    for (int s = 0; s < KS; s++)
        gm[s] = RMS ? *reinterpret_cast<const float4*>(p.gamma + wave * kq + 16 * s + g * 4)
                    : make_float4(1.f, 1.f, 1.f, 1.f);
    float4 wf[NTILE][KS];  // every tile of the workgroup is in flight from the start
#pragma unroll
    for (int f = 0; f < NTILE; f++) fetch_tile(tile0 + f, wf[f]);

    // A moves to the operand layout once; RMSNorm's gain is applied here and the
    // rows' sums of squares come from the same fragments.
    {
        float ss[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) {
            ss[t] = 0.0f;
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const float4 a = to_operand(as[t][s]);
                as[t][s] = a;
                if (RMS) {
                    ss[t] += dot4(a, a);
                    as[t][s] = make_float4(a.x * gm[s].x, a.y * gm[s].y, a.z * gm[s].z, a.w * gm[s].w);
                }
            }
        }
        if (RMS) {
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float v = ss[t];
                v += __shfl_xor(v, 16, kWave);
                v += __shfl_xor(v, 32, kWave);
                if (lane < 16) ssq[wave][t][lane] = v;
            }
            __syncthreads();
            if (threadIdx.x < MT * 16) {
                const int t = threadIdx.x >> 4, i = threadIdx.x & 15;
                float ms = 0.0f;
#pragma unroll
                for (int w = 0; w < KW; w++) ms += ssq[w][t][i];
                rinv[t][i] = 1.0f / sqrtf(ms / static_cast<float>(K) + kNormEps);
            }
            // the barrier inside the first tile orders rinv before its readers
        }
    }
    // outputs of this thread in every tile: row m, column pair (jp, jp + 1)
    const int e = threadIdx.x;
    const int et = min(e >> 7, MT - 1), ei = (e & 127) >> 3, ejp = (e & 7) * 2;
    const int em = et * 16 + ei;
    const bool e_live = e < MT * 128 && em < M;

    // Straight-line code over the tiles: no loop carries loads across a back edge,
    // so every wait names exactly the tile it needs.  Tiles past the end were read
    // as zeros and their stores are dropped.
    {
#pragma unroll
        for (int f = 0; f < NTILE; f++) {
            const int tile = tile0 + f;
            v4f acc[MT];
#pragma unroll
            for (int t = 0; t < MT; t++) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const float4 b = to_operand(wf[f][s]);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(as[t][s].x, b.x, acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(as[t][s].y, b.y, acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(as[t][s].z, b.z, acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(as[t][s].w, b.w, acc[t], 0, 0, 0);
                }
            }
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) red[wave][t][(4 * g + r) * 16 + j] = acc[t][r];
            __syncthreads();
            const int n = tile * 16 + ejp;
            {
                const int at = ei * 16 + ejp;
                float v0 = 0.0f, v1 = 0.0f;
#pragma unroll
                for (int w = 0; w < KW; w++) {
                    v0 += red[w][et][at];
                    v1 += red[w][et][at + 1];
                }
                if (RMS) {
                    const float r = rinv[et][ei];
                    v0 *= r;
                    v1 *= r;
                }
                const unsigned o = (static_cast<unsigned>(em) * p.out_stride + n) * 4u;
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_int(v0), rs_o, e_live && n < p.N ? o : kPastEnd, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_int(v1), rs_o,
                                                      e_live && n + 1 < p.N ? o + 4u : kPastEnd, 0, 0);
                if (p.best) {
                    // eight neighbouring lanes hold the tile's 16 columns of one row, in column order
                    const bool has1 = n + 1 < p.N;
                    float bv = n < p.N ? ((has1 && v1 > v0) ? v1 : v0) : -INFINITY;
                    int bn = (has1 && v1 > v0) ? n + 1 : n;
                    first_max_step<0xB1, 0xF>(bv, bn);
                    first_max_step<0x4E, 0xF>(bv, bn);
                    first_max_step<0x141, 0xF>(bv, bn);
                    if ((e & 7) == 0 && e_live && n < p.N)
                        p.best[static_cast<size_t>(em) * p.best_stride + tile] = make_float2(bv, __int_as_float(bn));
                }
            }
            __syncthreads();  // red is rewritten by the next tile
        }
    }
    // the launch that makes the logits also ends the step (inference.cpp:256)
    if (p.advance && blockIdx.x == 0 && threadIdx.x == 0) p.advance->pos += 1;
}

// The wide kernel takes a plain store without bias, K = 128 * KS (A fits in
// registers) and matrices whose byte offsets stay below 2 GiB.
inline bool gemm_wide_ok(const GemvParams& p, int M) {
    // Up to 32 rows: at 64 the products (10 us of fp32 MFMA for 16000 x 768) bound
    // the launch and the 16 x 16 tiling is as fast (measured 25.8 us either way).
    if (p.N <= 8192 || M > 32 || p.K % 128 != 0 || p.bias != nullptr) return false;
    if (static_cast<unsigned long long>(p.N) * p.K * 4ull >= 0x80000000ull) return false;
    if ((static_cast<unsigned long long>(M - 1) * p.out_stride + p.N) * 4ull >= 0x80000000ull) return false;
    const int ks = p.K / 128;
    return ks == 4 || ks == 6 || ks == 8;
}

template <bool RMS, int MT, int KS>
inline void launch_gemm_wide_as(const GemvParams& p, int M, hipStream_t st) {
    const int n_tiles = (p.N + 15) / 16;
    hipLaunchKernelGGL((gemm_wide_kernel<RMS, MT, KS>), dim3((n_tiles + kWideTiles - 1) / kWideTiles), dim3(512),
                       0, st, p, M);
}

template <bool RMS, int MT>
inline void launch_gemm_wide_ks(const GemvParams& p, int M, hipStream_t st) {
    const int ks = p.K / 128;
    if (ks == 8) launch_gemm_wide_as<RMS, MT, 8>(p, M, st);
    else if (ks == 6) launch_gemm_wide_as<RMS, MT, 6>(p, M, st);
    else launch_gemm_wide_as<RMS, MT, 4>(p, M, st);
}

template <bool RMS>
inline void launch_gemm_wide(const GemvParams& p, int M, hipStream_t st) {
    if (M <= 16) launch_gemm_wide_ks<RMS, 1>(p, M, st);
    else launch_gemm_wide_ks<RMS, 2>(p, M, st);
}

// At 64 rows (0.4575 ms per step with 2 x 1 tiles on 8 wavefronts for the wide projections and
// 2 x 2 on 4 for the logits): wide 2 x 1 on 4 wavefronts 0.4384 (2 x 2 on 8: 0.4432, 1 x 4: 0.4504,
// 2 x 4: 0.4742, 4 x 2: 0.4990, 2 x 1 on 2: 0.5125, 4 x 1 on 4: 0.5128); narrow 1 x 1 on 8 stays
// (on 4: 0.4488, 2 x 1: 0.4615-0.5073); logits 2 x 4 on 8 0.4303 (2 x 2 on 8: 0.4351, 4 x 2: 0.4336).
// Tile shapes by measurement on the decode shapes (M = 64 rows): every launch
// is bound by latency (kernel start, one trip to memory, the merge across the K
// split), not by the weights, so small tiles on many workgroups win; long row
// blocks (a prompt pass) take the whole 64-row tile so each weight row is
// fetched once per workgroup.  K is split over 8 wavefronts when that leaves
// each a multiple of 16.
template <int EPI, bool RMS>
inline void launch_gemm16(const GemvParams& p, int M, hipStream_t st) {
    if constexpr (EPI == EPI_STORE) {
        if (gemm_wide_ok(p, M)) return launch_gemm_wide<RMS>(p, M, st);
    }
    const bool k8 = p.K % 128 == 0;
    if (p.N <= 1024 || M <= 16) {
        if (k8) launch_gemm16_as<EPI, RMS, 1, 1, 8>(p, M, st);
        else launch_gemm16_as<EPI, RMS, 1, 1, 4>(p, M, st);
    } else if (p.N > 8192) {
        if (M <= 64 && k8) launch_gemm16_as<EPI, RMS, 2, 4, 8>(p, M, st);
        else if (M <= 64) launch_gemm16_as<EPI, RMS, 2, 2, 4>(p, M, st);
        else launch_gemm16_as<EPI, RMS, 4, 2, 4>(p, M, st);
    } else if (M <= 64) {
        // more than 32 rows: K over four wavefronts, twice as many (smaller) workgroups per compute unit
        if (k8 && M <= 32) launch_gemm16_as<EPI, RMS, 2, 1, 8>(p, M, st);
        else launch_gemm16_as<EPI, RMS, 2, 1, 4>(p, M, st);
    } else {
        if (k8) launch_gemm16_as<EPI, RMS, 4, 1, 8>(p, M, st);
        else launch_gemm16_as<EPI, RMS, 4, 1, 4>(p, M, st);
    }
}

// The MFMA path needs K % 64 == 0 and 16-byte aligned rows; other shapes walk
// the batch with the batch-1 kernels.
inline bool gemm_shape_ok(int K, int in_stride) { return K % 64 == 0 && in_stride % 4 == 0; }

}  // namespace gh

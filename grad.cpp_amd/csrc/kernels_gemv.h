// Batch-1 projections: one wavefront per pair of output rows, weights stored
// (out, in) so each row is one contiguous fp32 stream; the norm that precedes
// the projection is recomputed per wavefront in registers (no LDS, no block
// barrier), and the op that follows it (bias, RoPE + cache write, residual add,
// GELU, SwiGLU) runs in the epilogue.
//
// Restates matvec / matvec_add / matvec_nobias / layer_norm_row / rope_row /
// gelu_row / silu_row of src/transformer/inference.cpp:14-115 as fused kernels.
#pragma once

#include "kernels_common.h"

namespace gh {

enum Prologue { PRO_PLAIN = 0, PRO_LAYERNORM = 1, PRO_RMSNORM = 2 };
enum Epilogue { EPI_STORE = 0, EPI_QKV = 1, EPI_RESID = 2, EPI_GELU = 3, EPI_SWIGLU = 4 };

// What a decode launch of a few dozen rows brings into the L2s for the launch after it.  Lines
// read by one launch are still in an XCD's L2 when the next launch on the stream reads them
// there, and a dependent launch is little more than its start plus one trip to memory per
// round of loads.  The next launch's matrix is cut into chunks of chunk_lines cache lines
// (one 16-row weight tile of that launch); chunk c will be read by workgroups on XCD c % 8
// (gemm16_kernel's id -> tile map), and `blocks` workgroups appended to the grid of this
// launch (a multiple of 8, so workgroup b runs on XCD b % 8 like every other) read one word
// of every line of their XCD's chunks.  Per decode step of the 69M Llama block at context
// 256, without and with: 2 sequences 247.0 -> 243.4 us, 8: 252.3 -> 248.2, 16: 277.3 ->
// 268.3, 24: 312.0 -> 299.7, 32: 328.6 -> 310.7, 48: 377.4 -> 371.2, 64: 397.6 -> 409.0; 16
// sequences at context 2048 516.0 -> 509.5 (the same touches dealt to the workgroups
// without regard to the XCD, which only fills the memory-side cache: 516.1 -> 513.3).  At 64
// sequences the launches that carry the touches lose more than the next ones gain, so the
// engine asks for it up to 48.  blocks == 0: nothing to do.
struct NextWeights {
    const float* base;
    int chunk_lines;
    int chunks;
    int blocks;
};

// Workgroup pb of f.blocks appended ones; nthreads threads, four loads in flight each.
__device__ __forceinline__ void touch_next_weights(const NextWeights& f, int pb, int nthreads) {
    const int xcd = pb & 7, slot = pb >> 3, slots = f.blocks >> 3;
    const int lines = ((f.chunks - xcd + 7) >> 3) * f.chunk_lines;  // this XCD's share
    const int stride = slots * nthreads;
    const int* base = reinterpret_cast<const int*>(f.base);
    for (int i0 = slot * nthreads + static_cast<int>(threadIdx.x); i0 < lines; i0 += 4 * stride) {
        int v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = min(i0 + u * stride, lines - 1);  // past the end: the last line again
            const int c = xcd + 8 * (i / f.chunk_lines), l = i % f.chunk_lines;
            v[u] = base[(static_cast<size_t>(c) * f.chunk_lines + l) * 32];
        }
        asm volatile("" ::"v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]));
    }
}

struct GemvParams {
    const float* W;     // (N, K) row-major: row n holds the weights of output n
    const float* bias;  // N floats or nullptr
    int N, K;
    const float* in;  // [batch][in_stride]
    int in_stride;
    const float* gamma;  // norm gain / shift (K floats) for PRO_*NORM
    const float* beta;
    float* out;  // [batch][out_stride]
    int out_stride;
    // EPI_QKV: rows [0,d) are q, [d,2d) k, [2d,3d) v.
    KvLayout kv;
    int layer;
    int d_model;
    int rope;               // rotate q and k pairs (2j, 2j+1)
    const float* rope_cos;  // [max_len][head_size/2]
    const float* rope_sin;
    const DevState* st;
    // EPI_STORE only: when set, the thread that stores element (0, 0) also ends the
    // step, pos_++ (inference.cpp:256).  Nothing else in that launch reads the state.
    DevState* advance;
    // Rows of one prompt pass: row m is token m % rows_per_seq of sequence
    // m / rows_per_seq and sits at position pos_base + m % rows_per_seq.
    // rows_per_seq == 0: one row per sequence, all at st->pos (a decode step).
    int rows_per_seq;
    int pos_base;
    // EPI_STORE on the matrix-core kernels only: when set, the largest output of every
    // row in every run of 16 columns and its first column, best[row * best_stride +
    // column / 16] = {value, column as int bits}: what an arg-max over the row needs
    // (text_gen.cpp:52-60) without reading the row back.
    float2* best;
    int best_stride;
    // gemm16_kernel up to 48 rows: the matrix of the launch that follows this one
    // (see NextWeights).
    NextWeights next;
};

// What the epilogue of one pair of outputs (row, row + 1) of input row b needs
// from memory besides the two products.  Fetching it is separate from applying
// it so that a kernel can issue these loads before its main loop: they do not
// depend on the products, and left to the end they are one or two more trips to
// memory on the tail of every launch (position -> page table and rotation
// tables -> store).
struct EpiOperands {
    float b0 = 0.0f, b1 = 0.0f;  // bias pair
    float r0 = 0.0f, r1 = 0.0f;  // EPI_RESID: the outputs' current values
    float cs = 1.0f, sn = 0.0f;  // EPI_QKV: rotation of the pair
    int pos = 0, seq = 0, page = 0;  // EPI_QKV: position, sequence, physical cache page
};

template <int EPI>
__device__ __forceinline__ EpiOperands epi_fetch(const GemvParams& p, int b, int row, bool has1) {
    EpiOperands o;
    if constexpr (EPI == EPI_STORE || EPI == EPI_RESID) {
        if (p.bias) {
            o.b0 = p.bias[row];
            if (has1) o.b1 = p.bias[row + 1];
        }
    }
    if constexpr (EPI == EPI_RESID) {
        const float* cur = p.out + static_cast<size_t>(b) * p.out_stride;
        o.r0 = cur[row];
        if (has1) o.r1 = cur[row + 1];
    }
    if constexpr (EPI == EPI_GELU || EPI == EPI_QKV) {
        o.b0 = p.bias[row];
        if (has1) o.b1 = p.bias[row + 1];
    }
    if constexpr (EPI == EPI_QKV) {
        // rows_per_seq == 0: one row per sequence, all at st->pos (a decode step)
        o.seq = b;
        if (p.rows_per_seq > 0) {
            o.seq = b / p.rows_per_seq;
            o.pos = p.pos_base + (b - o.seq * p.rows_per_seq);
        } else {
            o.pos = p.st->pos;
        }
        if (p.rope && row < 2 * p.d_model) {
            // head_size is even under RoPE, so (row, row+1) is one rotation pair.
            const int hs = p.kv.head_size;
            const int j = ((row % p.d_model) % hs) >> 1;
            o.cs = p.rope_cos[o.pos * (hs >> 1) + j];
            o.sn = p.rope_sin[o.pos * (hs >> 1) + j];
        }
        // row + 1 may already be a key row when d_model is odd
        if (row + 1 >= p.d_model) o.page = p.kv.page_table[o.seq * p.kv.pages_per_seq + (o.pos >> p.kv.page_shift)];
    }
    return o;
}

// One projected value of the fused QKV product goes to the q buffer or straight
// into the cache row of the current position (inference.cpp:195-199).
__device__ __forceinline__ void store_qkv(const GemvParams& p, int m, int row, float v, const EpiOperands& o) {
    const int d = p.d_model;
    const int sec = row / d, c = row - sec * d;
    if (sec == 0) {
        p.out[static_cast<size_t>(m) * p.out_stride + c] = v;
    } else {
        const int hs = p.kv.head_size;
        const int head = c / hs, j = c - head * hs;
        const int slot = o.pos & ((1 << p.kv.page_shift) - 1);
        // The page number is first touched here: widened to 64 bits where it was
        // fetched, it would have to arrive before the kernel's main loads go out.
        int page = o.page;
        asm volatile("" : "+v"(page));
        const size_t run =
            (((static_cast<size_t>(p.layer) * p.kv.n_pages + page) * 2 + (sec - 1)) * p.kv.heads + head);
        p.kv.pool[((run << p.kv.page_shift) + slot) * hs + j] = v;
    }
}

template <int EPI>
__device__ __forceinline__ void epi_apply(const GemvParams& p, int b, int row, float v0, float v1, bool has1,
                                          const EpiOperands& o) {
    if constexpr (EPI == EPI_STORE) {
        float* out = p.out + static_cast<size_t>(b) * p.out_stride;
        out[row] = v0 + o.b0;
        if (has1) out[row + 1] = v1 + o.b1;
        if (p.advance && b == 0 && row == 0) p.advance->pos += 1;
    } else if constexpr (EPI == EPI_RESID) {
        // y += b, then y += x @ W (inference.cpp:22-28)
        float* out = p.out + static_cast<size_t>(b) * p.out_stride;
        out[row] = (o.r0 + o.b0) + v0;
        if (has1) out[row + 1] = (o.r1 + o.b1) + v1;
    } else if constexpr (EPI == EPI_GELU) {
        float* out = p.out + static_cast<size_t>(b) * p.out_stride;
        out[row] = gelu_tanh(v0 + o.b0);
        if (has1) out[row + 1] = gelu_tanh(v1 + o.b1);
    } else if constexpr (EPI == EPI_SWIGLU) {
        // rows (2p, 2p+1) = (gate_p, up_p): hidden_p = up * silu(gate) (inference.cpp:234-239)
        p.out[static_cast<size_t>(b) * p.out_stride + (row >> 1)] = v1 * silu(v0);
    } else if constexpr (EPI == EPI_QKV) {
        float a = v0 + o.b0;
        float c = has1 ? v1 + o.b1 : 0.0f;
        if (p.rope && row < 2 * p.d_model) {
            const float ra = a * o.cs - c * o.sn;
            const float rc = a * o.sn + c * o.cs;
            a = ra;
            c = rc;
        }
        store_qkv(p, b, row, a, o);
        if (has1) store_qkv(p, b, row + 1, c, o);
    }
}

template <int EPI>
__device__ __forceinline__ void gemv_epilogue(const GemvParams& p, int b, int row, float v0,
                                              float v1, bool has1) {
    epi_apply<EPI>(p, b, row, v0, v1, has1, epi_fetch<EPI>(p, b, row, has1));
}

// Normalises a register-resident row slice in place (layer_norm_row,
// inference.cpp:30-58): lane holds float4 i at elements (i*64 + lane)*4 .. +3 of
// a K-long row, K = KV * 256.  The two reductions are wave-wide.
template <int KV, int PRO>
__device__ __forceinline__ void norm_in_registers(float4 (&h)[KV], const float* gamma,
                                                  const float* beta, int K, int lane) {
    if constexpr (PRO == PRO_RMSNORM) {
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < KV; i++) ss += dot4(h[i], h[i]);
        ss = wave_sum(ss);
        const float r = 1.0f / sqrtf(ss / static_cast<float>(K) + kNormEps);
#pragma unroll
        for (int i = 0; i < KV; i++) {
            const float4 g = reinterpret_cast<const float4*>(gamma)[i * 64 + lane];
            h[i] = make_float4(g.x * h[i].x * r, g.y * h[i].y * r, g.z * h[i].z * r, g.w * h[i].w * r);
        }
    } else if constexpr (PRO == PRO_LAYERNORM) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < KV; i++) s += (h[i].x + h[i].y) + (h[i].z + h[i].w);
        const float mean = wave_sum(s) / static_cast<float>(K);
        float var = 0.0f;
#pragma unroll
        for (int i = 0; i < KV; i++) {
            h[i] = make_float4(h[i].x - mean, h[i].y - mean, h[i].z - mean, h[i].w - mean);
            var += dot4(h[i], h[i]);
        }
        var = wave_sum(var) / static_cast<float>(K);
        const float inv_std = 1.0f / sqrtf(var + kNormEps);
#pragma unroll
        for (int i = 0; i < KV; i++) {
            const float4 g = reinterpret_cast<const float4*>(gamma)[i * 64 + lane];
            const float4 be = reinterpret_cast<const float4*>(beta)[i * 64 + lane];
            h[i] = make_float4(g.x * h[i].x * inv_std + be.x, g.y * h[i].y * inv_std + be.y,
                               g.z * h[i].z * inv_std + be.z, g.w * h[i].w * inv_std + be.w);
        }
    }
}

// KV: float4 loads per lane per row when K == KV * 256 (fast path); KV == 0 is
// the any-K path.  PAIRS: row pairs per wavefront.
template <int KV, int PAIRS, int PRO, int EPI>
__global__ __launch_bounds__(256) void gemv_kernel(const GemvParams p) {
    constexpr int R = 2 * PAIRS;
    const int lane = threadIdx.x & 63;
    const int wid = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int b = blockIdx.y;
    const int row0 = wid * R;
    if (row0 >= p.N) return;
    const int K = p.K;
    const float* xin = p.in + static_cast<size_t>(b) * p.in_stride;
    float acc[R];
    // what the epilogue reads is requested before the products (every lane asks
    // for the same addresses; lane 0 uses them)
    EpiOperands epi[PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; q++) {
        const int row = row0 + 2 * q;
        if (row < p.N) epi[q] = epi_fetch<EPI>(p, b, row, row + 1 < p.N);
    }

    if constexpr (KV > 0) {
        // Weight loads are issued first: they do not depend on the activations.
        float4 w[R][KV];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = min(row0 + r, p.N - 1);
            const float4* wr = reinterpret_cast<const float4*>(p.W + static_cast<size_t>(row) * K);
#pragma unroll
            for (int i = 0; i < KV; i++) w[r][i] = wr[i * 64 + lane];
        }
        float4 h[KV];
#pragma unroll
        for (int i = 0; i < KV; i++) h[i] = reinterpret_cast<const float4*>(xin)[i * 64 + lane];

        norm_in_registers<KV, PRO>(h, p.gamma, p.beta, K, lane);
#pragma unroll
        for (int r = 0; r < R; r++) {
            float a = 0.0f;
#pragma unroll
            for (int i = 0; i < KV; i++) a += dot4(w[r][i], h[i]);
            acc[r] = wave_sum(a);
        }
    } else {
        // Any K: the norm statistics come from two strided passes over x, the
        // normalised value is rebuilt on the fly inside the dot products.
        float mean = 0.0f, scale = 1.0f;
        if constexpr (PRO == PRO_RMSNORM) {
            float ss = 0.0f;
            for (int k = lane; k < K; k += 64) ss += xin[k] * xin[k];
            scale = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(K) + kNormEps);
        } else if constexpr (PRO == PRO_LAYERNORM) {
            float s = 0.0f;
            for (int k = lane; k < K; k += 64) s += xin[k];
            mean = wave_sum(s) / static_cast<float>(K);
            float var = 0.0f;
            for (int k = lane; k < K; k += 64) var += (xin[k] - mean) * (xin[k] - mean);
            scale = 1.0f / sqrtf(wave_sum(var) / static_cast<float>(K) + kNormEps);
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = min(row0 + r, p.N - 1);
            const float* wr = p.W + static_cast<size_t>(row) * K;
            float a = 0.0f;
            for (int k = lane; k < K; k += 64) {
                float hv = xin[k];
                if constexpr (PRO == PRO_RMSNORM) hv = p.gamma[k] * hv * scale;
                if constexpr (PRO == PRO_LAYERNORM) hv = p.gamma[k] * (hv - mean) * scale + p.beta[k];
                a += wr[k] * hv;
            }
            acc[r] = wave_sum(a);
        }
    }

    if (lane == 0) {
#pragma unroll
        for (int q = 0; q < PAIRS; q++) {
            const int row = row0 + 2 * q;
            if (row < p.N) epi_apply<EPI>(p, b, row, acc[2 * q], acc[2 * q + 1], row + 1 < p.N, epi[q]);
        }
    }
}

// x[b] = E[token[b]] * 1.0 (+ P[pos]) — inference.cpp:159-182 (the embedding
// scale is 1.0, token_embedding.h:12).
__global__ void embed_kernel(const float* __restrict__ E, const float* __restrict__ P,
                             const int* __restrict__ tok, const DevState* st, float* x, int d) {
    const int b = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= d) return;
    float v = E[static_cast<size_t>(tok[b]) * d + j];
    if (P) v += P[static_cast<size_t>(st->pos) * d + j];
    x[static_cast<size_t>(b) * d + j] = v;
}

// The same for every token of a prompt pass: row m = seq * len + t holds token
// t of sequence seq, at position pos_base + t.
__global__ void embed_rows_kernel(const float* __restrict__ E, const float* __restrict__ P,
                                  const int* __restrict__ hist, int hist_stride, int hist_base, int len,
                                  int pos_base, float* x, int d) {
    const int m = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= d) return;
    const int seq = m / len, t = m - seq * len;
    const int tok = hist[static_cast<size_t>(seq) * hist_stride + hist_base + t];
    float v = E[static_cast<size_t>(tok) * d + j];
    if (P) v += P[static_cast<size_t>(pos_base + t) * d + j];
    x[static_cast<size_t>(m) * d + j] = v;
}

// rows[b] = x[b * len + len - 1]: the last position of every sequence.
__global__ void take_last_rows_kernel(const float* __restrict__ x, int len, float* rows, int d) {
    const int b = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < d) rows[static_cast<size_t>(b) * d + j] = x[(static_cast<size_t>(b) * len + len - 1) * d + j];
}


// Negative log-likelihood of one target per logits row: Variable::cross_entropy's
// log_softmax + nll_loss (variable.cpp:589-592) before the mean over rows.  One
// workgroup per row; row r of this launch is row `row0 + r` of a prompt pass
// whose row m = seq * slice_len + t holds position t0 + t of sequence seq.
// nll[seq * len + t0 + t] = log(sum_j exp(x_j - max)) + max - x_target.
__global__ __launch_bounds__(256) void nll_rows_kernel(const float* __restrict__ logits, int V, int row0,
                                                       int slice_len, int t0, int len,
                                                       const int* __restrict__ targets, float* __restrict__ nll) {
    __shared__ float scratch[4];
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + static_cast<size_t>(r) * V;
    float mx = -INFINITY;
    for (int j = tid; j < V; j += 256) mx = fmaxf(mx, x[j]);
    mx = block_max(mx, scratch);
    float sum = 0.0f;
    for (int j = tid; j < V; j += 256) sum += expf(x[j] - mx);
    sum = block_sum(sum, scratch);
    if (tid == 0) {
        const int m = row0 + r, seq = m / slice_len, t = m - seq * slice_len;
        const size_t at = static_cast<size_t>(seq) * len + t0 + t;
        nll[at] = (logf(sum) + mx) - x[targets[at]];
    }
}

}  // namespace gh

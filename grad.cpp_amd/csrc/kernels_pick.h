// Next-token choice on the GPU, one workgroup per sequence:
// repetition penalty -> arg-max, or temperature -> top-k -> softmax -> top-p ->
// inverse-CDF draw.  Restates logits_with_penalty (src/transformer/text_gen.cpp:14-33),
// the greedy arg-max (:52-60) and sample_from_logits (:135-209), including the
// rules that are easy to lose: the penalty is applied once per occurrence in
// the 50-token window; ties at the top-k threshold survive; a top-p that is
// never reached keeps only the maximum; the final walk is in index order.
#pragma once

#include "kernels_common.h"

namespace gh {

constexpr int kPickThreads = 1024;
constexpr int kPenaltyWindow = 50;  // text_gen.cpp:22
constexpr int kSeqWalkLimit = 4096; // survivors walked by one lane, in exact index order

struct PickParams {
    const float* logits;  // [batch][V]
    float* work;          // [batch][V] scratch
    float* kept_p;        // [batch][V] scratch: surviving probabilities in index order
    int* kept_i;          // [batch][V] scratch: their indices
    int V;
    int* hist;  // [batch][hist_stride] token history (prompt + picks)
    int hist_stride;
    int n_hist;    // tokens currently in the history
    int pick_idx;  // index of this pick (selects the uniform draw)
    int* tok;      // [batch] next input token (written)
    float temperature;
    int top_k;
    float top_p;
    float penalty;
    int greedy;
    const float* uniforms;  // [batch][u_stride] or nullptr
    int u_stride;
    unsigned seed_lo, seed_hi;
    int sort_cap;  // floats of LDS available for the descending sort (power of two)
    int* err;      // set to 1 when top-p needs a sort larger than sort_cap
};

__device__ __forceinline__ unsigned mulhi32(unsigned a, unsigned b) { return __umulhi(a, b); }

// Philox4x32-10; word `lane` of block `block` of stream (key0, key1).
__device__ inline unsigned philox4x32_10(unsigned block, unsigned lane, unsigned k0, unsigned k1) {
    unsigned c0 = block, c1 = 0u, c2 = 0u, c3 = 0u;
#pragma unroll
    for (int r = 0; r < 10; r++) {
        const unsigned hi0 = mulhi32(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const unsigned hi1 = mulhi32(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        const unsigned n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
        c0 = n0;
        c1 = lo1;
        c2 = n2;
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return lane == 0 ? c0 : lane == 1 ? c1 : lane == 2 ? c2 : c3;
}

// Order-preserving map float -> uint (larger float, larger key).
__device__ __forceinline__ unsigned float_key(float f) {
    const unsigned u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(unsigned k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}

// The k-th largest of v[0..n) (k >= 1), duplicates counted: the value
// std::sort(descending)[k-1] of text_gen.cpp:145-148.  8-bit radix select.
__device__ inline float kth_largest(const float* v, int n, int k, unsigned* hist /*256*/,
                                    unsigned* bcast /*2*/) {
    unsigned prefix = 0u, mask = 0u;
    int remaining = k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0u;
        __syncthreads();
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const unsigned key = float_key(v[i]);
            if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int left = remaining;
            int bin = 255;
            for (; bin > 0; bin--) {
                if (static_cast<int>(hist[bin]) >= left) break;
                left -= static_cast<int>(hist[bin]);
            }
            bcast[0] = static_cast<unsigned>(bin);
            bcast[1] = static_cast<unsigned>(left);
        }
        __syncthreads();
        prefix |= bcast[0] << shift;
        mask |= 255u << shift;
        remaining = static_cast<int>(bcast[1]);
        __syncthreads();
    }
    return key_float(prefix);
}

// Descending bitonic sort of s[0..n2), n2 a power of two.
__device__ inline void bitonic_desc(float* s, int n2) {
    for (int k = 2; k <= n2; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < n2; i += blockDim.x) {
                const int ixj = i ^ j;
                if (ixj > i) {
                    const float a = s[i], b = s[ixj];
                    const bool desc = (i & k) == 0;
                    if (desc ? (a < b) : (a > b)) {
                        s[i] = b;
                        s[ixj] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
}

__global__ __launch_bounds__(kPickThreads) void pick_kernel(const PickParams p) {
    extern __shared__ float lds[];  // sort buffer (sort_cap floats), top-p only
    __shared__ float red[kPickThreads / 64];
    __shared__ int redi[kPickThreads / 64];
    __shared__ unsigned hist256[256];
    __shared__ unsigned bcast[2];
    __shared__ int win_tok[kPenaltyWindow];
    __shared__ float fshare[2];
    __shared__ int ishare[2];

    const int b = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
    const int V = p.V;
    const float* logits = p.logits + static_cast<size_t>(b) * V;
    float* work = p.work + static_cast<size_t>(b) * V;
    int* hist = p.hist + static_cast<size_t>(b) * p.hist_stride;

    // ---- logits_with_penalty (text_gen.cpp:14-33)
    for (int i = tid; i < V; i += nt) work[i] = logits[i];
    const int window = min(kPenaltyWindow, p.n_hist);
    if (tid < window) win_tok[tid] = hist[p.n_hist - window + tid];
    __syncthreads();
    if (p.penalty != 1.0f && tid < window) {
        const int id = win_tok[tid];
        bool first = true;
        for (int e = 0; e < tid; e++) first = first && (win_tok[e] != id);
        if (first) {
            int count = 0;
            for (int e = tid; e < window; e++) count += (win_tok[e] == id);
            float v = work[id];
            for (int c = 0; c < count; c++) v = (v > 0.0f) ? v / p.penalty : v * p.penalty;
            work[id] = v;
        }
    }
    __syncthreads();

    int chosen;
    if (p.greedy) {
        // First index of the maximum (strict '>' in text_gen.cpp:55-59).
        float best = -INFINITY;
        int bi = 0x7FFFFFFF;
        for (int i = tid; i < V; i += nt) {
            const float v = work[i];
            if (v > best) {
                best = v;
                bi = i;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, kWave);
            const int oi = __shfl_xor(bi, o, kWave);
            if (ov > best || (ov == best && oi < bi)) {
                best = ov;
                bi = oi;
            }
        }
        if ((tid & 63) == 0) {
            red[tid >> 6] = best;
            redi[tid >> 6] = bi;
        }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < nt / 64; w++) {
                if (red[w] > best || (red[w] == best && redi[w] < bi)) {
                    best = red[w];
                    bi = redi[w];
                }
            }
            // data[0] seeds the scan in the reference, so an all-NaN or -inf row picks 0.
            ishare[0] = (bi == 0x7FFFFFFF) ? 0 : bi;
        }
        __syncthreads();
        chosen = ishare[0];
    } else {
        // ---- sample_from_logits (text_gen.cpp:135-209)
        const float inv_t = 1.0f / p.temperature;
        for (int i = tid; i < V; i += nt) work[i] = work[i] * inv_t;
        __syncthreads();
        if (p.top_k > 0 && p.top_k < V) {
            const float thr = kth_largest(work, V, p.top_k, hist256, bcast);
            for (int i = tid; i < V; i += nt)
                if (work[i] < thr) work[i] = -1e10f;
            __syncthreads();
        }
        // Tensor::softmax (tensor.cpp:421-452)
        float m = -INFINITY;
        for (int i = tid; i < V; i += nt) m = fmaxf(m, work[i]);
        m = block_max(m, red);
        float sum = 0.0f;
        for (int i = tid; i < V; i += nt) {
            const float e = expf(work[i] - m);
            work[i] = e;
            sum += e;
        }
        sum = block_sum(sum, red);
        const float inv_sum = 1.0f / sum;
        for (int i = tid; i < V; i += nt) work[i] *= inv_sum;
        __syncthreads();

        float cutoff = 0.0f;  // keep p >= cutoff; without top-p every entry stays
        if (p.top_p < 1.0f) {
            // Sorted-descending cumulative sum until >= top_p (text_gen.cpp:164-177).
            // Zero probabilities sort last and add nothing, so only the non-zero
            // entries are sorted.
            if (tid == 0) ishare[0] = 0;
            __syncthreads();
            int mine = 0;
            for (int i = tid; i < V; i += nt) mine += (work[i] > 0.0f);
            atomicAdd(&ishare[0], mine);
            __syncthreads();
            const int M = ishare[0];
            __syncthreads();
            if (M > p.sort_cap) {
                if (tid == 0) *p.err = 1;
                cutoff = 2.0f;  // nothing survives; falls through to the V-1 return
            } else {
                int n2 = 1;
                while (n2 < M) n2 <<= 1;
                if (tid == 0) ishare[1] = 0;
                __syncthreads();
                for (int i = tid; i < V; i += nt) {
                    const float v = work[i];
                    if (v > 0.0f) lds[atomicAdd(&ishare[1], 1)] = v;
                }
                for (int i = M + tid; i < n2; i += nt) lds[i] = -1.0f;
                __syncthreads();
                bitonic_desc(lds, n2);
                if (tid == 0) {
                    float cumulative = 0.0f;
                    int cutoff_idx = 0;
                    for (int i = 0; i < M; i++) {
                        cumulative += lds[i];
                        if (cumulative >= p.top_p) {
                            cutoff_idx = i;
                            break;
                        }
                    }
                    fshare[0] = lds[cutoff_idx];
                }
                __syncthreads();
                cutoff = fshare[0];
            }
        }

        // Survivors (p >= cutoff and p > 0), compacted in index order.
        float* kp = p.kept_p + static_cast<size_t>(b) * V;
        int* ki = p.kept_i + static_cast<size_t>(b) * V;
        const int per = (V + nt - 1) / nt;
        const int lo = min(V, tid * per), hi = min(V, lo + per);
        int cnt = 0;
        for (int i = lo; i < hi; i++) cnt += (work[i] >= cutoff && work[i] > 0.0f);
        // exclusive scan of cnt over the block
        __shared__ int scan[kPickThreads];
        scan[tid] = cnt;
        __syncthreads();
        for (int o = 1; o < nt; o <<= 1) {
            const int v = tid >= o ? scan[tid - o] : 0;
            __syncthreads();
            scan[tid] += v;
            __syncthreads();
        }
        int at = scan[tid] - cnt;
        const int S = scan[nt - 1];
        for (int i = lo; i < hi; i++) {
            const float v = work[i];
            if (v >= cutoff && v > 0.0f) {
                kp[at] = v;
                ki[at] = i;
                at++;
            }
        }
        __syncthreads();

        float u;
        if (p.uniforms) {
            u = p.uniforms[static_cast<size_t>(b) * p.u_stride + p.pick_idx];
        } else {
            const unsigned w = philox4x32_10(static_cast<unsigned>(p.pick_idx) >> 2,
                                             static_cast<unsigned>(p.pick_idx) & 3u, p.seed_lo,
                                             p.seed_hi ^ static_cast<unsigned>(b));
            u = static_cast<float>(w >> 8) * (1.0f / 16777216.0f);
        }

        const bool renorm = p.top_p < 1.0f;
        if (S <= kSeqWalkLimit) {
            // One lane, exact index order: total_kept, the division, the walk
            // (text_gen.cpp:178-208).  Dropped entries are zeros and add nothing.
            if (tid == 0) {
                float total = 0.0f;
                if (renorm)
                    for (int i = 0; i < S; i++) total += kp[i];
                const bool divide = renorm && total > 0.0f;
                int pick = V - 1;
                if (u <= 0.0f) {
                    pick = 0;  // `u <= cumulative` already holds at index 0
                } else {
                    float cumulative = 0.0f;
                    for (int i = 0; i < S; i++) {
                        cumulative += divide ? kp[i] / total : kp[i];
                        if (u <= cumulative) {
                            pick = ki[i];
                            break;
                        }
                    }
                }
                ishare[0] = pick;
            }
        } else {
            // Many survivors: each thread sums a contiguous run in index order,
            // one lane walks the run totals and then the run that crosses u.
            const int run = (S + nt - 1) / nt;
            const int rlo = min(S, tid * run), rhi = min(S, rlo + run);
            float part = 0.0f;
            for (int i = rlo; i < rhi; i++) part += kp[i];
            float* parts = reinterpret_cast<float*>(scan);
            __syncthreads();
            parts[tid] = part;
            __syncthreads();
            if (tid == 0) {
                float total = 0.0f;
                if (renorm)
                    for (int t = 0; t < nt; t++) total += parts[t];
                const bool divide = renorm && total > 0.0f;
                int pick = V - 1;
                if (u <= 0.0f) {
                    pick = 0;
                } else {
                    float cumulative = 0.0f;
                    for (int t = 0; t < nt; t++) {
                        const float next = cumulative + (divide ? parts[t] / total : parts[t]);
                        if (u <= next) {
                            const int a = min(S, t * run), e = min(S, a + run);
                            for (int i = a; i < e; i++) {
                                cumulative += divide ? kp[i] / total : kp[i];
                                if (u <= cumulative) {
                                    pick = ki[i];
                                    break;
                                }
                            }
                            if (pick == V - 1 && e > a) pick = ki[e - 1];
                            break;
                        }
                        cumulative = next;
                    }
                }
                ishare[0] = pick;
            }
        }
        __syncthreads();
        chosen = ishare[0];
    }

    if (tid == 0) {
        hist[p.n_hist] = chosen;  // tokens.push_back(next_token)
        p.tok[b] = chosen;
    }
}

// ---------------------------------------------------------------------------
// LDS-resident variant: the whole logits row lives in LDS, every pass over it is
// an LDS pass, and the serial parts (sorted running sum, final walk) touch only
// the survivors.  Used whenever vocab + its sort area fit in LDS; the kernel
// above is the fallback for larger vocabularies.

// Suffix scan of a 256-bin histogram by one wavefront: finds the bin holding the
// `want`-th largest key and how many keys are wanted inside it.
__device__ __forceinline__ void select_bin_wave(const unsigned* hist, int want, unsigned* bcast) {
    const int lane = threadIdx.x;  // wave 0 only
    unsigned c[4];
#pragma unroll
    for (int q = 0; q < 4; q++) c[q] = hist[4 * lane + q];
    const unsigned mine = (c[0] + c[1]) + (c[2] + c[3]);
    // above = keys in bins of higher lanes
    unsigned incl = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned v = __shfl_down(incl, o, kWave);
        if (lane + o < 64) incl += v;
    }
    const unsigned above = incl - mine;
    if (static_cast<unsigned>(want) > above && static_cast<unsigned>(want) <= above + mine) {
        unsigned left = static_cast<unsigned>(want) - above;
        int q = 3;
        for (; q > 0; q--) {
            if (c[q] >= left) break;
            left -= c[q];
        }
        bcast[0] = static_cast<unsigned>(4 * lane + q);
        bcast[1] = left;
    }
}

__device__ inline float kth_largest_lds(const float* v, int n, int k, unsigned* hist, unsigned* bcast) {
    unsigned prefix = 0u, mask = 0u;
    int remaining = k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0u;
        __syncthreads();
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const unsigned key = float_key(v[i]);
            if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (threadIdx.x < 64) select_bin_wave(hist, remaining, bcast);
        __syncthreads();
        prefix |= bcast[0] << shift;
        mask |= 255u << shift;
        remaining = static_cast<int>(bcast[1]);
    }
    return key_float(prefix);
}

// Ascending bitonic sort of ints, n2 a power of two.
__device__ inline void bitonic_asc_int(int* s, int n2) {
    for (int k = 2; k <= n2; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < n2; i += blockDim.x) {
                const int ixj = i ^ j;
                if (ixj > i) {
                    const int a = s[i], b = s[ixj];
                    const bool asc = (i & k) == 0;
                    if (asc ? (a > b) : (a < b)) {
                        s[i] = b;
                        s[ixj] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
}

__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    int r = 0;
    for (int w = 0; w < nw; w++) r += scratch[w];
    return r;
}

constexpr int kOrderedWalkLimit = 2048;  // survivors sorted by index and walked by one lane

__global__ __launch_bounds__(kPickThreads) void pick_lds_kernel(const PickParams p) {
    extern __shared__ float lds[];  // [V] logits -> probabilities, then [sort_cap] sort area
    __shared__ float red[kPickThreads / 64];
    __shared__ int redi[kPickThreads / 64];
    __shared__ unsigned hist256[256];
    __shared__ unsigned bcast[2];
    __shared__ int win_tok[kPenaltyWindow];
    __shared__ float fshare[2];
    __shared__ int ishare[2];

    const int b = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
    const int V = p.V;
    const float* logits = p.logits + static_cast<size_t>(b) * V;
    float* val = lds;
    float* srt = lds + V;
    int* hist = p.hist + static_cast<size_t>(b) * p.hist_stride;

    // ---- logits_with_penalty (text_gen.cpp:14-33)
    for (int i = tid; i < V; i += nt) val[i] = logits[i];
    const int window = min(kPenaltyWindow, p.n_hist);
    if (tid < window) win_tok[tid] = hist[p.n_hist - window + tid];
    __syncthreads();
    if (p.penalty != 1.0f && tid < window) {
        const int id = win_tok[tid];
        bool first = true;
        for (int e = 0; e < tid; e++) first = first && (win_tok[e] != id);
        if (first) {
            int count = 0;
            for (int e = tid; e < window; e++) count += (win_tok[e] == id);
            float v = val[id];
            for (int c = 0; c < count; c++) v = (v > 0.0f) ? v / p.penalty : v * p.penalty;
            val[id] = v;
        }
    }
    __syncthreads();

    int chosen;
    if (p.greedy) {
        float best = -INFINITY;
        int bi = 0x7FFFFFFF;
        for (int i = tid; i < V; i += nt) {
            const float v = val[i];
            if (v > best) {
                best = v;
                bi = i;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, kWave);
            const int oi = __shfl_xor(bi, o, kWave);
            if (ov > best || (ov == best && oi < bi)) {
                best = ov;
                bi = oi;
            }
        }
        if ((tid & 63) == 0) {
            red[tid >> 6] = best;
            redi[tid >> 6] = bi;
        }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < nt / 64; w++) {
                if (red[w] > best || (red[w] == best && redi[w] < bi)) {
                    best = red[w];
                    bi = redi[w];
                }
            }
            ishare[0] = (bi == 0x7FFFFFFF) ? 0 : bi;
        }
        __syncthreads();
        chosen = ishare[0];
    } else {
        // ---- sample_from_logits (text_gen.cpp:135-209)
        const float inv_t = 1.0f / p.temperature;
        for (int i = tid; i < V; i += nt) val[i] = val[i] * inv_t;
        __syncthreads();
        if (p.top_k > 0 && p.top_k < V) {
            const float thr = kth_largest_lds(val, V, p.top_k, hist256, bcast);
            for (int i = tid; i < V; i += nt)
                if (val[i] < thr) val[i] = -1e10f;
            __syncthreads();
        }
        float m = -INFINITY;
        for (int i = tid; i < V; i += nt) m = fmaxf(m, val[i]);
        m = block_max(m, red);
        float sum = 0.0f;
        for (int i = tid; i < V; i += nt) {
            const float e = expf(val[i] - m);
            val[i] = e;
            sum += e;
        }
        sum = block_sum(sum, red);
        const float inv_sum = 1.0f / sum;
        int nonzero = 0;
        for (int i = tid; i < V; i += nt) {
            const float pr = val[i] * inv_sum;
            val[i] = pr;
            nonzero += (pr > 0.0f);
        }
        int S = block_sum_int(nonzero, redi);  // entries with p > 0

        if (p.top_p < 1.0f) {
            float cutoff;
            if (S > p.sort_cap) {
                if (tid == 0) *p.err = 1;
                cutoff = 2.0f;
            } else {
                int n2 = 1;
                while (n2 < S) n2 <<= 1;
                if (tid == 0) ishare[1] = 0;
                __syncthreads();
                for (int i = tid; i < V; i += nt) {
                    const float v = val[i];
                    if (v > 0.0f) srt[atomicAdd(&ishare[1], 1)] = v;
                }
                for (int i = S + tid; i < n2; i += nt) srt[i] = -1.0f;
                __syncthreads();
                bitonic_desc(srt, n2);
                if (tid == 0) {
                    float cumulative = 0.0f;
                    int cutoff_idx = 0;
                    for (int i = 0; i < S; i++) {
                        cumulative += srt[i];
                        if (cumulative >= p.top_p) {
                            cutoff_idx = i;
                            break;
                        }
                    }
                    fshare[0] = srt[cutoff_idx];
                }
                __syncthreads();
                cutoff = fshare[0];
            }
            int kept = 0;
            for (int i = tid; i < V; i += nt) {
                const float v = val[i];
                if (v < cutoff) val[i] = 0.0f;
                else kept += (v > 0.0f);
            }
            S = block_sum_int(kept, redi);
        }
        __syncthreads();

        float u;
        if (p.uniforms) {
            u = p.uniforms[static_cast<size_t>(b) * p.u_stride + p.pick_idx];
        } else {
            const unsigned w = philox4x32_10(static_cast<unsigned>(p.pick_idx) >> 2,
                                             static_cast<unsigned>(p.pick_idx) & 3u, p.seed_lo,
                                             p.seed_hi ^ static_cast<unsigned>(b));
            u = static_cast<float>(w >> 8) * (1.0f / 16777216.0f);
        }
        const bool renorm = p.top_p < 1.0f;

        if (S <= kOrderedWalkLimit && S <= p.sort_cap) {
            // Few survivors: list their indices, sort ascending, and let one lane
            // do the exact index-order sums (text_gen.cpp:178-208).
            int* idx = reinterpret_cast<int*>(srt);
            int n2 = 1;
            while (n2 < S) n2 <<= 1;
            if (tid == 0) ishare[1] = 0;
            __syncthreads();
            for (int i = tid; i < V; i += nt)
                if (val[i] > 0.0f) idx[atomicAdd(&ishare[1], 1)] = i;
            for (int i = S + tid; i < n2; i += nt) idx[i] = 0x7FFFFFFF;
            __syncthreads();
            bitonic_asc_int(idx, n2);
            if (tid == 0) {
                float total = 0.0f;
                if (renorm)
                    for (int i = 0; i < S; i++) total += val[idx[i]];
                const bool divide = renorm && total > 0.0f;
                int pick = V - 1;
                if (u <= 0.0f) {
                    pick = 0;
                } else {
                    float cumulative = 0.0f;
                    for (int i = 0; i < S; i++) {
                        const float pr = val[idx[i]];
                        cumulative += divide ? pr / total : pr;
                        if (u <= cumulative) {
                            pick = idx[i];
                            break;
                        }
                    }
                }
                ishare[0] = pick;
            }
        } else {
            // Many survivors: every thread sums a contiguous run of the row in
            // index order, one lane walks the run totals, then the crossing run.
            const int run = (V + nt - 1) / nt;
            const int lo = min(V, tid * run), hi = min(V, lo + run);
            float part = 0.0f;
            for (int i = lo; i < hi; i++) part += val[i];
            float* parts = srt;  // sort area is free again (nt <= sort_cap whenever this path runs)
            __syncthreads();
            parts[tid] = part;
            __syncthreads();
            if (tid == 0) {
                float total = 0.0f;
                if (renorm)
                    for (int t = 0; t < nt; t++) total += parts[t];
                const bool divide = renorm && total > 0.0f;
                int pick = V - 1;
                if (u <= 0.0f) {
                    pick = 0;
                } else {
                    float cumulative = 0.0f;
                    for (int t = 0; t < nt; t++) {
                        const float next = cumulative + (divide ? parts[t] / total : parts[t]);
                        if (u <= next) {
                            const int a = min(V, t * run), e = min(V, a + run);
                            int last = -1;
                            bool found = false;
                            for (int i = a; i < e; i++) {
                                const float pr = val[i];
                                if (pr > 0.0f) last = i;
                                cumulative += divide ? pr / total : pr;
                                if (u <= cumulative && pr > 0.0f) {
                                    pick = i;
                                    found = true;
                                    break;
                                }
                            }
                            if (!found && last >= 0) pick = last;
                            break;
                        }
                        cumulative = next;
                    }
                }
                ishare[0] = pick;
            }
        }
        __syncthreads();
        chosen = ishare[0];
    }

    if (tid == 0) {
        hist[p.n_hist] = chosen;
        p.tok[b] = chosen;
    }
}

}  // namespace gh

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

struct PickParams {
    const float* logits;  // [batch][V]
    float* work;          // [batch][work_stride] working rows when they do not fit in LDS
    int work_stride;      // >= V + kPickThreads (passes may read, and discard, floats past V)
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
    int sort_cap;  // floats of LDS work area next to (or instead of) the row
};

// LDS work area of the pick: the small-k selection wants two floats per thread
// and a few more, the fast sampler kFastLdsFloats, and a pass may read up to one
// float per thread past the end of a row held in LDS.
constexpr int kPickWorkFloats = 2 * kPickThreads + 64;

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

// One pass of the workgroup over v[0..n): f(i, v[i]) for i = tid, tid + nt, ...
// Eight loads are issued before the first use, so a row in global memory costs
// one memory latency per eight elements of a thread, not one per element.
// f may store to v[i].  nt: threads of the workgroup (a caller that knows it at
// compile time passes it; blockDim.x is a load from the dispatch packet).
template <class F>
__device__ __forceinline__ void row_pass(const float* v, int n, F f, int nt = blockDim.x) {
    int i = threadIdx.x;
    for (; i + 7 * nt < n; i += 8 * nt) {
        float x[8];
#pragma unroll
        for (int q = 0; q < 8; q++) x[q] = v[i + q * nt];
#pragma unroll
        for (int q = 0; q < 8; q++) f(i + q * nt, x[q]);
    }
    if (i < n) {
        // what is left (fewer than eight elements per thread) goes out as one more round
        // at clamped offsets: one at a time it was up to seven dependent trips to memory
        float x[8];
#pragma unroll
        for (int q = 0; q < 8; q++) x[q] = v[min(i + q * nt, n - 1)];
#pragma unroll
        for (int q = 0; q < 8; q++)
            if (i + q * nt < n) f(i + q * nt, x[q]);
    }
}

// f(i, get(i)) for i = lo .. hi - 1 in that order, the values fetched eight at a
// time; f returns false to stop.
template <class Get, class F>
__device__ __forceinline__ void run_pass(Get get, int lo, int hi, F f) {
    int i = lo;
    for (; i + 8 <= hi; i += 8) {
        float x[8];
#pragma unroll
        for (int q = 0; q < 8; q++) x[q] = get(i + q);
#pragma unroll
        for (int q = 0; q < 8; q++)
            if (!f(i + q, x[q])) return;
    }
    for (; i < hi; i++)
        if (!f(i, get(i))) return;
}

// ---------------------------------------------------------------------------
// The working copy of the logits row ("the row") lives in LDS when vocab plus
// the work area fit there, in global memory (cached in L2, read and written by
// this workgroup only) otherwise.  Every pass below goes over the row through a
// plain pointer; the serial parts touch only the survivors of the cuts.

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

__device__ inline float kth_largest_lds(const float* v, int n, int k, unsigned* hist, unsigned* bcast,
                                        int nt = blockDim.x) {
    unsigned prefix = 0u, mask = 0u;
    int remaining = k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += nt) hist[i] = 0u;
        __syncthreads();
        // Keys cluster in a few bins (same sign and exponent), so lanes that hit
        // the same bin are counted with one atomic per wavefront.
        const int n_round = (n + nt - 1) / nt * nt;
        for (int i = threadIdx.x; i < n_round; i += nt) {
            unsigned key = 0u;
            bool active = false;
            if (i < n) {
                key = float_key(v[i]);
                active = (key & mask) == prefix;
            }
            const unsigned bin = (key >> shift) & 255u;
            // up to two crowded bins are counted once per wavefront; what is left is
            // spread out and goes through per-lane atomics
            unsigned long long todo = __ballot(active);
            for (int rep = 0; rep < 2 && todo; rep++) {
                const int leader = __ffsll(static_cast<long long>(todo)) - 1;
                const unsigned lb = __builtin_amdgcn_readlane(bin, leader);
                const unsigned long long same = __ballot(active && bin == lb);
                if ((threadIdx.x & 63) == leader) atomicAdd(&hist[lb], static_cast<unsigned>(__popcll(same)));
                if (bin == lb) active = false;
                todo &= ~same;
            }
            if (active) atomicAdd(&hist[bin], 1u);
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

// The k-th largest of v[0..n) for small k, without passes over radix digits:
// the k-th largest of the per-thread maxima is a lower bound T of the answer (at
// least k elements are >= T), the elements >= T are few, and the answer is the
// k-th largest of those.  Falls back to the radix select when k exceeds the
// workgroup size or `work` (work_cap floats) cannot hold 2 * nt + 16.
__device__ __forceinline__ float kth_largest_block(const float* v, int n, int k, float* work, int work_cap,
                                          unsigned* hist, unsigned* bcast, int* ishare,
                                          int nt = blockDim.x) {
    const int tid = threadIdx.x;
    if (k > nt || work_cap < 2 * nt + 16) return kth_largest_lds(v, n, k, hist, bcast, nt);
    float mx = -INFINITY;
    row_pass(v, n, [&](int, float x) { mx = fmaxf(mx, x); }, nt);
    work[tid] = mx;
    if (tid == 0) ishare[1] = 0;
    __syncthreads();
    // one maximum per thread: a radix select over them is four short passes
    const float T = kth_largest_lds(work, nt, k, hist, bcast, nt);
    __syncthreads();
    float* cand = work + nt;  // [nt + 16]
    row_pass(v, n, [&](int, float x) {
        if (x >= T) {
            const int slot = atomicAdd(&ishare[1], 1);
            if (slot < nt) cand[slot] = x;
        }
    }, nt);
    __syncthreads();
    const int c = ishare[1];
    __syncthreads();
    if (c > nt) return kth_largest_lds(v, n, k, hist, bcast, nt);
    {
        const float mine = tid < c ? cand[tid] : -INFINITY;
        for (int j = c + tid; j < ((c + 15) & ~15); j += nt) cand[j] = -INFINITY;  // pad to 16
        __syncthreads();
        int rank = 0;
        for (int j0 = 0; j0 < c; j0 += 16) {
            float o[16];
#pragma unroll
            for (int q = 0; q < 16; q++) o[q] = cand[j0 + q];
#pragma unroll
            for (int q = 0; q < 16; q++) rank += (o[q] > mine) || (o[q] == mine && j0 + q < tid);
        }
        if (tid < c && rank == k - 1) bcast[0] = __float_as_uint(mine);
    }
    __syncthreads();
    return __uint_as_float(bcast[0]);
}

// The sampler's tail for at most 64 survivors of the top-k cut, run by one
// wavefront with lane i holding survivor i in index order: softmax, top-p,
// renormalisation and the inverse-CDF walk (text_gen.cpp:156-208).  Every sum the
// reference forms in index or sorted order is formed in that same order here
// (entries cut by top-k are exact zeros there and add nothing).
__device__ __forceinline__ int pick_small_wave(const float* val, const int* cidx, int S, float top_p, float u,
                                      int V, float* scratch /* >= 256 floats */) {
    const int lane = threadIdx.x & 63;
    int* sidx = reinterpret_cast<int*>(scratch);  // [64] survivor indices, ascending
    float* se = scratch + 64;                     // [64] values in index order, zero padded
    float* sp = scratch + 128;                    // [64] probabilities, descending, zero padded
    // index order (all loops run a fixed 64 rounds over padded arrays so that
    // their LDS reads can be issued together)
    const int my = lane < S ? cidx[lane] : 0x7FFFFFFF;
    sidx[lane] = my;
    __builtin_amdgcn_wave_barrier();
    int rank = 0;
#pragma unroll
    for (int j = 0; j < 64; j++) rank += (sidx[j] < my);
    __builtin_amdgcn_wave_barrier();
    if (lane < S) sidx[rank] = my;
    __builtin_amdgcn_wave_barrier();
    const int idx = lane < S ? sidx[lane] : 0;
    const float v = lane < S ? val[idx] : -INFINITY;
    const float m = wave_max(v);
    const float e = lane < S ? expf(v - m) : 0.0f;
    se[lane] = e;
    __builtin_amdgcn_wave_barrier();
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 64; j++) sum += se[j];  // index order; padding adds exact zeros
    float pr = e * (1.0f / sum);
    bool keep = lane < S && pr > 0.0f;
    __builtin_amdgcn_wave_barrier();
    se[lane] = pr;
    __builtin_amdgcn_wave_barrier();
    if (top_p < 1.0f) {
        int r = 0;
#pragma unroll
        for (int j = 0; j < 64; j++) {
            const float pj = se[j];
            r += (pj > pr) || (pj == pr && j < lane);
        }
        sp[r] = pr;  // ranks are a permutation of 0..63: padding zeros land at the end
        __builtin_amdgcn_wave_barrier();
        float cumulative = 0.0f, cutoff = 0.0f;
        bool found = false;
#pragma unroll
        for (int j = 0; j < 64; j++) {
            const float x = sp[j];
            cumulative += x;
            if (!found && j < S && cumulative >= top_p) {
                cutoff = x;
                found = true;
            }
        }
        if (!found) cutoff = sp[0];  // never reached: only the maximum survives
        keep = keep && pr >= cutoff;
        if (!keep) pr = 0.0f;
        __builtin_amdgcn_wave_barrier();
        se[lane] = pr;
        __builtin_amdgcn_wave_barrier();
        float total = 0.0f;
#pragma unroll
        for (int j = 0; j < 64; j++) total += se[j];  // cut entries add an exact zero
        if (total > 0.0f) pr = pr / total;
        __builtin_amdgcn_wave_barrier();
        se[lane] = pr;
        __builtin_amdgcn_wave_barrier();
    }
    int chosen = V - 1;
    if (u <= 0.0f) {
        chosen = 0;
    } else {
        float cumulative = 0.0f;
        bool found = false;
#pragma unroll
        for (int j = 0; j < 64; j++) {
            cumulative += se[j];
            if (!found && j < S && u <= cumulative) {
                chosen = sidx[j];
                found = true;
            }
        }
    }
    return chosen;
}

// ---------------------------------------------------------------------------
// Fast sampler for a small top-k (the usual 20..64): no pass over radix digits
// and no serial loop over LDS.
//
// Wave-level helpers: a value per lane, lane order = list order.

// Number of prefixes x[0], x[0] + x[1], ... (added strictly left to right, the
// order a serial loop over the list uses) that are below thr.  The x are >= 0, so
// the prefixes never decrease and this is the index of the first prefix that
// reaches thr (n when none does).  Same value in every lane.
__device__ __forceinline__ int wave_prefixes_below(float x, int n, float thr) {
    float acc = 0.0f;
    int below = 0;
#pragma unroll 8
    for (int j = 0; j < n; j++) {
        acc += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), j));
        below += (acc < thr) ? 1 : 0;
    }
    return below;
}

// x[0] + ... + x[n-1] left to right, in every lane.
__device__ __forceinline__ float wave_total_in_order(float x, int n) {
    float acc = 0.0f;
#pragma unroll 8
    for (int j = 0; j < n; j++) acc += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), j));
    return acc;
}

// Running sums in the order a serial loop forms them, p[l] = ((x[0] + x[1]) + ...) + x[l],
// for the first n lanes (n a multiple of 8, x >= 0 and 0 from lane n on), in n steps of
// one shifted addition each: after step t lane l holds x[l - t] + ... + x[l] added left to
// right, and once t reaches l that is the whole prefix and stays it (what shifts into
// lane 0 is a zero, and 0 + x[0] is x[0]).  No trip to LDS and no lane-to-scalar move.
__device__ __forceinline__ float wave_serial_prefix(float x, int n) {
    float acc = x;
    for (int t = 0; t < n; t += 8) {
#pragma unroll
        for (int q = 0; q < 8; q++)
            acc = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc), 0x138 /* wave_shr:1 */, 0xF, 0xF,
                                                             true))
                  + x;
    }
    return acc;
}

// Developer aid (-DGH_PICK_TICKS): time thread 0 of workgroup 0 spends in each stage of
// the fast sampler, summed over picks, on the 100 MHz clock.
#ifdef GH_PICK_TICKS
__device__ unsigned long long g_pick_ticks[32];
#define PTICK_BEGIN() unsigned long long ptick_last_ = __builtin_amdgcn_s_memrealtime()
#define PTICK(i)                                                             \
    do {                                                                     \
        if (threadIdx.x == 0 && blockIdx.x == 0) {                           \
            const unsigned long long t_ = __builtin_amdgcn_s_memrealtime();  \
            g_pick_ticks[i] += t_ - ptick_last_;                             \
            ptick_last_ = t_;                                                \
        }                                                                    \
    } while (0)
#else
#define PTICK_BEGIN() do {} while (0)
#define PTICK(i) do {} while (0)
#endif

constexpr int kFastCandCap = 512;
// LDS floats the fast sampler needs: candidate values, indices and ranks, the
// survivors (value, index, index rank) and a permutation area.
constexpr int kFastLdsFloats = 3 * kFastCandCap + 3 * 64 + 128;

// Temperature, top-k, softmax, top-p and the draw (text_gen.cpp:135-209) for
// 0 < top_k <= 64 over val[0..V) (penalised, unscaled logits in LDS), by the
// whole workgroup.  Returns the chosen id, or -1 when this path does not apply
// (too many values tie near the threshold); val is left untouched either way.
//
// The k-th largest is found without sorting the row: take each thread's
// maximum, then in every wavefront the R-th largest of those (R = ceil(k /
// wavefronts)); the smallest of these, T, has at least k values at or above it
// and only a few more.  Those candidates are ranked against each other by all
// threads at once, which also leaves the survivors of the cut in descending
// order.  One wavefront finishes: every sum the reference forms in index order
// (softmax denominator, renormalisation, the final walk) or in descending order
// (top-p) is formed in that order, lane by lane.
// NT = threads of the workgroup and ROUNDS = elements per thread (compile time,
// so that a thread's elements sit at immediate offsets and stay in registers
// between the two passes); needs V <= ROUNDS * NT.
// ids: the token id of every element when val is not a row of logits but a list of
// candidates from one (index order means token order); outside: the largest value
// that is not in val, below which the k-th largest must not fall for the cut to be
// the row's (-1 otherwise); last_id: the row's last token id (the walk's answer when
// rounding keeps the running sum below the draw, text_gen.cpp:202-208).
template <int NT, int ROUNDS>
__device__ inline int sample_topk_fast(const float* val, int V, float inv_t, int k, float top_p, float u,
                                       float* work, float* red, int* ishare, const int* ids = nullptr,
                                       float outside = -INFINITY, int last_id = 0) {
    constexpr int nt = NT, nw = NT / 64;
    static_assert(ROUNDS <= 64, "one mask bit per element of a thread");
    static_assert(NT >= kFastCandCap, "every candidate needs a thread");
    // Inside a kernel that picks once per iteration of a long loop, everything below
    // that depends only on the thread and on V is loop-invariant; hoisted, the
    // per-round masks alone are 2 * ROUNDS scalar registers, which end up spilled to
    // scratch memory and reloaded one trip per round.  Opaque copies keep them here.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid), "+s"(V));
    const int lane = tid & 63, wave = tid >> 6;
    if (V > ROUNDS * NT) return -1;
    PTICK_BEGIN();
    float* cand_v = work;
    int* cand_i = reinterpret_cast<int*>(work + kFastCandCap);
    int* rank = cand_i + kFastCandCap;
    float* sv = work + 3 * kFastCandCap;  // [64] survivors, descending
    int* si = reinterpret_cast<int*>(sv + 64);
    int* ridx = si + 64;                  // [64] position of each survivor in index order
    int* perm = ridx + 64;                // [128]

    // element r * NT + tid of the row, scaled; -inf past the end
    // (all reads first, at clamped offsets, so that they are in flight together)
    float x[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) x[r] = val[min(r * NT + tid, V - 1)];
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) x[r] = (tid < V - r * NT) ? x[r] * inv_t : -INFINITY;
    float mx = x[0];
#pragma unroll
    for (int r = 1; r < ROUNDS; r++) mx = fmaxf(mx, x[r]);
    const int R = (k + nw - 1) / nw;
    float sel = mx, rest = mx;
    for (int r = 0; r < R; r++) {
        sel = wave_max(rest);
        const unsigned long long at = __ballot(rest == sel);
        if (lane == __ffsll(static_cast<long long>(at)) - 1) rest = -INFINITY;
    }
    if (lane == 0) red[wave] = sel;
    if (tid == 0) ishare[1] = 0;
    if (tid < kFastCandCap) rank[tid] = 0;
    if (tid < 64) {
        sv[tid] = -INFINITY;
        ridx[tid] = 0;
    }
    __syncthreads();
    PTICK(0);
    float T = red[0];
    for (int w = 1; w < nw; w++) T = fminf(T, red[w]);

    if (!(T > -INFINITY)) return -1;  // some wavefront has fewer than R finite values
    // candidates: values >= T with their indices, in arbitrary slots
    unsigned long long mine = 0ull;
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) mine |= static_cast<unsigned long long>(x[r] >= T) << r;
    // slots: one atomic per wavefront (a running count over its lanes), not one per thread
    const int mine_n = __popcll(mine);
    const int upto = wave_inclusive_scan(mine_n);
    const int wave_n = __builtin_amdgcn_readlane(upto, 63);
    int wave_base = 0;
    if (wave_n) {  // uniform
        if (lane == 63) wave_base = atomicAdd(&ishare[1], wave_n);
        wave_base = __builtin_amdgcn_readlane(wave_base, 63);
    }
    if (mine) {
        int slot = wave_base + upto - mine_n;
        while (mine) {
            const int r = __ffsll(static_cast<long long>(mine)) - 1;
            mine &= mine - 1ull;
            if (slot < kFastCandCap) {
                const int i = r * nt + tid;
                cand_v[slot] = val[i] * inv_t;
                cand_i[slot] = ids ? ids[i] : i;
            }
            slot++;
        }
    }
    __syncthreads();
    PTICK(1);
    const int c = ishare[1];
#ifdef GH_PICK_TICKS
    if (threadIdx.x == 0 && blockIdx.x == 0) g_pick_ticks[14] += c;
#endif
    if (c > kFastCandCap || c < k) return -1;  // uniform: every thread reads the same count

    // descending rank of every candidate (ties: lower slot first), all threads:
    // candidate L = tid % P is compared with one slice of the list per group of P threads
    {
        int P = 64;
        while (P < c) P <<= 1;
        const int parts = nt / P, L = tid & (P - 1), part = tid / P;
        const int chunk = (c + parts - 1) / parts;
        const int j0 = part * chunk, j1 = min(c, j0 + chunk);
        const float me = L < c ? cand_v[L] : INFINITY;
        int partial = 0;
#pragma unroll 4
        for (int j = j0; j < j1; j++) {
            const float o = cand_v[j];  // same address in every lane: one broadcast read
            partial += (o > me) || (o == me && j < L);
        }
        if (L < c && partial) atomicAdd(&rank[L], partial);
    }
    __syncthreads();
    PTICK(2);
    if (tid < c) {
        const int r = rank[tid];
        if (r < 64) {
            sv[r] = cand_v[tid];
            si[r] = cand_i[tid];
        }
    }
    __syncthreads();
    PTICK(3);
    // the cut keeps ties at the threshold (text_gen.cpp:150-154)
    const float thr = sv[k - 1];
    if (!(outside < thr)) return -1;  // uniform
    const unsigned long long kept = __ballot(sv[lane] >= thr);
    const int S = __popcll(kept);
#ifdef GH_PICK_TICKS
    if (threadIdx.x == 0 && blockIdx.x == 0) g_pick_ticks[15] += S;
#endif
    if (S == 64 && c > 64) return -1;  // the ties may run past what one wavefront holds
    {
        // position of every survivor in index order
        const int chunk = (S + nw - 1) / nw;
        const int j0 = wave * chunk, j1 = min(S, j0 + chunk);
        const int me = lane < S ? si[lane] : 0;
        int partial = 0;
        for (int j = j0; j < j1; j++) partial += si[j] < me;
        if (lane < S && partial) atomicAdd(&ridx[lane], partial);
    }
    __syncthreads();
    PTICK(4);
    if (tid < 64) {
        const int n = min(64, (S + 7) & ~7);
        const bool live = lane < S;
        const float v = sv[lane];
        const int ri = live ? ridx[lane] : lane;
        const float e = live ? expf(v - sv[0]) : 0.0f;
        float* in_order = reinterpret_cast<float*>(perm);  // [64] a value per survivor, index order
        // index-order copies of e and of the token ids
        perm[lane] = 0;
        perm[64 + lane] = 0x7FFFFFFF;
        __builtin_amdgcn_wave_barrier();
        if (live) {
            in_order[ri] = e;
            perm[64 + ri] = si[lane];
        }
        __builtin_amdgcn_wave_barrier();
        const float eo = in_order[lane];
        const float inv_sum =
            1.0f / __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wave_serial_prefix(eo, n)), n - 1));
        float po = eo * inv_sum;  // index order
        if (top_p < 1.0f) {
            float pr = e * inv_sum;  // descending order
            // first position whose running sum reaches top_p; never reached: only the
            // maximum survives
            const float run = wave_serial_prefix(pr, n);
            const int reach = __popcll(__ballot(lane < n && run < top_p));
            const int at = reach < S ? reach : 0;
            const float cutoff = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pr), at));
            if (!(live && pr > 0.0f && pr >= cutoff)) pr = 0.0f;
            in_order[lane] = 0.0f;
            __builtin_amdgcn_wave_barrier();
            if (live) in_order[ri] = pr;
            __builtin_amdgcn_wave_barrier();
            po = in_order[lane];
            const float total = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wave_serial_prefix(po, n)), n - 1));
            if (total > 0.0f) po = po / total;
        }
        int chosen = 0;
        if (u > 0.0f) {
            const float run = wave_serial_prefix(po, n);
            const int hit = __popcll(__ballot(lane < n && run < u));  // first i with u <= cumulative
            chosen = hit < S ? perm[64 + hit] : (ids ? last_id : V - 1);
        }
        if (tid == 0) ishare[1] = chosen;
    }
    PTICK(5);
    __syncthreads();
    PTICK(6);
    return ishare[1];
}

// Ordered sums by the whole workgroup: x(0) + x(1) + ... with x(i) >= 0 from
// get(i).  Every thread adds a contiguous run left to right, the run totals are
// combined left to right, so the result is the serial sum up to regrouping.
// parts: one float of LDS per wavefront.  Every thread must call these.
template <class Get>
__device__ inline float block_ordered_total(Get get, int n, float* parts, int nt = blockDim.x) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
    // an odd run length: lane l starts at l * run, and an even stride would put
    // many lanes of a wavefront on the same LDS bank at every step of the walk
    const int run = ((n + nt - 1) / nt) | 1;
    const int lo = min(n, tid * run), hi = min(n, lo + run);
    float part = 0.0f;
    run_pass(get, lo, hi, [&](int, float x) {
        part += x;
        return true;
    });
    const float wtotal = wave_total_in_order(part, 64);
    __syncthreads();
    if (lane == 0) parts[wave] = wtotal;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < nw; w++) total += parts[w];
    __syncthreads();
    return total;
}

// First i in [0, n) whose running sum x(0) + ... + x(i) reaches thr, n when none
// does.  slot: one int of LDS.
template <class Get>
__device__ inline int block_first_reach(Get get, int n, float thr, float* parts, int* slot,
                                        int nt = blockDim.x) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // an odd run length: lane l starts at l * run, and an even stride would put
    // many lanes of a wavefront on the same LDS bank at every step of the walk
    const int run = ((n + nt - 1) / nt) | 1;
    const int lo = min(n, tid * run), hi = min(n, lo + run);
    float part = 0.0f;
    run_pass(get, lo, hi, [&](int, float x) {
        part += x;
        return true;
    });
    // sum of the runs of lower lanes of this wavefront, then of lower wavefronts
    float before = 0.0f;
#pragma unroll 8
    for (int j = 0; j < 64; j++) {
        const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(part), j));
        before += (j < lane) ? pj : 0.0f;
    }
    const float wtotal = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(before + part), 63));
    __syncthreads();
    if (lane == 0) parts[wave] = wtotal;
    if (tid == 0) *slot = n;
    __syncthreads();
    float base = 0.0f;
    for (int w = 0; w < wave; w++) base += parts[w];
    base += before;
    if (base < thr) {
        float cumulative = base;
        run_pass(get, lo, hi, [&](int i, float x) {
            cumulative += x;
            if (cumulative >= thr) {
                atomicMin(slot, i);
                return false;
            }
            return true;
        });
    }
    __syncthreads();
    const int at = *slot;
    __syncthreads();
    return at;
}


// The top-p cut without sorting (text_gen.cpp:160-177).  The reference sorts the
// probabilities, adds them in descending order until the sum reaches top_p and
// cuts below the value found there.  That value is the largest probability c
// whose upper mass (the sum of everything >= c) reaches top_p, which a bisection
// over the bit patterns of the (positive) probabilities finds in 31 passes of
// compare-and-add.  If even the whole mass stays below top_p the reference keeps
// only the maximum.  NT > 0: the workgroup has NT threads and V <= ROUNDS * NT,
// so a thread's elements stay in registers across the passes; NT == 0 reads the
// row on every pass.
template <int NT, int ROUNDS>
__device__ inline float top_p_cutoff(const float* val, int V, float top_p, float* red) {
    const int tid = threadIdx.x, nt = NT > 0 ? NT : static_cast<int>(blockDim.x);
    float x[ROUNDS];
    float pmax = 0.0f;
    if constexpr (NT > 0) {
#pragma unroll
        for (int r = 0; r < ROUNDS; r++) {
            x[r] = 0.0f;
            if (r * NT < V) {  // uniform; the last round may read (and discard) floats just past V
                const float raw = val[r * NT + tid];
                x[r] = (tid < V - r * NT) ? raw : 0.0f;
            }
            pmax = fmaxf(pmax, x[r]);
        }
    } else {
        row_pass(val, V, [&](int, float v) { pmax = fmaxf(pmax, v); }, nt);
    }
    pmax = block_max(pmax, red, nt);
    __shared__ float sums[2][kPickThreads / 64];
    int calls = 0;
    auto upper_mass = [&](unsigned key) {
        const float t = __uint_as_float(key);
        float mass = 0.0f;
        if constexpr (NT > 0) {
#pragma unroll
            for (int r = 0; r < ROUNDS; r++) mass += (x[r] >= t) ? x[r] : 0.0f;
        } else {
            row_pass(val, V, [&](int, float v) { mass += (v >= t) ? v : 0.0f; }, nt);
        }
        // block sum with one barrier per call: successive calls alternate between two
        // sets of per-wavefront slots
        const float w = wave_sum(mass);
        float* slot = sums[calls & 1];
        calls++;
        if ((tid & 63) == 0) slot[tid >> 6] = w;
        __syncthreads();
        float total = 0.0f;
        for (int q = 0; q < (nt >> 6); q++) total += slot[q];
        return total;
    };
    const unsigned top = __float_as_uint(pmax);  // bit patterns of positive floats order like the floats
    if (top < 1u || upper_mass(1u) < top_p) {
        __syncthreads();
        return pmax;
    }
    // the cut is rarely more than 2^-20 below the maximum: try that as the lower end
    unsigned lo = 1u, hi = top;
    if (top > (20u << 23) && upper_mass(top - (20u << 23)) >= top_p) lo = top - (20u << 23);
    while (lo < hi) {
        const unsigned mid = lo + (hi - lo + 1u) / 2u;
        if (upper_mass(mid) >= top_p) lo = mid;
        else hi = mid - 1u;
    }
    __syncthreads();
    return __uint_as_float(lo);
}

// The pick for sequence b.  val: the working row ([V] floats, LDS or global,
// with one float per thread readable behind it); srt: p.sort_cap floats of LDS.
// Every thread of the workgroup must call it; all get the chosen id.
// coherent: read the logits with device-scope loads (they were written by other
// workgroups of the same running kernel).
// NT: threads of the workgroup.
// Always inlined: each call site knows whether val is LDS or global memory, and
// the row's loads and stores are compiled for that address space.
// The uniform draw of pick p.pick_idx of sequence b: the caller's, or word
// pick_idx of the Philox stream keyed by (seed, sequence), as a 24-bit fraction.
__device__ __forceinline__ float pick_draw(const PickParams& p, int b) {
    if (p.uniforms) return p.uniforms[static_cast<size_t>(b) * p.u_stride + p.pick_idx];
    const unsigned w = philox4x32_10(static_cast<unsigned>(p.pick_idx) >> 2, static_cast<unsigned>(p.pick_idx) & 3u,
                                     p.seed_lo, p.seed_hi ^ static_cast<unsigned>(b));
    return static_cast<float>(w >> 8) * (1.0f / 16777216.0f);
}

// u_ready: the draw when the caller has already formed it (it does not depend on
// the logits, so it can be had while they are still on their way); negative: form it here.
template <bool coherent, int NT>
__device__ __forceinline__ int pick_body(const PickParams& p, int b, float* val, float* srt,
                                         float u_ready = -1.0f) {
    __shared__ float red[kPickThreads / 64];
    __shared__ int redi[kPickThreads / 64];
    __shared__ unsigned hist256[256];
    __shared__ unsigned bcast[2];
    __shared__ int ishare[2];

    constexpr int nt = NT;
    // Opaque copies, as in sample_topk_fast: nothing derived from them is computed
    // ahead of a caller's loop and kept in registers through it.
    int tid = threadIdx.x;
    int V = p.V;
    asm volatile("" : "+v"(tid), "+s"(V));
    const float* logits = p.logits + static_cast<size_t>(b) * V;
    const int* hist = p.hist + static_cast<size_t>(b) * p.hist_stride;

    // ---- logits_with_penalty (text_gen.cpp:14-33)
    // The window's tokens are requested first so that their latency hides behind the row's.
    const int window = min(kPenaltyWindow, p.n_hist);
    int window_token = -1;
    if (tid < window) {
        const int* hp = &hist[p.n_hist - window + tid];
        window_token = coherent ? __hip_atomic_load(hp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *hp;
    }
    // How often each entry of the window occurs, and whether it is the first of its
    // kind (that one applies the penalty, once per occurrence): wavefront 0 holds the
    // window one entry per lane and compares in registers, while the row is on its way.
    int pen_first = 0, pen_times = 0;
    auto count_window = [&]() {
        if (p.penalty != 1.0f && tid < 64) {
            const int id = tid < window ? window_token : -1 - tid;
            int before = 0;
            for (int e = 0; e < window; e++) {
                const int other = __builtin_amdgcn_readlane(id, e);
                before += (e < tid && other == id) ? 1 : 0;
                pen_times += (other == id) ? 1 : 0;
            }
            pen_first = (tid < window && before == 0) ? 1 : 0;
        }
    };
    if (coherent) {
        const __amdgpu_buffer_rsrc_t rs = make_buffer(logits, static_cast<unsigned>(V) * 4u);
        // eight 16-byte loads per thread in flight; reads past the end return zero.  The
        // loop runs over rounds of the whole workgroup, so every wavefront is converged
        // when wavefront 0 counts the window behind the first round of loads (the count
        // reads other lanes' registers: with the loop bound depending on the thread, a
        // vocabulary below four times the window left some of those lanes inactive).
        for (int b0 = 0; b0 < V; b0 += 32 * nt) {
            const int base = b0 + 4 * tid;
            v4i w[8];
#pragma unroll
            for (int q = 0; q < 8; q++) w[q] = coherent_load16(rs, static_cast<unsigned>(base + q * 4 * nt) * 4u);
            if (b0 == 0) count_window();
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const int i = base + q * 4 * nt;
                if (i + 3 < V) {
                    *reinterpret_cast<float4*>(val + i) =
                        make_float4(__int_as_float(w[q].x), __int_as_float(w[q].y), __int_as_float(w[q].z),
                                    __int_as_float(w[q].w));
                } else {
                    if (i < V) val[i] = __int_as_float(w[q].x);
                    if (i + 1 < V) val[i + 1] = __int_as_float(w[q].y);
                    if (i + 2 < V) val[i + 2] = __int_as_float(w[q].z);
                }
            }
        }
    } else {
        row_pass(logits, V, [&](int i, float v) { val[i] = v; }, nt);
        count_window();
    }
    __syncthreads();
    if (p.penalty != 1.0f) {
        // ids come from the session's own history, or from the caller's device memory in the
        // entry point that allocates nothing: one outside the vocabulary is left alone
        if (pen_first && static_cast<unsigned>(window_token) < static_cast<unsigned>(V)) {
            float v = val[window_token];
            for (int c = 0; c < pen_times; c++) v = (v > 0.0f) ? v / p.penalty : v * p.penalty;
            val[window_token] = v;
        }
        __syncthreads();
    }

    int chosen;
    if (p.greedy) {
        float best = -INFINITY;
        int bi = 0x7FFFFFFF;
        row_pass(val, V, [&](int i, float v) {
            if (v > best) {
                best = v;
                bi = i;
            }
        }, nt);
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
        const float u = u_ready >= 0.0f ? u_ready : pick_draw(p, b);
        // elements per thread when a thread keeps its share of the row in registers
        const int per_thread = (V + nt - 1) / nt;
        if (p.top_k > 0 && p.top_k <= 64 && p.top_k < V && p.sort_cap >= kFastLdsFloats && per_thread <= 64) {
            const int c = per_thread <= 32
                              ? sample_topk_fast<NT, 32>(val, V, inv_t, p.top_k, p.top_p, u, srt, red, ishare)
                              : sample_topk_fast<NT, 64>(val, V, inv_t, p.top_k, p.top_p, u, srt, red, ishare);
            __syncthreads();
            if (c >= 0) return c;
        }
        row_pass(val, V, [&](int i, float v) { val[i] = v * inv_t; }, nt);
        __syncthreads();
        if (p.top_k > 0 && p.top_k < V) {
            const float thr = kth_largest_block(val, V, p.top_k, srt, p.sort_cap, hist256, bcast, ishare, nt);
            // Survivors of the cut (ties at the threshold included).  When they fit
            // one wavefront the rest of the sampler runs there.
            int* cidx = reinterpret_cast<int*>(srt);
            if (tid == 0) ishare[1] = 0;
            __syncthreads();
            row_pass(val, V, [&](int i, float v) {
                if (v >= thr) {
                    const int slot = atomicAdd(&ishare[1], 1);
                    if (slot < 64) cidx[slot] = i;
                }
            }, nt);
            __syncthreads();
            const int S0 = ishare[1];
            if (S0 <= 64 && p.sort_cap >= 512) {
                if (tid < 64) {
                    const int c = pick_small_wave(val, cidx, S0, p.top_p, u, V, srt + 64);
                    if (tid == 0) ishare[0] = c;
                }
                __syncthreads();
                const int c = ishare[0];
                __syncthreads();
                return c;
            }
            row_pass(val, V, [&](int i, float v) {
                if (v < thr) val[i] = -1e10f;
            }, nt);
            __syncthreads();
        }
        float m = -INFINITY;
        row_pass(val, V, [&](int, float v) { m = fmaxf(m, v); }, nt);
        m = block_max(m, red, nt);
        float sum = 0.0f;
        row_pass(val, V, [&](int i, float v) {
            const float e = expf(v - m);
            val[i] = e;
            sum += e;
        }, nt);
        sum = block_sum(sum, red, nt);
        const float inv_sum = 1.0f / sum;
        row_pass(val, V, [&](int i, float v) { val[i] = v * inv_sum; }, nt);

        if (p.top_p < 1.0f) {
            float cutoff;
            if (per_thread <= 32) cutoff = top_p_cutoff<NT, 32>(val, V, p.top_p, red);
            else if (per_thread <= 64) cutoff = top_p_cutoff<NT, 64>(val, V, p.top_p, red);
            else cutoff = top_p_cutoff<0, 1>(val, V, p.top_p, red);
            row_pass(val, V, [&](int i, float v) {
                if (v < cutoff) val[i] = 0.0f;
            }, nt);
        }
        __syncthreads();

        // Renormalise by the index-order total of what is left (text_gen.cpp:178-192) and
        // walk the cumulative sums in index order (:202-208); cut entries are exact zeros.
        float* parts = red;
        const bool renorm = p.top_p < 1.0f;
        float total = 1.0f;
        bool divide = false;
        if (renorm) {
            total = block_ordered_total([&](int q) { return val[q]; }, V, parts, nt);
            divide = total > 0.0f;
        }
        if (u <= 0.0f) {
            if (tid == 0) ishare[0] = 0;
        } else {
            const int at = divide ? block_first_reach([&](int q) { return val[q] / total; }, V, u, parts, &ishare[1], nt)
                                  : block_first_reach([&](int q) { return val[q]; }, V, u, parts, &ishare[1], nt);
            if (tid == 0) ishare[0] = at < V ? at : V - 1;
        }
        __syncthreads();
        chosen = ishare[0];
    }
    __syncthreads();
    return chosen;
}

// ROW_LDS: the working row sits in LDS in front of the work area; otherwise in
// p.work.
template <bool ROW_LDS>
__global__ __launch_bounds__(kPickThreads) void pick_kernel(const PickParams p) {
    extern __shared__ __attribute__((aligned(128))) float lds[];
    const int b = blockIdx.x;
    const int chosen =
        ROW_LDS ? pick_body<false, kPickThreads>(p, b, lds, lds + p.V)
                : pick_body<false, kPickThreads>(p, b, p.work + static_cast<size_t>(b) * p.work_stride, lds);
    if (threadIdx.x == 0) {
        p.hist[static_cast<size_t>(b) * p.hist_stride + p.n_hist] = chosen;  // tokens.push_back(next)
        p.tok[b] = chosen;
    }
}

// The greedy pick without a penalty for every sequence of a batched step, and the
// embedding of what it picked, in one launch (text_gen.cpp:52-60, inference.cpp:159-182).
// The logits launch left the largest value and first column of every run of 16 columns
// of every row; one workgroup per sequence takes the first maximum of those, records
// the token in the history and writes the step's input row.
constexpr int kArgmaxThreads = 256;

__global__ __launch_bounds__(kArgmaxThreads) void argmax_embed_kernel(const float2* __restrict__ best, int n16,
                                                                      const DevState* st, int* hist, int hist_stride,
                                                                      int* tok, const float* __restrict__ E,
                                                                      const float* __restrict__ P, float* x, int d) {
    __shared__ float wv[kArgmaxThreads / 64];
    __shared__ int wi[kArgmaxThreads / 64];
    const int b = blockIdx.x, tid = threadIdx.x;
    const int pos = st->pos, at = st->pos + st->hist_lead;
    const float2* row = best + static_cast<size_t>(b) * n16;
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int i0 = 0; i0 < n16; i0 += 4 * kArgmaxThreads) {
        float2 e[4];
#pragma unroll
        for (int q = 0; q < 4; q++) e[q] = row[min(i0 + q * kArgmaxThreads + tid, n16 - 1)];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            // a thread's runs come in rising column order: the first maximum stays
            if (i0 + q * kArgmaxThreads + tid < n16 && e[q].x > bv) {
                bv = e[q].x;
                bi = __float_as_int(e[q].y);
            }
        }
    }
    wave_first_max(bv, bi);
    if ((tid & 63) == 0) {
        wv[tid >> 6] = bv;
        wi[tid >> 6] = bi;
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kArgmaxThreads / 64; w++) {
        if (w == 0 || wv[w] > bv || (wv[w] == bv && wi[w] < bi)) {
            bv = wv[w];
            bi = wi[w];
        }
    }
    const int chosen = bi == 0x7FFFFFFF ? 0 : bi;
    if (tid == 0) {
        hist[static_cast<size_t>(b) * hist_stride + at] = chosen;  // tokens.push_back(next)
        tok[b] = chosen;
    }
    for (int j = tid; j < d; j += kArgmaxThreads) {
        float v = E[static_cast<size_t>(chosen) * d + j];
        if (P) v += P[static_cast<size_t>(pos) * d + j];
        x[static_cast<size_t>(b) * d + j] = v;
    }
}

}  // namespace gh

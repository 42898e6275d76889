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

// How chunks of one (sequence, head) meet without flushing caches: a chunk writes
// its partial (running max m, sum l, unnormalised acc) with device-scope stores,
// waits for them to be acknowledged, then takes a ticket with a device-scope
// atomic; the chunk that draws the last ticket reads all partials back with
// device-scope loads and merges them.
__device__ __forceinline__ void partial_store(float* dst, float v) {
    __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Every thread of the workgroup calls this after its partial_store calls;
// returns true in the workgroup that must merge.
__device__ __forceinline__ bool last_chunk_arrived(unsigned* ticket_ctr, int nchunk, unsigned* lds_slot) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0)
        *lds_slot = __hip_atomic_fetch_add(ticket_ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    return *lds_slot == static_cast<unsigned>(nchunk - 1);
}

__device__ __forceinline__ void attn_merge(const AttnParams& p, int b, int h, int nchunk, int hs) {
    const float* base = p.part + (static_cast<size_t>(b) * p.kv.heads + h) * p.max_chunks * (hs + 2);
    const __amdgpu_buffer_rsrc_t rs = make_buffer(base, static_cast<unsigned>(nchunk * (hs + 2)) * 4u);
    // Element i of the partials through a device-scope load of the 16 bytes around it.
    // The loads of four chunks go out together: one after the other, each waited for,
    // they were three dependent trips to memory per chunk at the very end of the launch,
    // where nothing else is left to hide them.
    auto fetch = [&](int i) { return coherent_load16(rs, static_cast<unsigned>(i & ~3) * 4u); };
    auto pick = [](const v4i& w, int i) { return __int_as_float(w[i & 3]); };
    const int stride = hs + 2;
    if (nchunk <= 4) {
        // everything in one round of loads
        const int tid = threadIdx.x;
        const int jj = tid < hs ? tid : 0;
        v4i wm[4], wl[4], wa[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int at = min(q, nchunk - 1) * stride;
            wm[q] = fetch(at);
            wl[q] = fetch(at + 1);
            wa[q] = fetch(at + 2 + jj);
        }
        float M = -INFINITY;
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (q < nchunk) M = fmaxf(M, pick(wm[q], q * stride));
        float L = 0.0f, o = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (q < nchunk) {
                const float f = expf(pick(wm[q], q * stride) - M);
                L += pick(wl[q], q * stride + 1) * f;
                o += pick(wa[q], q * stride + 2 + jj) * f;
            }
        }
        if (tid < hs && hs <= static_cast<int>(blockDim.x)) {
            p.out[static_cast<size_t>(b) * p.d_model + h * hs + tid] = o * (1.0f / L);
            return;
        }
        if (hs <= static_cast<int>(blockDim.x)) return;
    }
    float M = -INFINITY;
    for (int s0 = 0; s0 < nchunk; s0 += 4) {
        v4i w[4];
#pragma unroll
        for (int q = 0; q < 4; q++) w[q] = fetch(min(s0 + q, nchunk - 1) * stride);
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (s0 + q < nchunk) M = fmaxf(M, pick(w[q], (s0 + q) * stride));
    }
    // every thread forms L (the same additions in the same order); thread j < hs forms output j
    const int tid = threadIdx.x;
    const int jj = tid < hs ? tid : 0;
    float L = 0.0f, o = 0.0f;
    for (int s0 = 0; s0 < nchunk; s0 += 4) {
        v4i wm[4], wl[4], wa[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int at = min(s0 + q, nchunk - 1) * stride;
            wm[q] = fetch(at);
            wl[q] = fetch(at + 1);
            wa[q] = fetch(at + 2 + jj);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (s0 + q < nchunk) {
                const int at = (s0 + q) * stride;
                const float f = expf(pick(wm[q], at) - M);
                L += pick(wl[q], at + 1) * f;
                o += pick(wa[q], at + 2 + jj) * f;
            }
        }
    }
    const float inv = 1.0f / L;
    if (tid < hs) p.out[static_cast<size_t>(b) * p.d_model + h * hs + tid] = o * inv;
    // head sizes beyond the workgroup (none of the shapes in use): the remaining outputs, one at a time
    for (int j = tid + blockDim.x; j < hs; j += blockDim.x) {
        float oj = 0.0f;
        for (int s = 0; s < nchunk; s++)
            oj += pick(fetch(s * stride + 2 + j), s * stride + 2 + j) * expf(pick(fetch(s * stride), s * stride) - M);
        p.out[static_cast<size_t>(b) * p.d_model + h * hs + j] = oj * inv;
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
        partial_store(mine + 2 + j, o);
    }
    if (tid == 0) {
        partial_store(mine, m);
        partial_store(mine + 1, l);
    }
    __shared__ unsigned ticket;
    if (!last_chunk_arrived(&p.tickets[b * p.kv.heads + h], nchunk, &ticket)) return;
    attn_merge(p, b, h, nchunk, hs);
    if (tid == 0) __hip_atomic_store(&p.tickets[b * p.kv.heads + h], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace gh

namespace gh {

// ---------------------------------------------------------------------------
// Head size 64, throughput form: each wavefront owns a contiguous run of
// positions and walks it 32 positions at a time entirely in registers — 16
// lanes hold one position's 64 floats, four positions per load instruction,
// eight K and eight V loads in flight per lane — keeping a running (max, sum,
// weighted V) that is rescaled when the maximum moves.  The four wavefronts of
// a workgroup, and the workgroups that share a (sequence, head), are merged the
// same way.  This is the kernel for many sequences or long contexts, where the
// cache, not the weights, is most of the bytes of a step.

// Sum over each aligned group of 16 lanes, every lane of the group gets it.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0xB1, 0xF>(v, 0.0f);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xF>(v, 0.0f);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xF>(v, 0.0f);  // row_half_mirror
    v += dpp_move<0x140, 0xF>(v, 0.0f);  // row_mirror
    return v;
}

// PAGE32: pages hold at least 32 positions, so an aligned batch of 32 sits in
// one page and its page number is one scalar lookup.
template <bool PAGE32>
__global__ __launch_bounds__(256) void attn_decode64_kernel(const AttnParams p) {
    constexpr int HS = 64;
    __shared__ float part[4][68];  // per wavefront: m, l, pad, pad, acc[64]
    __shared__ unsigned ticket;
    const int ck = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int ctx = p.st->pos + 1;
    const int nchunk = (ctx + p.chunk - 1) / p.chunk;
    if (ck >= nchunk) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane >> 4, dl = lane & 15;
    const int c0 = ck * p.chunk, c1 = min(ctx, c0 + p.chunk);
    // positions of the chunk are dealt to the wavefronts in runs that are multiples of 32
    const int run = ((((c1 - c0) + 3) / 4) + 31) & ~31;
    const int t0 = c0 + wave * run, t1 = min(c1, t0 + run);
    const float* pool = p.kv.pool;
    const float4 q4 = reinterpret_cast<const float4*>(p.q + static_cast<size_t>(b) * p.d_model + h * HS)[dl];
    const int shift = p.kv.page_shift;
    const int* table = p.kv.page_table + b * p.kv.pages_per_seq;
    const size_t head_stride = static_cast<size_t>(HS) << shift;               // floats per (page, K|V, head)
    const size_t kv_stride = head_stride * p.kv.heads;                         // K -> V within a page
    const size_t page_stride = 2 * kv_stride;
    const size_t layer_base = static_cast<size_t>(p.layer) * p.kv.n_pages * page_stride + h * head_stride;

    float m = -INFINITY, lsum = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    // The page of a batch of 32 positions is looked up one batch ahead, beside the
    // rows of the current batch: a lookup at the top of its own batch is one more
    // trip to memory before that batch's rows can be requested.
    int page = 0;
    if (PAGE32 && t0 < t1) page = table[t0 >> shift];
    for (int tb = t0; tb < t1; tb += 32) {
        float4 k4[8], v4[8];
        size_t base = 0;
        if (PAGE32) base = layer_base + static_cast<size_t>(page) * page_stride;
        if (PAGE32 && tb + 32 < t1) page = table[(tb + 32) >> shift];
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int tt = tb + it * 4 + sub;
            k4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            v4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (tt < t1) {
                size_t off;
                if (PAGE32) {
                    off = base + static_cast<size_t>(tt & ((1 << shift) - 1)) * HS + dl * 4;
                } else {
                    off = layer_base + static_cast<size_t>(table[tt >> shift]) * page_stride
                          + static_cast<size_t>(tt & ((1 << shift) - 1)) * HS + dl * 4;
                }
                k4[it] = *reinterpret_cast<const float4*>(pool + off);
                v4[it] = *reinterpret_cast<const float4*>(pool + off + kv_stride);
            }
        }
        float sc[8];
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int tt = tb + it * 4 + sub;
            const float sdot = row16_sum(dot4(q4, k4[it]));
            sc[it] = tt < t1 ? sdot * p.scale : -INFINITY;
        }
        float mb = sc[0];
#pragma unroll
        for (int it = 1; it < 8; it++) mb = fmaxf(mb, sc[it]);
        // the four position groups of the wavefront share one running maximum
        mb = fmaxf(mb, dpp_move<0x142, 0xA>(mb, mb));
        mb = fmaxf(mb, dpp_move<0x143, 0xC>(mb, mb));
        mb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mb), 63));
        const float mn = fmaxf(m, mb);
        // The 16 lanes of a position group hold the same eight scores and the same
        // running maximum: lane dl forms one exponential, that of score dl (lane 8:
        // of the old maximum, the rescaling factor), and the group shares them by row
        // broadcasts, one exponential per lane and batch instead of nine.
        float arg = sc[0];
#pragma unroll
        for (int it = 1; it < 8; it++) arg = (dl == it) ? sc[it] : arg;
        arg = (dl == 8) ? m : arg;
        const float em = expf(arg - mn);  // exp(-inf) = 0: past the end of the run, first batch
        const float f = row_lane<8>(em);
        lsum *= f;
        acc.x *= f;
        acc.y *= f;
        acc.z *= f;
        acc.w *= f;
        const float e[8] = {row_lane<0>(em), row_lane<1>(em), row_lane<2>(em), row_lane<3>(em),
                            row_lane<4>(em), row_lane<5>(em), row_lane<6>(em), row_lane<7>(em)};
#pragma unroll
        for (int it = 0; it < 8; it++) {
            lsum += e[it];
            acc.x += e[it] * v4[it].x;
            acc.y += e[it] * v4[it].y;
            acc.z += e[it] * v4[it].z;
            acc.w += e[it] * v4[it].w;
        }
        m = mn;
    }
    // fold the four position groups (lanes 16 apart hold the same dims)
    lsum += __shfl_xor(lsum, 16, kWave);
    lsum += __shfl_xor(lsum, 32, kWave);
#pragma unroll
    for (int o = 16; o < 64; o <<= 1) {
        acc.x += __shfl_xor(acc.x, o, kWave);
        acc.y += __shfl_xor(acc.y, o, kWave);
        acc.z += __shfl_xor(acc.z, o, kWave);
        acc.w += __shfl_xor(acc.w, o, kWave);
    }
    if (lane < 16) reinterpret_cast<float4*>(&part[wave][4])[lane] = acc;
    if (lane == 0) {
        part[wave][0] = m;
        part[wave][1] = lsum;
    }
    __syncthreads();
    if (tid >= HS) {
        if (nchunk == 1) return;
    }
    float M = -INFINITY, L = 0.0f, o = 0.0f;
    if (tid < HS) {
        for (int w = 0; w < 4; w++) M = fmaxf(M, part[w][0]);
        for (int w = 0; w < 4; w++) {
            const float f = expf(part[w][0] - M);  // 0 for a wavefront without positions
            L += part[w][1] * f;
            o += part[w][4 + tid] * f;
        }
        if (nchunk == 1) {
            p.out[static_cast<size_t>(b) * p.d_model + h * HS + tid] = o * (1.0f / L);
            return;
        }
        float* mine = p.part + ((static_cast<size_t>(b) * p.kv.heads + h) * p.max_chunks + ck) * (HS + 2);
        partial_store(mine + 2 + tid, o);
        if (tid == 0) {
            partial_store(mine, M);
            partial_store(mine + 1, L);
        }
    }
    if (!last_chunk_arrived(&p.tickets[b * p.kv.heads + h], nchunk, &ticket)) return;
    attn_merge(p, b, h, nchunk, HS);
    if (tid == 0) __hip_atomic_store(&p.tickets[b * p.kv.heads + h], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------
// Prompt pass: causal attention of every new position at once (head size 64).
// It must give what the per-token loop gives (text_gen.cpp:44-46 stepping
// inference.cpp:211-225): query t of a sequence sees the cache up to its own
// position, which the QKV projection of this pass has already written.
//
// One workgroup = 64 queries of one (sequence, head).  Keys and values come
// through LDS in tiles of 64 positions; four threads share a query, each takes
// every fourth key of a tile and keeps its own running softmax, and the four
// are merged with quad permutations at the end.
struct PrefillAttnParams {
    const float* q;  // [batch * len][d_model], rotated
    float* out;      // [batch * len][d_model]
    KvLayout kv;
    int layer, d_model, len, pos_base;
    float scale;
};

// Causal attention of a prompt pass on the fp32 matrix cores (head size 64):
// one workgroup = 64 consecutive queries of one (sequence, head), 16 per
// wavefront; keys and values of the cache (earlier passes included) stream
// through LDS in tiles of 64 positions.  Both products are formed transposed,
//   S^T[key][query] = K . Q^T        O^T[dim][query] += V^T . P^T
// because the accumulator layout of S^T (a lane holds one query and four
// consecutive keys) is exactly the B-operand layout the second product needs:
// the probabilities never leave their registers.  The softmax is the online
// form (running maximum and sum per query, rescaled when the maximum moves);
// inference.cpp:211-225 computes the same numbers one query at a time.
typedef float attn_v4f __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void attn_prefill64_kernel(const PrefillAttnParams p) {
    constexpr int HS = 64, TILE = 64, LDK = HS + 4, LDV = TILE + 4;  // padded rows: float4 reads of 16 rows hit 64 banks
    __shared__ float Ks[TILE * LDK];  // [key][dim]
    __shared__ float Vt[HS * LDV];    // [dim][key]
    const int qb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int t = qb * TILE + wave * 16 + j;  // this lane's query (token index in the pass)
    const bool live = t < p.len;
    const int qpos = p.pos_base + min(t, p.len - 1);
    const int last_pos = p.pos_base + min(p.len, qb * TILE + TILE) - 1;              // last key the workgroup needs
    const int wave_last = p.pos_base + min(p.len, qb * TILE + wave * 16 + 16) - 1;  // ... and this wavefront
    // Q^T as the B operand: lane (query j, group g) holds dims 16 * db + 4g .. + 3, pre-scaled
    float4 qf[4];
    {
        const float* qr = p.q + (static_cast<size_t>(b) * p.len + min(t, p.len - 1)) * p.d_model + h * HS;
#pragma unroll
        for (int db = 0; db < 4; db++) {
            const float4 v = *reinterpret_cast<const float4*>(qr + db * 16 + g * 4);
            qf[db] = make_float4(v.x * p.scale, v.y * p.scale, v.z * p.scale, v.w * p.scale);
        }
    }
    attn_v4f o[4];  // O^T: lane holds query j, dims 16 * db + 4g + r
#pragma unroll
    for (int db = 0; db < 4; db++) o[db] = attn_v4f{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.0f;

    for (int k0 = 0; k0 <= last_pos; k0 += TILE) {
        __syncthreads();
        // stage the tile: K as it is, V transposed; 4 + 4 loads of 16 bytes per thread
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int e = tid + r * 256, row = e >> 4, col = e & 15;
            const int kp = k0 + row;
            float4 kv4 = make_float4(0.f, 0.f, 0.f, 0.f), vv4 = kv4;
            if (kp <= last_pos) {
                kv4 = *reinterpret_cast<const float4*>(p.kv.pool + kv_offset(p.kv, p.layer, b, 0, h, kp) + col * 4);
                vv4 = *reinterpret_cast<const float4*>(p.kv.pool + kv_offset(p.kv, p.layer, b, 1, h, kp) + col * 4);
            }
            *reinterpret_cast<float4*>(&Ks[row * LDK + col * 4]) = kv4;
            Vt[(col * 4 + 0) * LDV + row] = vv4.x;
            Vt[(col * 4 + 1) * LDV + row] = vv4.y;
            Vt[(col * 4 + 2) * LDV + row] = vv4.z;
            Vt[(col * 4 + 3) * LDV + row] = vv4.w;
        }
        __syncthreads();
        if (k0 > wave_last) continue;  // every key of the tile is in the future of this wavefront's queries

        // S^T: four blocks of 16 keys; lane holds query j, keys k0 + 16 kb + 4g + r
        attn_v4f sc[4];
#pragma unroll
        for (int kb = 0; kb < 4; kb++) {
            sc[kb] = attn_v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int db = 0; db < 4; db++) {
                const float4 a = *reinterpret_cast<const float4*>(&Ks[(kb * 16 + j) * LDK + db * 16 + g * 4]);
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, qf[db].x, sc[kb], 0, 0, 0);
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, qf[db].y, sc[kb], 0, 0, 0);
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, qf[db].z, sc[kb], 0, 0, 0);
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, qf[db].w, sc[kb], 0, 0, 0);
            }
        }
        // causal mask (keys up to the query's own position) and the tile's maximum per query
        float mb = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float s = (k0 + kb * 16 + 4 * g + r <= qpos) ? sc[kb][r] : -INFINITY;
                sc[kb][r] = s;
                mb = fmaxf(mb, s);
            }
        mb = fmaxf(mb, __shfl_xor(mb, 16, kWave));  // the four lane groups hold different keys of the same query
        mb = fmaxf(mb, __shfl_xor(mb, 32, kWave));
        const float mn = fmaxf(m, mb);  // finite: key 0 is never in the future
        const float f = expf(m - mn);   // 0 on the first tile
        float psum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float e = expf(sc[kb][r] - mn);  // exp(-inf) = 0 for masked keys
                sc[kb][r] = e;
                psum += e;
            }
        psum += __shfl_xor(psum, 16, kWave);
        psum += __shfl_xor(psum, 32, kWave);
        l = l * f + psum;
#pragma unroll
        for (int db = 0; db < 4; db++) {
            o[db][0] *= f;
            o[db][1] *= f;
            o[db][2] *= f;
            o[db][3] *= f;
        }
        // O^T += V^T . P^T: K-slot g of step r is key 16 kb + 4g + r on both operands
#pragma unroll
        for (int kb = 0; kb < 4; kb++)
#pragma unroll
            for (int db = 0; db < 4; db++) {
                const float4 a = *reinterpret_cast<const float4*>(&Vt[(db * 16 + j) * LDV + kb * 16 + g * 4]);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, sc[kb][0], o[db], 0, 0, 0);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, sc[kb][1], o[db], 0, 0, 0);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, sc[kb][2], o[db], 0, 0, 0);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, sc[kb][3], o[db], 0, 0, 0);
            }
        m = mn;
    }
    if (live) {
        const float inv = 1.0f / l;
        float* orow = p.out + (static_cast<size_t>(b) * p.len + t) * p.d_model + h * HS;
#pragma unroll
        for (int db = 0; db < 4; db++)
            *reinterpret_cast<float4*>(orow + db * 16 + g * 4) =
                make_float4(o[db][0] * inv, o[db][1] * inv, o[db][2] * inv, o[db][3] * inv);
    }
}

// The same attention for longer prompts: one workgroup = 128 consecutive queries of one
// (sequence, head), 32 per wavefront, on the 32 x 32 x 2 form of the fp32 matrix product.
// Against the 64-query kernel above a staged K/V tile serves twice as many queries and an
// operand read from LDS twice as many products, the next tile's rows travel from memory
// into registers while the current tile is multiplied, and the workgroups with the most
// keys in front of them are dealt first.  Both products are again formed transposed:
//   S^T[key][query] = K . Q^T : a lane holds one query (lane % 32) and, of every block of
//   32 keys, keys 8 (r / 4) + 4 (lane / 32) + r % 4 for r = 0..15,
// which is the B-operand layout of O^T[dim][query] += V^T . P^T when K-slot lane / 32 of
// product step e of key group c stands for key 8 c + 4 (lane / 32) + e on both operands.
// The online softmax is inference.cpp:211-225 taken a tile at a time.
// What bounds it: on this part nothing else issues on a SIMD while an fp32 matrix product
// runs (a wavefront's ordinary arithmetic takes as long beside another wavefront's
// v_mfma_f32_32x32x2_f32 chain as the two take one after the other), so the softmax
// arithmetic adds to the 128 products of a tile instead of hiding behind them.  With expf
// it was about 700 vector instructions per wavefront and tile, 430 of them the 33
// exponentials, and 16 x 12 heads x 1536 tokens took 0.86 ms, of which the products alone
// are 0.39; with scores in units of ln 2 and the hardware's 2^x it is 0.78 ms.
typedef float attn_v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_prefill128_kernel(const PrefillAttnParams p) {
    constexpr int HS = 64, TILE = 64, QB = 128, LDK = HS + 4, LDV = TILE + 4;
    __shared__ float Ks[TILE * LDK];  // [key][dim]
    __shared__ float Vt[HS * LDV];    // [dim][key]
    const int qb = static_cast<int>(gridDim.x) - 1 - static_cast<int>(blockIdx.x);  // longest first
    const int h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n32 = lane & 31, h32 = lane >> 5;
    const int t = qb * QB + wave * 32 + n32;  // this lane's query (token index in the pass)
    const bool live = t < p.len;
    const int qpos = p.pos_base + min(t, p.len - 1);
    const int last_pos = p.pos_base + min(p.len, qb * QB + QB) - 1;              // last key the workgroup needs
    const int wave_last = p.pos_base + min(p.len, qb * QB + wave * 32 + 32) - 1;  // ... and this wavefront
    const int wave_first = p.pos_base + min(p.len - 1, qb * QB + wave * 32);  // position of its first query
    // Q^T as the B operand: lane (query, half) holds dims 8 c + 4 half .. + 3 for c = 0..7, pre-scaled.
    // The scale carries log2(e): scores are kept in units of ln 2 and the exponentials below are the
    // hardware's 2^x (one instruction, 1 ulp) instead of expf's thirteen.  What expf's exact argument
    // reduction would add is below what the fp32 dot products in front of it already lose: a score s
    // carries an error of ~|s| 2^-23 from its 64 products, and so does s log2(e) formed this way.
    const float qscale = p.scale * 1.44269504088896341f;
    float4 qf[8];
    {
        const float* qr = p.q + (static_cast<size_t>(b) * p.len + min(t, p.len - 1)) * p.d_model + h * HS;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const float4 v = *reinterpret_cast<const float4*>(qr + c * 8 + h32 * 4);
            qf[c] = make_float4(v.x * qscale, v.y * qscale, v.z * qscale, v.w * qscale);
        }
    }
    attn_v16f o[2];  // O^T: lane holds its query, dims 32 db + 8 (r / 4) + 4 half + r % 4
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    float m = -INFINITY, l = 0.0f;

    // A tile on its way: 4 + 4 loads of 16 bytes per thread, rows tid / 16 + 16 r.  The
    // cache page of a row is looked up a tile before its rows are requested, and the rows a
    // tile before they are multiplied, so neither trip to memory is waited for in the loop;
    // rows past the last key are read as the last key's (every query masks them).
    attn_v4f kreg[4], vreg[4];  // native vectors: a struct copied whole into LDS keeps the array in memory
    int page[4];
    const int* ptab = p.kv.page_table + b * p.kv.pages_per_seq;
    const int shift = p.kv.page_shift, slot_mask = (1 << shift) - 1;
    const int row0 = tid >> 4, col = tid & 15;
    const size_t kv_stride = (static_cast<size_t>(p.kv.heads) << shift) * HS;  // from a page's K rows to its V rows
    const auto lookup = [&](int k0) {
#pragma unroll
        for (int r = 0; r < 4; r++) page[r] = ptab[min(k0 + row0 + 16 * r, last_pos) >> shift];
    };
    const auto fetch = [&](int k0) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int kp = min(k0 + row0 + 16 * r, last_pos);
            const size_t run = ((static_cast<size_t>(p.layer) * p.kv.n_pages + page[r]) * 2) * p.kv.heads + h;
            const float* kr = p.kv.pool + ((run << shift) + (kp & slot_mask)) * HS + col * 4;
            kreg[r] = *reinterpret_cast<const attn_v4f*>(kr);
            vreg[r] = *reinterpret_cast<const attn_v4f*>(kr + kv_stride);
        }
    };
    lookup(0);
    fetch(0);
    lookup(TILE);
    for (int k0 = 0; k0 <= last_pos; k0 += TILE) {
        __syncthreads();  // the tile before has been read by everyone
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = row0 + 16 * r;
            *reinterpret_cast<attn_v4f*>(&Ks[row * LDK + col * 4]) = kreg[r];
            Vt[(col * 4 + 0) * LDV + row] = vreg[r].x;
            Vt[(col * 4 + 1) * LDV + row] = vreg[r].y;
            Vt[(col * 4 + 2) * LDV + row] = vreg[r].z;
            Vt[(col * 4 + 3) * LDV + row] = vreg[r].w;
        }
        __syncthreads();
        fetch(k0 + TILE);  // in flight beside the products below (past the end: the last key again)
        lookup(k0 + 2 * TILE);
        if (k0 > wave_last) continue;  // every key of the tile is in the future of this wavefront's queries
        // S^T: two blocks of 32 keys.  All sixteen operand reads go out before the first
        // product: a read waited for between products leaves the matrix core idle for the
        // LDS latency every time.  (The half of a tile on the diagonal that lies in the future
        // of all of the wavefront's queries is multiplied too and masked: about 2 % of the
        // products, for a loop without branches.)
        attn_v4f ka[2][8];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int c = 0; c < 8; c++)
                ka[kb][c] = *reinterpret_cast<const attn_v4f*>(&Ks[(kb * 32 + n32) * LDK + c * 8 + h32 * 4]);
        __builtin_amdgcn_sched_barrier(0);
        attn_v16f sc[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int r = 0; r < 16; r++) sc[kb][r] = 0.0f;
#pragma unroll
            for (int c = 0; c < 8; c++) {
                sc[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[kb][c][0], qf[c].x, sc[kb], 0, 0, 0);
                sc[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[kb][c][1], qf[c].y, sc[kb], 0, 0, 0);
                sc[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[kb][c][2], qf[c].z, sc[kb], 0, 0, 0);
                sc[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[kb][c][3], qf[c].w, sc[kb], 0, 0, 0);
            }
        }
        // the operands of the second product do not depend on the softmax: requested in front of it
        attn_v4f va[2][2][4];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int db = 0; db < 2; db++)
#pragma unroll
                for (int c = 0; c < 4; c++)
                    va[kb][db][c] =
                        *reinterpret_cast<const attn_v4f*>(&Vt[(db * 32 + n32) * LDV + kb * 32 + c * 8 + h32 * 4]);
        __builtin_amdgcn_sched_barrier(0);
        // causal mask (keys up to the query's own position) and the tile's maximum per query
        float mb = -INFINITY;
        if (k0 + TILE - 1 > wave_first) {  // only the tiles on the diagonal need the comparisons
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = k0 + kb * 32 + 8 * (r >> 2) + 4 * h32 + (r & 3);
                    sc[kb][r] = (key <= qpos) ? sc[kb][r] : -INFINITY;
                }
        }
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) mb = fmaxf(mb, sc[kb][r]);
        mb = fmaxf(mb, __shfl_xor(mb, 32, kWave));  // the two halves hold different keys of the same query
        const float mn = fmaxf(m, mb);  // finite: key 0 is never in the future
        const float f = __builtin_amdgcn_exp2f(m - mn);  // 0 on the first tile
        float psum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float e = __builtin_amdgcn_exp2f(sc[kb][r] - mn);  // 2^(-inf) = 0 for masked keys
                sc[kb][r] = e;
                psum += e;
            }
        psum += __shfl_xor(psum, 32, kWave);
        l = l * f + psum;
#pragma unroll
        for (int db = 0; db < 2; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= f;
        // O^T += V^T . P^T
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int db = 0; db < 2; db++)
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[kb][db][c][0], sc[kb][4 * c + 0], o[db], 0, 0, 0);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[kb][db][c][1], sc[kb][4 * c + 1], o[db], 0, 0, 0);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[kb][db][c][2], sc[kb][4 * c + 2], o[db], 0, 0, 0);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[kb][db][c][3], sc[kb][4 * c + 3], o[db], 0, 0, 0);
                }
        m = mn;
    }
    if (live) {
        const float inv = 1.0f / l;
        float* orow = p.out + (static_cast<size_t>(b) * p.len + t) * p.d_model + h * HS;
#pragma unroll
        for (int db = 0; db < 2; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++)
                *reinterpret_cast<float4*>(orow + db * 32 + q4 * 8 + h32 * 4) =
                    make_float4(o[db][4 * q4 + 0] * inv, o[db][4 * q4 + 1] * inv, o[db][4 * q4 + 2] * inv,
                                o[db][4 * q4 + 3] * inv);
    }
}

}  // namespace gh

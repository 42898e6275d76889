// Persistent batch-1 decoder sharded over the chip's eight XCDs, with the weights
// streamed through LDS.
//
// One launch runs a whole run of steps with one workgroup per compute unit,
// like persist_decode_kernel.  Two things are different.
//
// 1. A layer is split over the XCDs (32 compute units behind one L2) the way
//    tensor parallelism splits it over devices.  XCD g owns one or two attention
//    heads and a contiguous range of FFN hidden units:
//
//      P1  norm1 + Q/K/V rows of the XCD's heads          -> q, k, v cells        (inside the XCD)
//      P2  attention, a head's context cut into slices,
//          one workgroup per slice                         -> (m, l, acc) cells    (inside the XCD)
//      P3  merge + W_o over the columns of the XCD's heads -> partial sums, d rows (across XCDs)
//      P4  rows [r d/32, (r+1) d/32): sum of the eight
//          partials in XCD order + residual                -> x' cells             (inside the XCD)
//      P5  norm2 + gate/up rows of the XCD's hidden units  -> hidden cells         (inside the XCD)
//      P6  W_down over the columns of the XCD's units      -> partial sums         (across XCDs)
//      P7  as P4                                           -> x cells              (inside the XCD)
//
//    so a layer crosses XCDs twice (a workgroup polls d/32 x 8 cells there) and
//    hands data over inside an XCD five times.  A hand-off inside an XCD goes
//    through its L2: ordinary stores, and loads with the non-temporal bit, which
//    the L2 serves and the compute unit's vector cache never keeps.  The memory
//    behind those cells is written by that one XCD only.  The eight partial sums
//    of a row are added in XCD order, so results do not depend on timing.
//
// 2. No wavefront that waits for activations ever requests weights.  Every
//    workgroup's share of the weights lies in one contiguous stream in the exact
//    order it is used (built once per model: QKV rows, W_o block, gate/up rows,
//    W_down block per layer, then its rows of the tied logits matrix; the norm
//    gains are folded into the rows that follow the norm).  Four "streamer"
//    wavefronts copy that stream into a ring in LDS, running ahead of the
//    arithmetic by up to the ring's size (through the pick and across token
//    boundaries as well), and eight "compute" wavefronts read their rows from
//    the ring.  A wavefront's vector loads return in order, so a poll issued
//    behind a bulk load would wait for it; here polls and bulk loads come from
//    different wavefronts, and the weight stream never stops for a hand-off.
//
// The arithmetic per phase is that of src/transformer/inference.cpp:150-258
// (Modern block: RMSNorm, biased Q/K/V/O projections, RoPE on pairs (2j, 2j+1),
// bias-free SwiGLU).
#pragma once

#include "kernels_persist.h"

namespace gh {

constexpr int kXcdThreads = 768;
constexpr int kXcdComputeWaves = 8;   // wavefronts 0..7
constexpr int kXcdStreamWaves = 4;    // wavefronts 8..11
constexpr int kXcdTeamWaves = 7;      // wavefronts 0..6 gather cells and meet at the LDS barrier
constexpr int kXcdTeamLanes = kXcdTeamWaves * 64;
constexpr int kXcdRowWaves = 6;       // wavefronts 0..5 own the rows of the W_o and W_down blocks
constexpr int kXcdRelayWave = 6;      // sums the partials of this workgroup's rows (P4, P7)
constexpr int kXcdAttnWave = 7;       // attention of one slice (P2); takes no part in anything else
constexpr int kXcds = 8, kWgPerXcd = 32;
constexpr int kXcdUnit = 1024;        // bytes one streamer instruction moves
constexpr int kXcdDepth = 12;         // loads a streamer keeps in flight
constexpr int kAuxNonTemporal = 2;    // nt on gfx94x / gfx950 buffer instructions
constexpr int kApCells = 66;          // cells of one attention partial: acc[64], m, l
constexpr int kXcdMaxUnitsPerWg = 2 * kXcdTeamWaves;

// What XCD g owns.
struct XcdShard {
    int nh;       // heads: 1 or 2
    int head[2];
    int u0, nu;   // hidden units [u0, u0 + nu), nu a multiple of 4
};

// The shape and the split, the same for every workgroup of a launch.
struct XcdGeom {
    int D, F, V, L, H;
    XcdShard shard[kXcds];
    unsigned stride_units;  // 1 KB units between the streams of two workgroups
};

// Where workgroup (XCD g, rank r) finds its things.  Byte offsets are relative to
// the start of a layer's section of the stream.
struct XcdWg {
    int nh, KC, ppw;       // heads, columns of the W_o block, pairs of QKV rows
    int ub, nu;            // hidden units [ub, ub + nu) of the model
    int u0, UG;            // the XCD's units
    // A layer of the stream: ppw blocks of {row 2j, row 2j + 1, their two biases, 8 bytes
    // of padding}; the W_o block [d/32][KC] and the d/32 entries of b_o; 2 nu gate / up
    // rows; the W_down block [d/32][UG].
    unsigned pair_bytes, o_wo, o_bo, o_gu, o_dn, layer_bytes;
    unsigned layers_units;  // units of all layers, rounded up to a multiple of four
    int v0, nrows;          // rows of the logits matrix
    unsigned logits_units;
};

__host__ __device__ inline XcdWg xcd_wg(const XcdGeom& gm, int g, int r) {
    const XcdShard& sh = gm.shard[g];
    XcdWg w;
    const unsigned D = static_cast<unsigned>(gm.D), RW = D / kWgPerXcd;
    w.nh = sh.nh;
    w.KC = 64 * sh.nh;
    w.ppw = 3 * sh.nh;
    w.u0 = sh.u0;
    w.UG = sh.nu;
    w.ub = sh.u0 + (r * sh.nu) / kWgPerXcd;
    w.nu = sh.u0 + ((r + 1) * sh.nu) / kWgPerXcd - w.ub;
    w.pair_bytes = 2u * D * 4u + 16u;
    w.o_wo = static_cast<unsigned>(w.ppw) * w.pair_bytes;
    w.o_bo = w.o_wo + RW * static_cast<unsigned>(w.KC) * 4u;
    w.o_gu = w.o_bo + RW * 4u;
    w.o_dn = w.o_gu + static_cast<unsigned>(w.nu) * 2u * D * 4u;
    w.layer_bytes = w.o_dn + RW * static_cast<unsigned>(w.UG) * 4u;
    w.layers_units = (static_cast<unsigned>(gm.L) * w.layer_bytes + 4095u) / 4096u * 4u;
    const int id = g * kWgPerXcd + r;
    w.v0 = static_cast<int>(static_cast<long long>(gm.V) * id / (kXcds * kWgPerXcd));
    w.nrows = static_cast<int>(static_cast<long long>(gm.V) * (id + 1) / (kXcds * kWgPerXcd)) - w.v0;
    w.logits_units = (static_cast<unsigned>(w.nrows) * D * 4u + 4095u) / 4096u * 4u;
    return w;
}

// Exchange cells of a session, in cells from one base.
struct XcdCells {
    unsigned qkv;   // [8][2 heads][3][64]                 inside an XCD
    unsigned ap;    // [8][32 slices][kApCells]            inside an XCD
    unsigned part;  // [2][8 source XCDs][D]               across XCDs
    unsigned xr;    // [2][8][D]                           inside an XCD
    unsigned hid;   // [8][hid_stride]                     inside an XCD
    unsigned tok;   // [1]                                 across XCDs
    unsigned hid_stride;
    unsigned total;
};

__host__ __device__ inline XcdCells xcd_cells(const XcdGeom& gm) {
    XcdCells c;
    unsigned at = 0;
    c.qkv = at, at += kXcds * 2 * 192;
    c.ap = at, at += kXcds * ((kWgPerXcd * kApCells + 15) / 16 * 16);
    c.part = at, at += 2u * kXcds * static_cast<unsigned>(gm.D);
    c.xr = at, at += 2u * kXcds * static_cast<unsigned>(gm.D);
    unsigned most = 0;
    for (int g = 0; g < kXcds; g++) most = most > static_cast<unsigned>(gm.shard[g].nu) ? most : static_cast<unsigned>(gm.shard[g].nu);
    c.hid_stride = (most + 15u) / 16u * 16u;
    c.hid = at, at += kXcds * c.hid_stride;
    c.tok = at, at += 16;
    c.total = at;
    return c;
}
constexpr unsigned kApStrideCells = (kWgPerXcd * kApCells + 15) / 16 * 16;  // cells of one XCD's partials

struct XcdParams {
    PersistParams b;          // model vectors, cache, logits, control block, history, pick, feed
    XcdGeom gm;
    const char* stream;       // workgroup (g, r)'s stream starts at (g * 32 + r) * stride_units KB
    Cell* xc;                 // exchange cells, laid out as xcd_cells() says
    unsigned ring_units;      // ring size of workgroups 1.. in 1 KB units (a power of two)
    unsigned ring_units_wg0;  // ... of workgroup 0, which also needs room for the pick
    unsigned launch_base;     // value of the per-XCD arrival counters when this launch starts
    int attn_slices;          // slices per head (8), or 0: every workgroup of the XCD takes one (32 / heads of the XCD)
};

// LDS control words of a workgroup.
enum {
    kXFilled = 0,     // [4] units written so far by streamer wavefront i
    kXConsumed = 4,   // [8] compute wavefront i reads nothing below this unit
    kXBar = 12,       // arrivals at the team's barrier
    kXDone = 13,      // the compute wavefronts have finished (or given up): streamers leave
    kXAbandon = 14,   // a wait was abandoned
    kXXcd = 15,
    kXRank = 16,
    kXWords = 32
};

__device__ __forceinline__ unsigned xcc_id() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xfu;
}

typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void lds_settle() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// Two wavefront sums side by side: the two chains fill each other's wait states.
__device__ __forceinline__ void wave_sum2(float& a, float& b) {
    a += dpp_move<0xB1, 0xF>(a, 0.0f);
    b += dpp_move<0xB1, 0xF>(b, 0.0f);
    a += dpp_move<0x4E, 0xF>(a, 0.0f);
    b += dpp_move<0x4E, 0xF>(b, 0.0f);
    a += dpp_move<0x141, 0xF>(a, 0.0f);
    b += dpp_move<0x141, 0xF>(b, 0.0f);
    a += dpp_move<0x140, 0xF>(a, 0.0f);
    b += dpp_move<0x140, 0xF>(b, 0.0f);
    a += dpp_move<0x142, 0xA>(a, 0.0f);
    b += dpp_move<0x142, 0xA>(b, 0.0f);
    a += dpp_move<0x143, 0xC>(a, 0.0f);
    b += dpp_move<0x143, 0xC>(b, 0.0f);
    a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(a), 63));
    b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(b), 63));
}

// A cell written for readers inside the XCD.  Also a device-scope (write-through)
// store: an ordinary store may sit in the compute unit's write path for
// microseconds while the memory system is busy (a two-workgroup ping-pong under a
// streaming load: 0.25 us per hand-off with write-through stores, 8 us with
// ordinary ones), and every workgroup of the XCD is waiting for this one.
#ifndef GH_XCD_BAR_SLEEP
#define GH_XCD_BAR_SLEEP 1
#endif
__device__ __forceinline__ void cell_put_local(Cell* c, float v, unsigned tag) {
    v2i w;
    w.x = __float_as_int(v);
    w.y = static_cast<int>(tag);
    *reinterpret_cast<v2i*>(c) = w;
}

// LDS control words: the address space is spelled out, because a pointer that
// travels through a struct is otherwise "generic" to the compiler and its
// accesses become flat loads, which wait on the vector-memory counter as well.
typedef volatile __attribute__((address_space(3))) unsigned* XcdCtl;

// The state every wait of the kernel shares.
struct XcdWait {
    XcdCtl ctl;  // LDS control words
    PersistCtl* gctl;
    unsigned spin_limit;
};

// A wait was abandoned: tell the workgroup, the grid and the host.
__device__ __forceinline__ void xcd_give_up(const XcdWait& w, unsigned where) {
    w.ctl[kXAbandon] = 1u;
    __hip_atomic_store(&w.gctl->where, where, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&w.gctl->abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Lanes [0, kXcdTeamLanes) wait until cells [0, n) of src carry `tag` and copy the
// values to dst (LDS).  Each lane polls only its own cells.  AUX: device scope for
// cells other XCDs wrote, non-temporal for cells of this XCD.  False: abandoned.
template <int AUX>
__device__ __forceinline__ bool xcd_gather(const Cell* src, int n, unsigned tag, float* dst, int ctid,
                                           const XcdWait& w, unsigned* rounds = nullptr, unsigned* first_trip = nullptr) {
    const __amdgpu_buffer_rsrc_t rs = make_buffer(src, static_cast<unsigned>(n) * 8u);
    const int itag = static_cast<int>(tag);
    unsigned spins = 0;
    if (first_trip) {
        // diagnostics: one poll, timed from issue to return
        const unsigned t0 = static_cast<unsigned>(__builtin_amdgcn_s_memtime());
        const v4i c = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<unsigned>(2 * ctid < n ? 2 * ctid : 0) * 8u, 0, AUX);
        asm volatile("s_waitcnt vmcnt(0)" ::"v"(c) : "memory");
        *first_trip += static_cast<unsigned>(__builtin_amdgcn_s_memtime()) - t0;
    }
#pragma nounroll
    for (;;) {
        bool ok = true;
        for (int i = 2 * ctid; i < n; i += 2 * kXcdTeamLanes) {
            const v4i c = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<unsigned>(i) * 8u, 0, AUX);
            ok = ok && c.y == itag && (i + 1 >= n || c.w == itag);
            dst[i] = __int_as_float(c.x);
            if (i + 1 < n) dst[i + 1] = __int_as_float(c.z);
        }
        if (ok) {
            if (rounds) *rounds += spins;
            return true;
        }
        ++spins;
        if (spins > w.spin_limit || w.ctl[kXAbandon] != 0u
            || ((spins & 63u) == 0u
                && __hip_atomic_load(&w.gctl->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
            xcd_give_up(w, tag);
            return false;
        }
    }
}

// The team's barrier: LDS writes made before it by any of the seven wavefronts are
// visible to all of them after it.  (The hardware barrier would include the
// streamers, which must never wait for anybody.)  gen counts this wavefront's
// barriers.  False: abandoned.
__device__ __forceinline__ bool xcd_team_sync(const XcdWait& w, unsigned& gen, int lane, unsigned* rounds = nullptr) {
    gen += kXcdTeamWaves;
    lds_settle();
    if (lane == 0)
        __hip_atomic_fetch_add((__attribute__((address_space(3))) unsigned*)(&w.ctl[kXBar]), 1u, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    unsigned spins = 0;
    // A waiting wavefront sleeps between looks: seven wavefronts reading the counter
    // as fast as they can take the LDS and the issue slots from the ones that work
    // (the attention wavefront ran four times slower beside such a loop).
#pragma nounroll
    while (static_cast<int>(w.ctl[kXBar] - gen) < 0) {
        ++spins;
        if ((spins & 15u) == 0u) {
            if (w.ctl[kXAbandon] != 0u) return false;
            if (spins > (1u << 22)) {
                xcd_give_up(w, 0xFFFFFFF0u);
                return false;
            }
        }
        __builtin_amdgcn_s_sleep(GH_XCD_BAR_SLEEP);
    }
    asm volatile("" ::: "memory");
    if (rounds) *rounds += spins;
    return true;
}

// Waits until the streamers have written every unit below `units` (counted from the
// start of the launch) into the ring.
__device__ __forceinline__ bool xcd_wait_filled(const XcdWait& w, unsigned units, unsigned* stalled = nullptr) {
    unsigned spins = 0;
#pragma nounroll
    for (;;) {
        bool ok = true;
#pragma unroll
        for (int i = 0; i < kXcdStreamWaves; i++) {
            // streamer i owns units i, i + 4, ...: it must have written (units + 3 - i) / 4 of them
            const unsigned need = (units + 3u - static_cast<unsigned>(i)) >> 2;
            ok = ok && static_cast<int>(w.ctl[kXFilled + i] - need) >= 0;
        }
        if (ok) {
            asm volatile("" ::: "memory");  // ring reads stay behind the wait
            if (stalled) *stalled += spins;
            return true;
        }
        if (w.ctl[kXAbandon] != 0u) return false;
        if (++spins > (1u << 22)) {
            xcd_give_up(w, 0xFFFFFFF1u);
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

// "This wavefront reads nothing below `unit` any more."  The compiler may not move
// ring reads across it (LDS executes a wavefront's operations in order).
__device__ __forceinline__ void xcd_set_consumed(const XcdWait& w, int wave, int lane, unsigned unit) {
    asm volatile("" ::: "memory");
    if (lane == 0) w.ctl[kXConsumed + wave] = unit;
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ float4 ring_ld4(const char* ring, unsigned mask, unsigned off) {
    return *reinterpret_cast<const float4*>(ring + (off & mask));
}

// Does step s of a launch compute logits?
__device__ __forceinline__ bool xcd_wants_logits(const PersistParams& p, int s) {
    return (s >= p.n_prompt - 1) || p.logit_log != nullptr || s == p.n_steps - 1;
}

// One streamer wavefront: copies units sw, sw + 4, ... of steps [s0, s1) into the
// ring, kXcdDepth loads in flight, never writing a unit before every compute
// wavefront is past the unit it overwrites.  unit_base: units of the launch before
// step s0 (updated); count: units this wavefront has written (updated).
//
// Steps without logits (all but the last of a prompt run) come first in a launch
// and are shorter; both kinds start at the beginning of the workgroup's stream.
// The loop is straight-line code over compile-time register indices: a data-
// dependent exit from it would turn the registers in flight into an array in
// scratch memory, with a wait behind every load.
struct XcdCursor {
    unsigned j;      // this wavefront's unit number inside the step (unit 4 j + sw of the step)
    unsigned per;    // units of this wavefront in the current step
    unsigned shorts; // steps without logits still to come, the current one included
    unsigned gbase;  // units of the launch before the current step
};

__device__ __forceinline__ void xcd_cursor_next(XcdCursor& c, unsigned per_short, unsigned per_full) {
    c.j++;
    const bool wrap = c.j == c.per;
    c.gbase += wrap ? 4u * c.per : 0u;
    c.j = wrap ? 0u : c.j;
    const unsigned left = (wrap && c.shorts > 0u) ? c.shorts - 1u : c.shorts;
    c.per = (wrap && left == 0u) ? per_full : c.per;
    c.shorts = left;
}

__device__ inline void xcd_stream(const XcdParams& p, const XcdWg& me, const char* src, char* ring,
                                  unsigned ring_units, const XcdWait& w, int sw, int lane, int s0, int s1,
                                  unsigned& unit_base, unsigned& count) {
    if (s0 >= s1) return;
    const unsigned mask = ring_units * kXcdUnit - 1u;
    const unsigned per_short = me.layers_units / kXcdStreamWaves;
    const unsigned per_full = (me.layers_units + me.logits_units) / kXcdStreamWaves;
    // steps [0, n_short) of the launch go without logits
    const int n_short = p.b.logit_log ? 0 : max(0, min(p.b.n_prompt - 1, p.b.n_steps - 1));
    const unsigned shorts = static_cast<unsigned>(max(0, min(s1, n_short) - s0));
    const unsigned fulls = static_cast<unsigned>(s1 - s0) - shorts;
    unsigned total = shorts * per_short + fulls * per_full;  // units of this wavefront
    XcdCursor ci{0u, shorts > 0u ? per_short : per_full, shorts, unit_base};
    XcdCursor cw = ci;
    unsigned issued = 0;
    unsigned space_end = 0;  // units below this may be written
    const char* lane_src = src + lane * 16 + sw * kXcdUnit;
    auto issue = [&](v4f& dst) {
        // past the end: a harmless reload of the first unit, so that no load sits under a branch
        const unsigned at = issued < total ? ci.j : 0u;
        dst = *reinterpret_cast<const v4f*>(lane_src + static_cast<size_t>(at) * (kXcdStreamWaves * kXcdUnit));
        asm volatile("" ::: "memory");  // loads go out in this order: the oldest is the one written next
        issued++;
        xcd_cursor_next(ci, per_short, per_full);
    };
    v4f buf[kXcdDepth];
#pragma unroll
    for (int i = 0; i < kXcdDepth; i++) issue(buf[i]);
    for (unsigned k0 = 0; k0 < total; k0 += kXcdDepth) {
#pragma unroll
        for (int i = 0; i < kXcdDepth; i++) {
            if (k0 + i < total) {
                const unsigned unit = cw.gbase + 4u * cw.j + static_cast<unsigned>(sw);
                if (static_cast<int>(unit - space_end) >= 0) {
                    unsigned spins = 0;
#pragma nounroll
                    for (;;) {
                        unsigned low = w.ctl[kXConsumed];
#pragma unroll
                        for (int q = 1; q < kXcdComputeWaves; q++) {
                            const unsigned c = w.ctl[kXConsumed + q];
                            low = c < low ? c : low;
                        }
                        space_end = low + ring_units;
                        if (static_cast<int>(unit - space_end) < 0) break;
                        if (w.ctl[kXDone] != 0u || w.ctl[kXAbandon] != 0u) {
                            total = 0;  // leave: nothing more is written
                            break;
                        }
                        if (++spins > (1u << 22)) {
                            xcd_give_up(w, 0xFFFFFFF2u);
                            total = 0;
                            break;
                        }
                        __builtin_amdgcn_s_sleep(2);
                    }
                }
                if (total != 0u) {
                    *reinterpret_cast<v4f*>(ring + ((unit * kXcdUnit + lane * 16) & mask)) = buf[i];
                    count++;
                    asm volatile("" ::: "memory");  // the unit, then its count: LDS keeps a wavefront's order
                    if (lane == 0) w.ctl[kXFilled + sw] = count;
                    xcd_cursor_next(cw, per_short, per_full);
                }
            }
            issue(buf[i]);
#ifdef GH_XCD_PACE
            __builtin_amdgcn_s_sleep(GH_XCD_PACE);
#endif
        }
    }
    // what is still in flight lands in registers only; let it arrive before leaving
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unit_base = cw.gbase;
}

// KD = d_model / 256; head size 64.  FEED: the streaming variant.
template <int KD, bool ROW_LDS, bool FEED>
__global__ __launch_bounds__(kXcdThreads) void xcd_decode_kernel(const XcdParams p) {
    extern __shared__ __attribute__((aligned(128))) float lds[];
    __shared__ unsigned ctl_words[kXWords];
    constexpr int D = KD * 256, HS = 64, RW = D / kWgPerXcd;
    static_assert(RW % 4 == 0, "rows of a block are dealt four to a wavefront");
    const PersistParams& pb = p.b;
    int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int wg = blockIdx.x, G = gridDim.x;
    const int L = pb.L, V = pb.V;
    XcdCtl ctl = (XcdCtl)ctl_words;
    XcdWait wt{ctl, pb.ctl, pb.spin_limit};

    // ---- which XCD is this, and which of its 32 workgroups
    if (tid == 0) {
        const unsigned g0 = xcc_id();
        unsigned r0 = 0xFFFFu;
        if (g0 < kXcds)
            r0 = __hip_atomic_fetch_add(&pb.ctl->xcd_count[g0 * 32], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                 - p.launch_base;
        for (int i = 0; i < kXWords; i++) ctl_words[i] = 0u;
        ctl_words[kXConsumed + kXcdAttnWave] = 0x7FFFFFFFu;  // reads no weights
        ctl_words[kXXcd] = g0;
        ctl_words[kXRank] = r0;
        g_wait_abandoned = 0u;
    }
    const unsigned ring_units = wg == 0 ? p.ring_units_wg0 : p.ring_units;
    char* ring = reinterpret_cast<char*>(lds);
    const unsigned ring_mask = ring_units * kXcdUnit - 1u;
    float* wa = lds + ring_units * (kXcdUnit / 4);  // work area behind the ring
    float* xs = wa;                                  // [D] input of the layer
    float* xs1 = xs + D;                             // [D] after the attention half
    float* apbuf = xs1 + D;                          // [32 * kApCells] the XCD's attention partials
    float* hbuf = apbuf + kWgPerXcd * kApCells;      // [<= 512] the XCD's hidden units
    float* att = hbuf + 512;                         // [row wavefronts][128 + 32] merged attention output, merge factors
    float* qkv7 = att + kXcdRowWaves * (128 + 32);   // [192] q, new key, new value (attention wavefront)
    int* ptab = reinterpret_cast<int*>(qkv7 + 192);  // [pages_per_seq]
    for (int i = tid; i < pb.kv.pages_per_seq; i += kXcdThreads) ptab[i] = pb.kv.page_table[i];
    __syncthreads();
    const int g = static_cast<int>(ctl_words[kXXcd]), r = static_cast<int>(ctl_words[kXRank]);
    if (g >= kXcds || r < 0 || r >= kWgPerXcd) {
        // not 32 workgroups on every XCD: this kernel's split does not apply
        if (tid == 0) {
            __hip_atomic_store(&pb.ctl->where, 0xFFFFFFFDu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&pb.ctl->abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }
    const XcdWg me = xcd_wg(p.gm, g, r);
    const XcdCells cl = xcd_cells(p.gm);
    const int wgid = g * kWgPerXcd + r;
    const char* my_stream = p.stream + static_cast<size_t>(wgid) * p.gm.stride_units * kXcdUnit;
    Cell* tok_cell = p.xc + cl.tok;

    auto kv_at = [&](int layer, int which, int head, int t) -> size_t {
        const int page = ptab[t >> pb.kv.page_shift];
        const int slot = t & ((1 << pb.kv.page_shift) - 1);
        const size_t run = ((static_cast<size_t>(layer) * pb.kv.n_pages + page) * 2 + which) * pb.H + head;
        return ((run << pb.kv.page_shift) + slot) * HS;
    };

    const bool streamer = wave >= kXcdComputeWaves;
    const int sw = wave - kXcdComputeWaves;
    // the wavefronts every workgroup of the XCD waits for go first when two are ready
    if (wave == kXcdAttnWave || wave == kXcdRelayWave) __builtin_amdgcn_s_setprio(3);
    else if (!streamer) __builtin_amdgcn_s_setprio(1);
    unsigned s_unit_base = 0, s_count = 0;  // streamer state
    unsigned unit_base = 0;                 // compute wavefronts: units of the launch before this step
    unsigned bar_gen = 0;
    int i_pick = 0;
    unsigned arrive_gen = pb.arrive_base;
    bool ended = false;
    // Diagnostics, compiled in with -DGH_XCD_TICKS only (the counters cost registers the
    // kernel does not have to spare): polls that found the ring not yet filled and poll
    // rounds of the gathers, per phase, and the core clock spent in every phase by
    // wavefront 0, the relay wavefront and the attention wavefront of workgroup 0.
#ifdef GH_XCD_TICKS
    unsigned stall[13] = {};
#define XSTALL(k) (&stall[k])
    unsigned dur[16] = {};
    unsigned last_tick = 0;
#define XTICK(k)                                                                  \
    do {                                                                          \
        const unsigned now_ = static_cast<unsigned>(__builtin_amdgcn_s_memtime()); \
        dur[k] += now_ - last_tick;                                               \
        last_tick = now_;                                                         \
    } while (0)
#define XTRIP(k) (&dur[k])
#define XROUNDS(k, n) dur[k] += (n)
#else
#define XSTALL(k) nullptr
#define XROUNDS(k, n) do { } while (0)
#define XTICK(k) do { } while (0)
#define XTRIP(k) nullptr
#endif
    int n_stamp = 0;
    auto stamp = [&]() {
        if (pb.prof && wg == 0 && tid == 0 && n_stamp < pb.prof_cap / 2) pb.prof[n_stamp] = __builtin_amdgcn_s_memrealtime();
        n_stamp++;
    };
    stamp();

    // Streamers of workgroups 1..: the whole launch in one go.  (Workgroup 0's take
    // part in the pick, whose barriers are the hardware's, and stream step by step.)
    if (streamer && wg != 0) {
        xcd_stream(p, me, my_stream, ring, ring_units, wt, sw, lane, 0, pb.n_steps, s_unit_base, s_count);
        return;
    }

    // attention slices
    const int SL = p.attn_slices > 0 ? p.attn_slices : kWgPerXcd / me.nh;
    const bool attn_wg = r < SL * me.nh;
    const int a_hi = r / SL, a_slice = r - a_hi * SL;
    const int a_head = p.gm.shard[g].head[a_hi < 2 ? a_hi : 0];

    for (int s = 0;; s++) {
        // ===== pick before step s (text_gen.cpp:48-61)
        if ((!FEED || !ended) && i_pick < pb.n_picks && s >= pb.n_prompt && (s > 0 || pb.start_with_pick)) {
            const unsigned tt = ((pb.epoch + static_cast<unsigned>(s)) * static_cast<unsigned>(L + 1)
                                 + static_cast<unsigned>(L)) * 8u + (s == 0 ? 6u : 7u);
            int chosen = 0;
            if (!persist_pick<ROW_LDS, FEED, kXcdThreads>(pb, wa, i_pick, arrive_gen, tt, s > 0, G, tok_cell, &chosen)) {
                if (tid == 0) ctl[kXDone] = 1u;
                return;
            }
            i_pick++;
            if (wg == 0) {
                // the pick used the work area; restore the page table
                __syncthreads();
                for (int i = tid; i < pb.kv.pages_per_seq; i += kXcdThreads) ptab[i] = pb.kv.page_table[i];
                __syncthreads();
                if (FEED && streamer) ended = chosen == pb.stop_token;
            }
        }
        stamp();
        if (s >= pb.n_steps) break;
        if (streamer) {
            // workgroup 0: this step's units; the step after a pick of the stop token is the last
            xcd_stream(p, me, my_stream, ring, ring_units, wt, sw, lane, s, s + 1, s_unit_base, s_count);
            if (ctl[kXAbandon] != 0u || ctl[kXDone] != 0u) return;
            if (FEED && ended) break;
            continue;
        }
        if (FEED && ended) break;
        const int pos = pb.pos0 + s;
        const unsigned sb = (pb.epoch + 1u + static_cast<unsigned>(s)) * static_cast<unsigned>(L + 1);
        auto tag_of = [&](int layer, int ph) {
            return (sb + static_cast<unsigned>(layer)) * 8u + static_cast<unsigned>(ph) + 1u;
        };
        const bool want_logits = xcd_wants_logits(pb, s);

        // ---- token (inference.cpp:159-182): every wavefront reads it for itself
        int tok;
        if (s < pb.n_prompt) {
            if (s == 0 && pb.tok0 >= 0) {
                tok = pb.tok0;  // handed over in the launch's arguments
                if (wg == 0 && tid == 0)
                    __hip_atomic_store(&pb.hist[pos], tok, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                tok = pb.hist[pos];
            }
        } else {
            const unsigned tt = ((pb.epoch + static_cast<unsigned>(s)) * static_cast<unsigned>(L + 1)
                                 + static_cast<unsigned>(L)) * 8u + (s == 0 ? 6u : 7u);
            unsigned spins = 0;
            float tv = 0.0f;
#pragma nounroll
            while (!cell_get(tok_cell, tt, tv)) {
                if (++spins > pb.spin_limit || ctl[kXAbandon] != 0u
                    || ((spins & 63u) == 0u
                        && __hip_atomic_load(&pb.ctl->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
                    xcd_give_up(wt, tt);
                    return;
                }
            }
            tok = __builtin_amdgcn_readfirstlane(__float_as_int(tv));
            if constexpr (FEED) {
                if (tok < 0) {  // the host asked for the run to end here
                    ctl[kXDone] = 1u;
                    return;
                }
                ended = tok == pb.stop_token;  // this step is the last one
            }
        }

#ifdef GH_XCD_TICKS
        last_tick = static_cast<unsigned>(__builtin_amdgcn_s_memtime());
#endif
        if (wave == kXcdAttnWave) {
            // ================= attention wavefront: P2 of every layer
            if (attn_wg) {
                const int ctx = pos + 1;
                const int chunk = (((ctx + SL - 1) / SL) + 3) & ~3;
                const int t0 = a_slice * chunk;
                const int t1 = min(t0 + chunk, ctx);  // may be <= t0: an empty slice
                const bool has_cur = pos >= t0 && pos < t0 + chunk;
                const int sub = lane >> 4, dl = lane & 15;
                const float* pool = pb.kv.pool;
                float4 k4[8], v4[8];
                auto fetch = [&](int layer, int batch) {
#pragma unroll
                    for (int it = 0; it < 8; it++) {
                        const int tt = t0 + batch * 32 + it * 4 + sub;
                        k4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
                        v4[it] = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (tt < t1 && tt < pos) {
                            k4[it] = *reinterpret_cast<const float4*>(pool + kv_at(layer, 0, a_head, tt) + dl * 4);
                            v4[it] = *reinterpret_cast<const float4*>(pool + kv_at(layer, 1, a_head, tt) + dl * 4);
                        }
                    }
                };
                fetch(0, 0);
                for (int l = 0; l < L; l++) {
                    XTICK(5);
                    // q (and the new key and value, if this slice holds the current position)
                    {
                        const unsigned t = tag_of(l, 0);
                        const Cell* src = p.xc + cl.qkv + (g * 2 + a_hi) * 192;
                        const int ncell = has_cur ? 192 : 64;
                        const __amdgpu_buffer_rsrc_t rs = make_buffer(src, static_cast<unsigned>(ncell) * 8u);
                        unsigned spins = 0;
#pragma nounroll
                        for (;;) {
                            bool ok = true;
                            for (int i = 2 * lane; i < ncell; i += 128) {
                                const v4i c = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<unsigned>(i) * 8u, 0,
                                                                                     kAuxNonTemporal);
                                ok = ok && c.y == static_cast<int>(t) && c.w == static_cast<int>(t);
                                qkv7[i] = __int_as_float(c.x);
                                qkv7[i + 1] = __int_as_float(c.z);
                            }
                            if (__builtin_amdgcn_readfirstlane(__all(ok))) break;
                            if (++spins > pb.spin_limit || ctl[kXAbandon] != 0u
                                || ((spins & 63u) == 0u
                                    && __hip_atomic_load(&pb.ctl->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
                                xcd_give_up(wt, t);
                                return;
                            }
                        }
                        lds_settle();
                        XROUNDS(6, spins);
                    }
                    XTICK(4);  // attention wavefront: 4 = wait for q, 5 = everything else
                    const float4 q4 = reinterpret_cast<const float4*>(qkv7)[dl];
                    float m = -INFINITY, lsum = 0.0f;
                    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
                    for (int batch = 0; t0 + batch * 32 < t1; batch++) {
                        if (batch >= 1) fetch(l, batch);
                        float sc[8];
#pragma unroll
                        for (int it = 0; it < 8; it++) {
                            const int tt = t0 + batch * 32 + it * 4 + sub;
                            if (tt == pos && tt < t1) {
                                k4[it] = reinterpret_cast<const float4*>(qkv7 + 64)[dl];
                                v4[it] = reinterpret_cast<const float4*>(qkv7 + 128)[dl];
                            }
                            const float sdot = row16_sum(dot4(q4, k4[it]));
                            sc[it] = tt < t1 ? sdot * 0.125f : -INFINITY;  // 1/sqrt(64)
                        }
                        float mb = sc[0];
#pragma unroll
                        for (int it = 1; it < 8; it++) mb = fmaxf(mb, sc[it]);
                        mb = fmaxf(mb, dpp_move<0x142, 0xA>(mb, mb));
                        mb = fmaxf(mb, dpp_move<0x143, 0xC>(mb, mb));
                        mb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mb), 63));
                        const float mn = fmaxf(m, mb);
                        if (mn > -INFINITY) {
                            // lane dl of a position group forms the exponential of score dl (lane 8:
                            // of the old maximum); the group shares them by row broadcasts
                            float arg = sc[0];
#pragma unroll
                            for (int it = 1; it < 8; it++) arg = (dl == it) ? sc[it] : arg;
                            arg = (dl == 8) ? m : arg;
                            const float em = expf(arg - mn);
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
                    }
                    // the four position groups share the running maximum: add their sums
                    lsum += __shfl_xor(lsum, 16, kWave);
                    acc.x += __shfl_xor(acc.x, 16, kWave);
                    acc.y += __shfl_xor(acc.y, 16, kWave);
                    acc.z += __shfl_xor(acc.z, 16, kWave);
                    acc.w += __shfl_xor(acc.w, 16, kWave);
                    lsum += __shfl_xor(lsum, 32, kWave);
                    acc.x += __shfl_xor(acc.x, 32, kWave);
                    acc.y += __shfl_xor(acc.y, 32, kWave);
                    acc.z += __shfl_xor(acc.z, 32, kWave);
                    acc.w += __shfl_xor(acc.w, 32, kWave);
                    {
                        Cell* out = p.xc + cl.ap + g * kApStrideCells + (a_hi * SL + a_slice) * kApCells;
                        const unsigned t = tag_of(l, 1);
                        if (sub == 0) {
                            cell_put_local(out + dl * 4 + 0, acc.x, t);
                            cell_put_local(out + dl * 4 + 1, acc.y, t);
                            cell_put_local(out + dl * 4 + 2, acc.z, t);
                            cell_put_local(out + dl * 4 + 3, acc.w, t);
                            if (dl == 0) {
                                cell_put_local(out + 64, m, t);
                                cell_put_local(out + 65, lsum, t);
                            }
                        }
                    }
                    // the next layer's cached rows do not depend on anything still to come
                    if (l + 1 < L) fetch(l + 1, 0);
                }
            }
            continue;
        }

        // ================= the team: wavefronts 0..6
        const int ctid = tid;  // 0..447
        // rotation of this workgroup's pairs at this position
        float rcs = 1.0f, rsn = 0.0f;
        int q_sec = 0, q_hi = 0, q_j = 0;
        if (wave < me.ppw) {
            const int pi = r * me.ppw + wave;
            q_hi = pi / 96;
            const int rem = pi - q_hi * 96;
            q_sec = rem >> 5;
            q_j = rem & 31;
            if (q_sec < 2) {
                rcs = pb.rope_cos[pos * (HS / 2) + q_j];
                rsn = pb.rope_sin[pos * (HS / 2) + q_j];
            }
        }
        for (int j = ctid; j < D; j += kXcdTeamLanes) xs[j] = pb.E[static_cast<size_t>(tok) * D + j];
        if (!xcd_team_sync(wt, bar_gen, lane)) return;

#ifdef GH_XCD_TICKS
        last_tick = static_cast<unsigned>(__builtin_amdgcn_s_memtime());
#endif
        for (int l = 0; l < L; l++) {
            const unsigned lay = static_cast<unsigned>(l) * me.layer_bytes;  // this layer in the step's stream
            auto unit_of = [&](unsigned off) { return unit_base + (off >> 10); };       // the unit holding byte off
            auto units_to = [&](unsigned off) { return unit_base + ((off + 1023u) >> 10); };  // units up to byte off

            // ===== P1: norm1 + QKV rows of this XCD's heads
            {
                float4 h[KD];
                float ss = 0.0f;
#pragma unroll
                for (int i = 0; i < KD; i++) {
                    h[i] = reinterpret_cast<const float4*>(xs)[i * 64 + lane];
                    ss += dot4(h[i], h[i]);
                }
                if (wave < me.ppw) {
                    const unsigned o = lay + static_cast<unsigned>(wave) * me.pair_bytes;
                    xcd_set_consumed(wt, wave, lane, unit_of(o));
                    if (!xcd_wait_filled(wt, units_to(o + me.pair_bytes), XSTALL(0))) return;
                    const float rn = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(D) + kNormEps);
                    float a = 0.0f, c = 0.0f;
                    const unsigned base = unit_base * kXcdUnit + o + lane * 16;
#pragma unroll
                    for (int i = 0; i < KD; i++) {
                        a += dot4(ring_ld4(ring, ring_mask, base + i * 1024), h[i]);
                        c += dot4(ring_ld4(ring, ring_mask, base + D * 4 + i * 1024), h[i]);
                    }
                    wave_sum2(a, c);
                    const float2 bias =
                        *reinterpret_cast<const float2*>(ring + ((unit_base * kXcdUnit + o + 2u * D * 4u) & ring_mask));
                    a = a * rn + bias.x;
                    c = c * rn + bias.y;
                    if (lane == 0) {
                        if (q_sec < 2) {
                            const float ra = a * rcs - c * rsn;
                            const float rc = a * rsn + c * rcs;
                            a = ra;
                            c = rc;
                        }
                        const unsigned t = tag_of(l, 0);
                        if (q_sec >= 1) {
                            float* cr = pb.kv.pool + kv_at(l, q_sec - 1, p.gm.shard[g].head[q_hi], pos) + 2 * q_j;
                            coherent_store(cr, a);
                            coherent_store(cr + 1, c);
                        }
                        Cell* dst = p.xc + cl.qkv + (g * 2 + q_hi) * 192 + q_sec * 64 + 2 * q_j;
                        cell_put_local(dst, a, t);
                        cell_put_local(dst + 1, c, t);
                    }
                }
                xcd_set_consumed(wt, wave, lane, unit_of(lay + me.o_wo));
            }
            XTICK(0);
            stamp();

            // ===== P3: merge the slices' partials, W_o over this XCD's columns -> partial sums
            float bo_row = 0.0f;
            {
                const int nap = SL * me.nh * kApCells;
                if (!xcd_gather<kAuxNonTemporal>(p.xc + cl.ap + g * kApStrideCells, nap, tag_of(l, 1), apbuf, ctid, wt, XSTALL(5)))
                    return;
                XTICK(1);
                if (!xcd_team_sync(wt, bar_gen, lane, XSTALL(9))) return;
                XTICK(2);
                stamp();
                if (wave < kXcdRowWaves) {
                    float* mine = att + wave * (128 + 32);
                    float* fw = mine + 128;  // [SL] this wavefront's merge factors
                    for (int hi = 0; hi < me.nh; hi++) {
                        // slice q's (m, l) sit in lane q; one exponential per lane
                        const float* ap = apbuf + hi * SL * kApCells;
                        const float mq = lane < SL ? ap[lane * kApCells + 64] : -INFINITY;
                        const float lq = lane < SL ? ap[lane * kApCells + 65] : 0.0f;
                        const float M = wave_max(mq);
                        const float fq = expf(mq - M);  // 0 for empty slices and idle lanes
                        const float Ls = wave_sum(lq * fq);
                        if (lane < SL) fw[lane] = fq;
                        lds_settle();
                        float o = 0.0f;
                        for (int q = 0; q < SL; q++) o += ap[q * kApCells + lane] * fw[q];
                        mine[hi * 64 + lane] = o * (1.0f / Ls);
                        lds_settle();
                    }
                    const int sub = lane >> 4, dl = lane & 15;
                    const int nk4 = me.KC / 4;  // 16 or 32 float4 per row
                    for (int row = 4 * wave + sub; row < RW; row += 4 * kXcdRowWaves) {
                        const unsigned o = lay + me.o_wo + static_cast<unsigned>(row) * me.KC * 4u;
                        if (!xcd_wait_filled(wt, units_to(lay + me.o_gu), XSTALL(1))) return;
                        const unsigned base = unit_base * kXcdUnit + o;
                        float a = 0.0f;
                        for (int i = dl; i < nk4; i += 16)
                            a += dot4(ring_ld4(ring, ring_mask, base + i * 16), reinterpret_cast<const float4*>(mine)[i]);
                        a = row16_sum(a);
                        if (dl == 0) cell_put(p.xc + cl.part + g * D + r * RW + row, a, tag_of(l, 2));
                    }
                }
                if (wave == kXcdRelayWave) {
                    // b_o of this workgroup's rows, for the sum that follows
                    if (!xcd_wait_filled(wt, units_to(lay + me.o_gu))) return;
                    bo_row = *reinterpret_cast<const float*>(
                        ring + ((unit_base * kXcdUnit + lay + me.o_bo + (lane < RW ? lane : 0) * 4) & ring_mask));
                }
                xcd_set_consumed(wt, wave, lane, unit_of(lay + me.o_gu));
            }
            XTICK(3);
            stamp();

            // ===== P4: this workgroup's rows: the eight partials in XCD order + residual -> x'
            auto relay = [&](int which, const float* resid, float bias, int ph_in, int ph_out) -> bool {
                const unsigned t = tag_of(l, ph_in);
                const int row = lane < RW ? lane : 0;
                const __amdgpu_buffer_rsrc_t rs =
                    make_buffer(p.xc + cl.part + which * kXcds * D, static_cast<unsigned>(kXcds * D) * 8u);
                float pv[kXcds];
                unsigned spins = 0;
                XTICK(14);
#pragma nounroll
                for (;;) {
                    bool ok = true;
#pragma unroll
                    for (int q = 0; q < kXcds; q++) {
                        const v2i c = __builtin_amdgcn_raw_buffer_load_b64(
                            rs, static_cast<unsigned>(q * D + r * RW + row) * 8u, 0, kAuxDeviceScope);
                        ok = ok && c.y == static_cast<int>(t);
                        pv[q] = __int_as_float(c.x);
                    }
                    if (__builtin_amdgcn_readfirstlane(__all(ok))) break;
                    if (++spins > pb.spin_limit || ctl[kXAbandon] != 0u
                        || ((spins & 63u) == 0u
                            && __hip_atomic_load(&pb.ctl->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
                        xcd_give_up(wt, t);
                        return false;
                    }
                }
                XTICK(which);  // relay wavefront: 0 / 1 = time in the two polls, 14 = everything else
                XROUNDS(2 + which, spins);
                float sum = pv[0];
#pragma unroll
                for (int q = 1; q < kXcds; q++) sum += pv[q];
                if (lane < RW)
                    cell_put_local(p.xc + cl.xr + (which * kXcds + g) * D + r * RW + lane,
                                   (resid[r * RW + lane] + bias) + sum, tag_of(l, ph_out));
                return true;
            };
            if (wave == kXcdRelayWave) {
                if (!relay(0, xs, bo_row, 2, 3)) return;
            }

            // ===== P5: norm2 + gate/up rows of this workgroup's hidden units -> hidden cells
            {
                if (!xcd_gather<kAuxNonTemporal>(p.xc + cl.xr + (0 * kXcds + g) * D, D, tag_of(l, 3), xs1, ctid, wt, XSTALL(6)))
                    return;
                XTICK(4);
                if (!xcd_team_sync(wt, bar_gen, lane, XSTALL(10))) return;
                XTICK(5);
                stamp();
                float4 h[KD];
                float ss = 0.0f;
#pragma unroll
                for (int i = 0; i < KD; i++) {
                    h[i] = reinterpret_cast<const float4*>(xs1)[i * 64 + lane];
                    ss += dot4(h[i], h[i]);
                }
                const float rn = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(D) + kNormEps);
                for (int k = wave; k < me.nu; k += kXcdTeamWaves) {
                    const unsigned o = lay + me.o_gu + static_cast<unsigned>(k) * 2u * D * 4u;
                    xcd_set_consumed(wt, wave, lane, unit_of(o));
                    if (!xcd_wait_filled(wt, units_to(o + 2u * D * 4u), XSTALL(2))) return;
                    const unsigned base = unit_base * kXcdUnit + o + lane * 16;
                    float a = 0.0f, c = 0.0f;
#pragma unroll
                    for (int i = 0; i < KD; i++) {
                        a += dot4(ring_ld4(ring, ring_mask, base + i * 1024), h[i]);
                        c += dot4(ring_ld4(ring, ring_mask, base + D * 4 + i * 1024), h[i]);
                    }
                    wave_sum2(a, c);
                    a *= rn;
                    c *= rn;
                    if (lane == 0)
                        cell_put_local(p.xc + cl.hid + g * cl.hid_stride + (me.ub - me.u0) + k, c * silu(a), tag_of(l, 4));
                }
                xcd_set_consumed(wt, wave, lane, unit_of(lay + me.o_dn));
            }
            XTICK(6);
            stamp();

            // ===== P6: W_down over this XCD's hidden units -> partial sums
            {
                if (!xcd_gather<kAuxNonTemporal>(p.xc + cl.hid + g * cl.hid_stride, me.UG, tag_of(l, 4), hbuf, ctid, wt, XSTALL(7), XTRIP(12)))
                    return;
                XTICK(7);
                if (!xcd_team_sync(wt, bar_gen, lane, XSTALL(11))) return;
                XTICK(8);
                stamp();
                if (wave < kXcdRowWaves) {
                    const int sub = lane >> 4, dl = lane & 15;
                    const int nk4 = me.UG / 4;
                    for (int row = 4 * wave + sub; row < RW; row += 4 * kXcdRowWaves) {
                        const unsigned o = lay + me.o_dn + static_cast<unsigned>(row) * me.UG * 4u;
                        if (!xcd_wait_filled(wt, units_to(lay + me.layer_bytes), XSTALL(3))) return;
                        const unsigned base = unit_base * kXcdUnit + o;
                        float a = 0.0f;
                        for (int i = dl; i < nk4; i += 16)
                            a += dot4(ring_ld4(ring, ring_mask, base + i * 16), reinterpret_cast<const float4*>(hbuf)[i]);
                        a = row16_sum(a);
                        if (dl == 0) cell_put(p.xc + cl.part + (kXcds + g) * D + r * RW + row, a, tag_of(l, 5));
                    }
                }
                xcd_set_consumed(wt, wave, lane, unit_of(lay + me.layer_bytes));
            }
            XTICK(9);
            stamp();

            // ===== P7: rows of this workgroup: partials + residual -> x of the next layer
            if (wave == kXcdRelayWave) {
                if (!relay(1, xs1, 0.0f, 5, 6)) return;
            }
            if (!xcd_gather<kAuxNonTemporal>(p.xc + cl.xr + (1 * kXcds + g) * D, D, tag_of(l, 6), xs, ctid, wt, XSTALL(8), XTRIP(13))) return;
            XTICK(10);
            if (!xcd_team_sync(wt, bar_gen, lane, XSTALL(12))) return;
            XTICK(11);
            stamp();
        }
        unit_base += me.layers_units;

        if (want_logits) {
            // ===== final norm + logits (inference.cpp:251-254): this workgroup's rows of E
            float4 h[KD];
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < KD; i++) {
                h[i] = reinterpret_cast<const float4*>(xs)[i * 64 + lane];
                ss += dot4(h[i], h[i]);
            }
            const float rn = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(D) + kNormEps);
            for (int row = 2 * wave; row < me.nrows; row += 2 * kXcdTeamWaves) {
                const bool two = row + 1 < me.nrows;
                const unsigned o = static_cast<unsigned>(row) * D * 4u;
                xcd_set_consumed(wt, wave, lane, unit_base + (o >> 10));
                if (!xcd_wait_filled(wt, unit_base + ((o + (two ? 2u : 1u) * D * 4u + 1023u) >> 10), XSTALL(4))) return;
                const unsigned base = unit_base * kXcdUnit + o + lane * 16;
                float a = 0.0f, c = 0.0f;
#pragma unroll
                for (int i = 0; i < KD; i++) {
                    a += dot4(ring_ld4(ring, ring_mask, base + i * 1024), h[i]);
                    if (two) c += dot4(ring_ld4(ring, ring_mask, base + D * 4 + i * 1024), h[i]);
                }
                wave_sum2(a, c);
                if (lane == 0) {
                    const int v = me.v0 + row;
                    coherent_store(pb.logits + v, a * rn);
                    if (pb.logit_log) pb.logit_log[static_cast<size_t>(s) * V + v] = a * rn;
                    if (two) {
                        coherent_store(pb.logits + v + 1, c * rn);
                        if (pb.logit_log) pb.logit_log[static_cast<size_t>(s) * V + v + 1] = c * rn;
                    }
                }
            }
            unit_base += me.logits_units;
            xcd_set_consumed(wt, wave, lane, unit_base);
            // this workgroup's rows are out (acknowledged by the memory side): signal
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (!xcd_team_sync(wt, bar_gen, lane)) return;
            arrive_gen++;
            if (tid == 0)
                __hip_atomic_fetch_add(&pb.ctl->arrive[(wgid & 15) * 32], 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        } else {
            xcd_set_consumed(wt, wave, lane, unit_base);
        }
        stamp();
    }
    if (!streamer && tid == 0) {
        ctl[kXDone] = 1u;
#ifdef GH_XCD_TICKS
        if (pb.prof && wg == 0) {
            for (int i = 0; i < 13; i++) pb.prof[pb.prof_cap - 16 + i] = stall[i] + 1u;
            for (int i = 0; i < 16; i++) pb.prof[pb.prof_cap - 48 + i] = dur[i] + 1u;
        }
#endif
    }
#ifdef GH_XCD_TICKS
    if (pb.prof && wg == 0 && lane == 0 && wave == kXcdRelayWave)
        for (int i = 0; i < 16; i++) pb.prof[pb.prof_cap - 80 + i] = dur[i] + 1u;
    if (pb.prof && wg == 0 && lane == 0 && wave == kXcdAttnWave)
        for (int i = 0; i < 16; i++) pb.prof[pb.prof_cap - 112 + i] = dur[i] + 1u;
#endif
}

}  // namespace gh

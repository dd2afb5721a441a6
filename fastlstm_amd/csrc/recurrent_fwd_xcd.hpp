// Persistent forward kernel, XCD-local form: the hidden tiles of one batch tile all run on ONE
// of the 8 XCDs of an MI355X and exchange h_t through that XCD's L2 instead of through memory.
//
// Same mathematics and the same results as lstm_fwd_persistent_kernel (which replaces
// fastlstm/kernels.py:414-663); what differs is where the data travels:
//  * placement: the hardware deals the workgroups of a dispatch to the XCDs in turn: workgroup i runs on
//    XCD (i + r) % 8, with one rotation r per dispatch.  A barrier group takes its members from the
//    workgroups with i % 8 == group % 8, which share an XCD whatever r is; workgroups that are not needed
//    return at once.  One workgroup fills the register file of a CU, so the up to 32 members of a group
//    sit on the 32 CUs of their XCD.  The host verifies the dealing once per device before it selects this
//    kernel, and every launch verifies that its workgroups saw one common r (check_xcd_placement);
//  * exchange data: ordinary stores (the vector L1 writes through to L2) into one of TWO slots (h_v in slot
//    v % 2: a slot is rewritten only after every member has published the version behind it, i.e. has read
//    it), and loads that bypass the L1 and are served by the XCD's L2 (sc1): nobody keeps the L1s coherent,
//    and a slot's address is reused every other step.  The exchange data never leaves the L2 (a ring with an
//    address per timestep, read through the L1, was 10 - 25 % slower per step and cost O(T) workspace);
//  * barrier: counters in L2.  Atomics execute in the L2, never in an L1: a member adds 1 to
//    each of kXcdReplicas counters of its group after its stores were acknowledged, and polls
//    one of them (its index % replicas) with scalar loads that bypass the scalar cache;
//  * W_h: a slice of 4*MT units x 4 gates x H no longer has to fit in LDS next to the peers'
//    (32 CUs x 160 KiB < 8 MiB for H = 1024): every wave keeps its K-share of the slice, MT x NKW
//    operand fragments, in registers (up to 256 of the 512 per lane).
// Requirements (host): H a multiple of the tile width and of 16 bytes' worth of elements,
// H / (4*MT) <= 32 members, ceil(H / KSTEP) <= 4*NKW k-steps, all batch tiles in one launch.
#pragma once
#include <type_traits>

#include "gemm.hpp"
#include "gemm16.hpp"
#include "recurrent_common.hpp"

namespace fastlstm {

constexpr int kXcdReplicas = 8;          // counters per barrier group, 128 bytes apart
constexpr int kXcdCounterStride = 32;    // ints between replicas
constexpr int kXcdGroupStride = kXcdReplicas * kXcdCounterStride;   // ints between groups (1 KiB)
constexpr int kXcdMaxGroups = 64;
static_assert((size_t)kXcdMaxGroups * kXcdGroupStride * sizeof(int) == kWsCounterBytes, "counter region of the workspace");
static_assert(kXcdMaxGroups % kNumXcd == 0, "the same number of groups on every XCD");

struct FwdXcdParams {
    void *ifgo;        // [T,B,4H] in: x.Wx^T+b, out: full pre-activations
    void *out, *cell;  // [T+1,B,H]
    const void *Wh;    // [4H,H]
    WsHeader *hdr;
    int *counters;        // [groups][kXcdReplicas][kXcdCounterStride], zero at launch
    unsigned char *xbuf;  // [2 slots][groups][NT][KS] operand blocks; h_v lives in slot v % 2
    int T, B, H;
    int n_ht;          // members of a barrier group (<= 32)
    int gpx;           // groups per XCD (32 / n_ht)
    int n_groups;      // batch tiles of this launch (<= 8 * gpx)
    int b_base;        // first batch row of this launch (a large batch runs as several launches over row ranges)
    int KS;            // k-steps covering H
    // In-kernel input projection (HELP instantiations, k1_tiles_n > 0): the workgroups without a
    // role in the recurrence compute ifgo = x.Wx^T + b in 256 x 256 tiles, earliest timesteps first;
    // k1_done[c] counts the finished tiles of chunk c (k1_chunk_tiles row tiles = k1_chunk_steps
    // timesteps), and the recurrence requests the gates of a timestep only when its chunk is done.
    GemmParams k1;        // M = T*B, N = 4H, K = I, A = x, B = Wx, C = ifgo, biases
    int k1_tiles_m, k1_tiles_n;
    int k1_chunk_tiles, k1_chunk_steps;
    int *k1_done;         // [<= kMaxChunks] device-scope counters, zero at launch
    // Two stacked layers in one launch (n_layers == 2, HELP instantiations): the second layer's barrier
    // groups follow the first layer's in the group numbering (so they sit on other XCDs or CUs), its
    // input projection reads the first layer's out[1:] chunk by chunk as that layer produces it
    // (out_ready[c] counts the first layer's workgroups whose h of chunk c are in memory), and its
    // recurrence follows its own projection like the first layer's does.
    int n_layers;
    void *ifgo2, *out2, *cell2;
    const void *Wh2;
    // Without helpers n_layers = 2 ... kMaxSideBySide independent recurrences of one shape share the launch (the two
    // directions of a bidirectional layer; the chunks of a wavefront over stacked layers): recurrence r >= 2 is
    // described by the r - 2-th entries here.
    void *ifgo_more[2], *out_more[2], *cell_more[2];
    const void *Wh_more[2];
    GemmParams k1b;       // M = T*B, N = 4H, K = H, A = out[1:] of the first layer, B = Wx2, C = ifgo2, biases
    int *k1_done2;        // chunk counters of the second projection
    int *out_ready;       // [<= kMaxChunks] device-scope counters, zero at launch
    int n_active;         // workgroups of one layer's recurrence (groups * members)
    int keep;             // 1: store pre-activations and every cell state (training); 0: inference, only cell[T]
    long long spin_limit;
    long long *trace;  // diagnostic build only
};

// Exchange ring accessed with ordinary (cached) 16-byte loads and ordinary stores.
struct XchgL2 {
    __amdgpu_buffer_rsrc_t rsrc;
    __device__ __forceinline__ XchgL2(unsigned char *b, unsigned bytes)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(b, 0, bytes, 0x00020000)) {}
    // ordinary load: may be served by the CU's L1 (only for addresses that are written once per launch)
    __device__ __forceinline__ u32x4 load16(unsigned off) const {
        return __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
    }
    // served by the L2: the L1, which may hold the line from the slot's previous use, is bypassed (sc1)
    __device__ __forceinline__ u32x4 load16_l2(unsigned off) const {
        return __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 16);
    }
    template <typename T> __device__ __forceinline__ void store_elem(unsigned off, T v) const {
        if constexpr (sizeof(T) == 2) __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), rsrc, off, 0, 0);
        else __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rsrc, off, 0, 0);
    }
};

// The calling wave polls `counter` in L2 until it reaches `target`.  The poll is a scalar load
// with the glc bit (it misses the scalar cache and is served by the L2; the vector L1, which
// could hold a stale line, is not on its path) -- half the round trip of a returning L2 atomic.
// A stale value can only be too small, i.e. delay the wait, never release it early.  Bounded like
// wait_versions.
__device__ __forceinline__ void wait_counter(int *counter, int target, WsHeader *hdr, long long spin_limit,
                                             int group, int step) {
    long long t0 = 0;
    int polls = 0;
    counter = uniform_ptr(counter);   // the scalar load needs its address in scalar registers
    for (;;) {
        int v;
        asm volatile("s_load_dword %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(counter) : "memory");
        if (v >= target) break;
        __builtin_amdgcn_s_sleep(1);
        if (++polls >= 64 || spin_limit <= 1) {
            polls = 0;
            if (__hip_atomic_load(&hdr->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
            const long long now = (long long)wall_clock64();
            if (t0 == 0 && spin_limit > 1) {
                t0 = now;
            } else if (now - t0 > spin_limit) {
                if ((threadIdx.x & (kWave - 1)) == 0) {
                    hdr->timeout_group = group;
                    hdr->timeout_step = step;
                    __hip_atomic_store(&hdr->abort_flag, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                }
                break;
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");   // compiler ordering only
}

// Rank of the calling workgroup among the workgroups of the launch that have no role in the
// recurrence, counted XCD by XCD, and their number: helpers with consecutive ranks share an L2.
// (Roles: see the placement rule at the top of the kernels.)
__device__ __forceinline__ int helper_rank(int n_ht, int gpx, int n_groups, int *n_helpers) {
    const int my_xcd = blockIdx.x % kNumXcd, my_slot = blockIdx.x / kNumXcd;
    const int slots = gridDim.x / kNumXcd;
    int rank = 0, total = 0;
    for (int x = 0; x < kNumXcd; ++x)
        for (int sl = 0; sl < slots; ++sl) {
            const int gl = sl / n_ht;
            const bool idle = gl >= gpx || gl * kNumXcd + x >= n_groups;
            total += idle;
            rank += idle && (x < my_xcd || (x == my_xcd && sl < my_slot));
        }
    *n_helpers = total;
    return rank;
}

// Input projection by a workgroup (8 waves) that has no role in the recurrence.  Helper h of n
// takes tiles h, h + n, ... of the time-ordered tile list of each layer.  A finished tile is made
// visible to the other XCDs (its stores acknowledged, this XCD's L2 written back: the release of the
// atomic) before it is counted.  With two layers a helper prefers the second layer's next tile
// whenever the first layer has delivered the timesteps that tile reads (one poll), and otherwise
// goes on with the first layer's list, which never has to wait for anything.
template <typename T>
__device__ __forceinline__ void k1_helper(const FwdXcdParams &p, unsigned char *smem) {
    int n_helpers;
    const int h = helper_rank(p.n_ht, p.gpx, p.n_groups * p.n_layers, &n_helpers);
    int total = p.k1_tiles_m * p.k1_tiles_n;   // length of the tile list
    int *ready_flag = reinterpret_cast<int *>(smem);
    // List position -> tile.  Plain: row-major over (row tile, column tile).  Where the helpers are whole
    // XCDs and the column tiles divide among them, the tiles of a round (n_helpers of them: the same
    // row tiles either way) are dealt so that an XCD keeps to its own column tiles: its panel of Wx
    // (a few MiB) stays in that XCD's L2 for the whole launch instead of all of Wx streaming through
    // every L2 once per pair of row tiles; x is then read by every helper XCD.
    const int tn = p.k1_tiles_n, xcds = n_helpers / 32, cpx = xcds ? tn / xcds : 0;
    const bool by_panel = n_helpers % 32 == 0 && xcds > 0 && tn % xcds == 0 && cpx > 0 && 32 % cpx == 0;
    auto tile_of = [&](int idx, int *rt, int *ct) {
        if (by_panel) {
            const int round = idx / n_helpers, k = h / 32, sl = h % 32;
            *rt = round * (32 / cpx) + sl / cpx;
            *ct = k * cpx + sl % cpx;
        } else {
            *rt = idx / tn;
            *ct = idx % tn;
        }
    };
    if (by_panel) total = cdiv(p.k1_tiles_m, 32 / cpx) * n_helpers;   // whole rounds; positions past the last row tile are skipped
    int i0 = h, i1 = p.n_layers > 1 ? h : total;
    while (i0 < total || i1 < total) {
        {
            int r_, c_;
            if (i0 < total) {
                tile_of(i0, &r_, &c_);
                if (r_ >= p.k1_tiles_m) { i0 += n_helpers; continue; }
            }
            if (i1 < total) {
                tile_of(i1, &r_, &c_);
                if (r_ >= p.k1_tiles_m) { i1 += n_helpers; continue; }
            }
        }
        bool second = false;
        if (i1 < total) {
            int rt1, ct1;
            tile_of(i1, &rt1, &ct1);
            const int c1 = rt1 / p.k1_chunk_tiles;
            if (i0 < total) {   // one poll: is the chunk there?
                if (threadIdx.x == 0)
                    *ready_flag = __hip_atomic_load(p.out_ready + c1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= p.n_active;
                __syncthreads();
                second = *ready_flag != 0;
                __syncthreads();   // the flag's LDS word is part of the GEMM stages
            } else {            // nothing else to do: wait for it
                if ((threadIdx.x >> 6) == 0)
                    wait_versions<100>(p.out_ready + c1, 1, p.n_active, p.hdr, p.spin_limit, -2, c1);
                __syncthreads();
                second = true;
            }
            if (second) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // the first layer's h, written on other XCDs
        }
        int rt, ct;
        tile_of(second ? i1 : i0, &rt, &ct);
        // (the ping-pong main loop, ordinary stores: the time loop reads these gates within a chunk or two)
        if (second) gemm16_tile<T, false, false, 256, 256, 2, 2, 4, 2, false, true>(p.k1b, rt * 256, ct * 256, 0, smem, 0);
        else gemm16_tile<T, false, false, 256, 256, 2, 2, 4, 2, false, true>(p.k1, rt * 256, ct * 256, 0, smem, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();   // every wave's part of the tile is in the L2 (and the LDS may be reused)
        if (threadIdx.x == 0)
            __hip_atomic_fetch_add((second ? p.k1_done2 : p.k1_done) + rt / p.k1_chunk_tiles, 1, __ATOMIC_RELEASE,
                                   __HIP_MEMORY_SCOPE_AGENT);
        if (second) i1 += n_helpers;
        else i0 += n_helpers;
    }
}

// The waves split K four ways: wave w owns k-steps w % 4, w % 4 + 4, ... (NKW of them).  With
// NWV = 8 waves (two per SIMD, 256 registers each) the two waves of a K-share split the MT unit
// tiles between them, which halves the fragments a wave holds and leaves registers to keep all
// operand loads of a step in flight.
template <typename T, int MT, int NKW, int NTW, int NWV, bool HELP = false>
__global__ __launch_bounds__(kWave * NWV) void lstm_fwd_xcd_kernel(const FwdXcdParams p) {
    static_assert(!HELP || (NWV == 8 && sizeof(T) == 2), "the in-kernel GEMM tile is the 8-wave 16-bit one");
    constexpr int NTHR = kWave * NWV;
    constexpr int MW = NWV / 4, MTW = MT / MW;       // M-split ways, unit tiles per wave
    static_assert(NWV == 4 || NWV == 8, "4 or 8 waves");
    static_assert(MT % MW == 0, "unit tiles divide among the waves of a K-share");
    using E = Elem<T>;
    constexpr bool ACC = (E::DT == FASTLSTM_FP32);
    constexpr int NT = NTW, TILES = MT * NT;
    constexpr int IPT = (TILES + NWV - 1) / NWV;     // (tile, lane) items per thread
    constexpr int HT = 4 * MT, BT = 16 * NT;
    constexpr int GSEG = HT * E::BYTES;              // bytes of one gate segment of a row (>= 16)
    static_assert(GSEG >= 16 && GSEG % 16 == 0, "tile I/O needs 16-byte gate segments");
    constexpr int GROW = 4 * GSEG + 16, SROW = GSEG + 16;
    constexpr int PPSEG = GSEG / 16;
    constexpr int GPIECES = BT * 4 * PPSEG, SPIECES = BT * PPSEG;
    constexpr int IOT = NTHR - kWave;                // waves 1.. move the tiles, wave 0 polls
    constexpr int GPT = (GPIECES + IOT - 1) / IOT, SPT = (SPIECES + IOT - 1) / IOT;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // (uniform: in a scalar register)
    const int q = lane >> 4, n = lane & 15;
    const int KS = p.KS, H = p.H, B = p.B, T_ = p.T;
    const bool keep = p.keep != 0;   // training: gate pre-activations and every cell state are stored

    // ---- placement: group g lives on XCD g % 8 ------------------------------------------
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int gl = slot / p.n_ht, j = slot % p.n_ht;
    const int vg = gl * kNumXcd + xcd;          // group index over all layers of the launch
    // (without helpers n_layers == 2 means two independent recurrences of the same shape side by side: the two
    // directions of a bidirectional layer; nothing links them)
    const int n_layers = HELP ? (p.n_layers > 1 ? 2 : 1) : max(1, min(p.n_layers, kMaxSideBySide));
    if (gl >= p.gpx || vg >= p.n_groups * n_layers) {
        if constexpr (HELP) {
            if (p.k1_tiles_n > 0) k1_helper<T>(p, smem);
        }
        return;
    }
    check_xcd_placement(p.hdr);
    const int layer = vg / p.n_groups, g = vg % p.n_groups;   // layer 1: the second of a stack
    const int u0 = j * HT, b0 = p.b_base + g * BT;   // b_base: first batch row of this launch
    const bool k1_live = HELP && p.k1_tiles_n > 0;
    // chunk c of ifgo is complete when all its tiles were counted
    auto wait_chunk = [&](int c, int t) {
        const int rows = min(p.k1_chunk_tiles, p.k1_tiles_m - c * p.k1_chunk_tiles);
        wait_versions((layer ? p.k1_done2 : p.k1_done) + c, 1, rows * p.k1_tiles_n, p.hdr, p.spin_limit, vg, t);
    };
    // a first layer tells the helpers which chunks of its h are in memory (see the step loop)
    const bool feeds = HELP && n_layers > 1 && layer == 0;

    f32x4 *red = reinterpret_cast<f32x4 *>(smem);                                  // [4][TILES][64]
    unsigned char *tiles = reinterpret_cast<unsigned char *>(red + 4 * TILES * kWave);   // gates, h, c tiles
    const int io_tid = tid - kWave;

    // (constant indices only: a run-time index into the kernel's arguments would move them all to scratch memory;
    // the helper instantiations never see more than two layers)
    auto pick = [&](auto a0, auto a1, auto a2, auto a3) {
        if constexpr (HELP) return layer ? a1 : a0;
        else return layer == 0 ? a0 : layer == 1 ? a1 : layer == 2 ? a2 : a3;
    };
    T *ifgo = static_cast<T *>(pick(p.ifgo, p.ifgo2, p.ifgo_more[0], p.ifgo_more[1]));
    T *out = static_cast<T *>(pick(p.out, p.out2, p.out_more[0], p.out_more[1]));
    T *cell = static_cast<T *>(pick(p.cell, p.cell2, p.cell_more[0], p.cell_more[1]));
    const T *Wh = static_cast<const T *>(pick(p.Wh, p.Wh2, p.Wh_more[0], p.Wh_more[1]));

#ifdef FASTLSTM_TIMELINE
    long long *tl = reinterpret_cast<long long *>(tiles + BT * GROW + 2 * BT * SROW + 64);
    for (int idx = tid; idx < 256; idx += NTHR) tl[idx] = 0;
    __syncthreads();
    if (tid == 0) {
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        tl[15] = (long long)(xcc & 15u);
    }
#define FASTLSTM_TP(ev)                                                                              \
    do {                                                                                             \
        if (lane == 0 && wave < 4 && t >= 200 && t < 204) tl[((t - 200) * 4 + wave) * 16 + (ev)] = (long long)wall_clock64(); \
    } while (0)
#else
#define FASTLSTM_TP(ev) do {} while (0)
#endif

    // ---- prologue 1: this wave's fragments of the W_h slice, global -> registers ---------
    // fragment (m-tile a, k-step ks): lane (q, r) holds row r = (unit a*4 + r/4, gate r%4),
    // k = ks*KSTEP + q*EPL .. + EPL-1, i.e. 16 contiguous bytes of W_h
    const int kq = wave & 3, mh = wave >> 2;         // K-share and M-half of this wave
    u32x4 wreg[MTW][NKW];
#pragma unroll
    for (int a = 0; a < MTW; ++a)
#pragma unroll
        for (int ki = 0; ki < NKW; ++ki) {
            const int ks = kq + 4 * ki;
            const int unit = u0 + (mh * MTW + a) * 4 + (n >> 2), gate = n & 3;
            const int k0 = ks * E::KSTEP + q * E::EPL;
            const bool ok = ks < KS && k0 < H;   // H % EPL == 0: a piece is inside or outside as a whole
            const size_t off = ok ? ((size_t)gate * H + unit) * H + k0 : 0;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(Wh + off);
            wreg[a][ki] = ok ? v : u32x4{0u, 0u, 0u, 0u};
        }

    // ---- per-thread items: (tile = wave + 4m, lane) -> (unit, batch row) -------------
    float c_state[IPT];
    size_t off_h[IPT];
    int xoff[IPT], goff[IPT], soff[IPT];
    bool valid[IPT];
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        const int tile = wave + NWV * m;
        const int mt = tile / NT, nt = tile % NT;
        const int unit = u0 + mt * 4 + q, b = b0 + nt * 16 + n;
        valid[m] = (tile < TILES) && b < B;
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        xoff[m] = nt * KS * kFragBytes + frag_offset<T>(n, unit);
        goff[m] = (nt * 16 + n) * GROW + (mt * 4 + q) * E::BYTES;
        soff[m] = (nt * 16 + n) * SROW + (mt * 4 + q) * E::BYTES;
        c_state[m] = valid[m] ? E::to_f32(cell[off_h[m]]) : 0.f;
    }

    // exchange ring: slot v holds h_{v-1}... slot s = version index: h_s for s = 0..T
    const unsigned xgrp = (unsigned)vg * NT * KS * kFragBytes;
    const size_t xslot = (size_t)p.n_groups * n_layers * NT * KS * kFragBytes;
    int *grp_counters = p.counters + (size_t)vg * kXcdGroupStride;
    int *my_counter = grp_counters + (j % kXcdReplicas) * kXcdCounterStride;

    auto publish = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's exchange stores have reached the L2
        __syncthreads();
        if (tid < kXcdReplicas)
            __hip_atomic_fetch_add(grp_counters + tid * kXcdCounterStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };

    // ---- prologue 2: publish h_0 (slot 0) -------------------------------------------------
    {
        const XchgL2 x0(p.xbuf, (unsigned)xslot);
#pragma unroll
        for (int m = 0; m < IPT; ++m)
            if (valid[m]) x0.store_elem(xgrp + xoff[m], out[off_h[m]]);
        publish();
    }

    const size_t BH = (size_t)B * H, B4H = (size_t)B * 4 * H;

    // ---- coalesced tile I/O (see lstm_fwd_persistent_kernel) --------------------------------
    // The gates tile of a step is requested ahead of its use.  Groups of 16 rows hold it in registers for two
    // steps (gpre) and copy it into the LDS tile when its step comes.  Groups of 32 rows have no registers to
    // spare for that (it was spilled right behind its load, and the spill waited for the load: a memory round
    // trip in every step): there the tile goes global -> LDS tile with LDS-direct loads, one step ahead, slot
    // by slot (a padded tile row is SPR slots of 16 bytes; lane l of wave instruction i fills slot 64 i + l,
    // the pad slot of a row and rows past B stay untouched), and leaves by the same slots.
    constexpr bool DMA = NTW == 2 && NWV == 8;
    constexpr int PD = DMA ? 1 : 2;
    constexpr int SPR = GROW / 16, SLOTS = BT * SPR;
    constexpr int DMA_N = (SLOTS + kWave - 1) / kWave, DPW = (DMA_N + NWV - 2) / (NWV - 1);
    constexpr int GD = DMA ? DPW : GPT;   // gate pieces (or slots) per thread
    u32x4 gpre[DMA ? 1 : PD][DMA ? 1 : GPT];
    const size_t tile_org = (size_t)b0 * 4 * H + u0;
    // Tile I/O goes through buffer loads / stores: the step's base address in scalar registers, per-lane byte offsets
    // that never change (no 64-bit address arithmetic in vector registers per step)
    unsigned g_off[GD], s_off[SPT];
    int g_lds[GD], s_lds[SPT];
    bool g_ok[GD], s_ok[SPT];
#pragma unroll
    for (int i = 0; i < GD; ++i) {
        int row, seg, k;
        if constexpr (DMA) {
            const int wi = (wave - 1) + (NWV - 1) * i, sl = wi * kWave + lane, idx = sl % SPR;
            row = sl / SPR; seg = idx / PPSEG; k = idx % PPSEG;
            g_ok[i] = wave >= 1 && wi < DMA_N && sl < SLOTS && idx < 4 * PPSEG && b0 + row < B;
            g_lds[i] = g_ok[i] ? sl * 16 : 0;
        } else {
            const int pc = io_tid + IOT * i, rem = pc % (4 * PPSEG);
            row = pc / (4 * PPSEG); seg = rem / PPSEG; k = rem % PPSEG;
            g_ok[i] = io_tid >= 0 && pc < GPIECES && b0 + row < B;
            g_lds[i] = g_ok[i] ? row * GROW + seg * GSEG + k * 16 : 0;
        }
        g_off[i] = g_ok[i] ? (unsigned)(((size_t)row * 4 * H + (size_t)seg * H + k * (16 / E::BYTES)) * E::BYTES) : 0u;
    }
#pragma unroll
    for (int i = 0; i < SPT; ++i) {
        const int pc = io_tid + IOT * i;
        const int row = pc / PPSEG, k = pc % PPSEG;
        s_ok[i] = io_tid >= 0 && pc < SPIECES && b0 + row < B;
        s_off[i] = s_ok[i] ? (unsigned)(((size_t)row * H + k * (16 / E::BYTES)) * E::BYTES) : 0u;
        s_lds[i] = s_ok[i] ? row * SROW + k * 16 : 0;
    }
    const size_t state_org = (size_t)b0 * H + u0;
    const unsigned g_bytes = (unsigned)((size_t)BT * 4 * H * E::BYTES), s_bytes = (unsigned)((size_t)BT * H * E::BYTES);
    auto fetch_tile = [&](int t, u32x4(&dst)[DMA ? 1 : GPT]) {
        if (io_tid < 0) return;
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(ifgo + (size_t)t * B4H + tile_org, 0, g_bytes, 0x00020000);
        if constexpr (DMA) {
#pragma unroll
            for (int i = 0; i < GD; ++i)
                if (g_ok[i]) load_block_to_lds(rg, tiles + (size_t)((wave - 1) + (NWV - 1) * i) * kFragBytes, g_off[i], 0);
        } else {
#pragma unroll
            for (int i = 0; i < GPT; ++i) dst[i] = __builtin_amdgcn_raw_buffer_load_b128(rg, g_off[i], 0, 0);   // (pieces that do not exist read the tile's first bytes)
        }
    };
    auto tile_to_lds = [&](const u32x4(&src)[DMA ? 1 : GPT], unsigned char *gt) {
        if constexpr (!DMA) {
#pragma unroll
            for (int i = 0; i < GPT; ++i) {
                const int pc = io_tid + IOT * i;
                const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG);
                if (io_tid >= 0 && pc < GPIECES)
                    *reinterpret_cast<u32x4 *>(gt + row * GROW + (rem / PPSEG) * GSEG + (rem % PPSEG) * 16) = src[i];
            }
        }
    };
    auto tiles_to_global = [&](int t, const unsigned char *gt) {
        const unsigned char *sth = gt + BT * GROW, *stc = sth + BT * SROW;
        if (keep) {
            const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(ifgo + (size_t)t * B4H + tile_org, 0, g_bytes, 0x00020000);
#pragma unroll
            for (int i = 0; i < GD; ++i)
                if (g_ok[i]) __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(gt + g_lds[i]), rg, g_off[i], 0, 0);
        }
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(out + (size_t)(t + 1) * BH + state_org, 0, s_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(cell + (size_t)(t + 1) * BH + state_org, 0, s_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < SPT; ++i)
            if (s_ok[i]) {
                // a first layer that feeds a second one in the same launch writes its h THROUGH to memory
                // (sc1): the chunk hand-over below then needs no write-back of this XCD's L2
                const u32x4 hv = *reinterpret_cast<const u32x4 *>(sth + s_lds[i]);
                if (feeds) __builtin_amdgcn_raw_buffer_store_b128(hv, rh, s_off[i], 0, 16);
                else __builtin_amdgcn_raw_buffer_store_b128(hv, rh, s_off[i], 0, 0);
                if (keep || t + 1 == T_)
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(stc + s_lds[i]), rc, s_off[i], 0, 0);
            }
    };
    auto prefetch = [&](int t, auto uc) __attribute__((always_inline)) {
        constexpr int u = DMA ? 0 : decltype(uc)::value;
        if (t < T_) fetch_tile(t, gpre[u]);
    };
    if (k1_live) {   // the first chunk of the input projection has to be there
        if (wave == 0) wait_chunk(0, 0);
        __syncthreads();
    }
    prefetch(0, std::integral_constant<int, 0>{});
    if constexpr (PD > 1) prefetch(1, std::integral_constant<int, 1>{});

    auto step = [&](const int t, auto uc) __attribute__((always_inline)) {
        constexpr int u = DMA ? 0 : decltype(uc)::value;
        unsigned char *gt = tiles;
        FASTLSTM_TP(0);
        // the gates of step t + PD are requested at the end of this step: their chunk must have landed
        // (the barrier below orders the poll before the request)
        if (k1_live && t + PD < T_ && (t + PD) % p.k1_chunk_steps == 0 && wave == 0)
            wait_chunk((t + PD) / p.k1_chunk_steps, t);
        if (wave == 0) wait_counter(my_counter, p.n_ht * (t + 1), p.hdr, p.spin_limit, vg, t);
        FASTLSTM_TP(1);
        __syncthreads();
        FASTLSTM_TP(2);
        // Every workgroup of the group has published h_t, behind the acknowledgement of everything it
        // stored before: out[t-1] (stored in step t-2, written through) is in memory.  When step t-2
        // closed a chunk, ONE workgroup counts the chunk for the whole group.
        if (feeds && j == 0 && tid == kWave && t >= 2 && (t - 1) % p.k1_chunk_steps == 0)
            __hip_atomic_fetch_add(p.out_ready + (t - 1) / p.k1_chunk_steps - 1, p.n_ht, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);

        // ---- acc[a][i] += Wslice(a) . h_{t-1}(i)^T over this wave's k-steps: all operand blocks
        // of the wave are requested at once, the weights come from registers
        const XchgL2 xr(p.xbuf + (size_t)(t & 1) * xslot, (unsigned)xslot);
        f32x4 acc[MTW][NTW];
#pragma unroll
        for (int a = 0; a < MTW; ++a)
#pragma unroll
            for (int i = 0; i < NTW; ++i) acc[a][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        u32x4 bq[NKW][NTW];
#pragma unroll
        for (int ki = 0; ki < NKW; ++ki) {
            const int ks = min(kq + 4 * ki, KS - 1);   // past the end: any valid block (its weights are zero)
#pragma unroll
            for (int i = 0; i < NTW; ++i) bq[ki][i] = xr.load16_l2(xgrp + (unsigned)((i * KS + ks) * kWave + lane) * 16u);
        }
        __builtin_amdgcn_sched_barrier(0);   // all loads are issued before the first MFMA: one round trip, not NKW
#pragma unroll
        for (int ki = 0; ki < NKW; ++ki)
#pragma unroll
            for (int a = 0; a < MTW; ++a)
#pragma unroll
                for (int i = 0; i < NTW; ++i) acc[a][i] = mfma_kstep<T>(wreg[a][ki], bq[ki][i], acc[a][i]);
#ifdef FASTLSTM_TIMELINE
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#endif
        FASTLSTM_TP(3);

        // ---- partial sums -> LDS, then every (tile, lane) item sums the 4 partials ---------
#pragma unroll
        for (int a = 0; a < MTW; ++a)
#pragma unroll
            for (int i = 0; i < NTW; ++i) red[(kq * TILES + (mh * MTW + a) * NT + i) * kWave + lane] = acc[a][i];
        tile_to_lds(gpre[u], gt);
        FASTLSTM_TP(4);
        __syncthreads();
        FASTLSTM_TP(5);

        const XchgL2 xw(p.xbuf + (size_t)((t + 1) & 1) * xslot, (unsigned)xslot);
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const int tile = wave + NWV * m;
            if (tile < TILES) {
                f32x4 s = red[tile * kWave + lane];
#pragma unroll
                for (int pp = 1; pp < 4; ++pp) s += red[(pp * TILES + tile) * kWave + lane];
                if (valid[m]) {
                    T *gl_ = reinterpret_cast<T *>(gt + goff[m]);   // the item's 4 gates in the LDS tile
                    const float pi = E::to_f32(gl_[0]) + s[0];
                    const float pf = E::to_f32(gl_[HT]) + s[1];
                    const float pg = E::to_f32(gl_[2 * HT]) + s[2];
                    const float po = E::to_f32(gl_[3 * HT]) + s[3];
                    const float c1 = sigmoidf_<ACC>(pf) * c_state[m] + sigmoidf_<ACC>(pi) * tanhf_<ACC>(pg);
                    const float h1 = sigmoidf_<ACC>(po) * tanhf_<ACC>(c1);
                    c_state[m] = c1;
                    const T hv = E::from_f32(h1);
                    xw.store_elem(xgrp + xoff[m], hv);
                    gl_[0] = E::from_f32(pi);
                    gl_[HT] = E::from_f32(pf);
                    gl_[2 * HT] = E::from_f32(pg);
                    gl_[3 * HT] = E::from_f32(po);
                    *reinterpret_cast<T *>(gt + BT * GROW + soff[m]) = hv;
                    *reinterpret_cast<T *>(gt + BT * GROW + BT * SROW + soff[m]) = E::from_f32(c1);
                }
            }
        }
        FASTLSTM_TP(6);
#ifdef FASTLSTM_TIMELINE
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        FASTLSTM_TP(7);
#endif
        if (t + 1 < T_) publish();
        else __syncthreads();   // last step: the tiles still have to be complete
        FASTLSTM_TP(8);
        tiles_to_global(t, gt);
        prefetch(t + PD, uc);
        FASTLSTM_TP(9);
    };
    for (int t0 = 0; t0 < T_; t0 += PD) {
        step(t0, std::integral_constant<int, 0>{});
        if constexpr (PD > 1)
            if (t0 + 1 < T_) step(t0 + 1, std::integral_constant<int, 1>{});
    }
    if (feeds) {   // the chunks that no step has counted: every workgroup counts its own part
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // in-loop: chunk c was counted at step (c + 1) * chunk_steps + 1 if that step exists
        const int chunks = (T_ + p.k1_chunk_steps - 1) / p.k1_chunk_steps;
        const int counted = T_ >= 2 ? (T_ - 2) / p.k1_chunk_steps : 0;   // chunks 0 .. counted-1 are done
        if (tid == kWave)
            for (int c = counted; c < chunks; ++c)
                __hip_atomic_fetch_add(p.out_ready + c, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#ifdef FASTLSTM_TIMELINE
    __syncthreads();
    if (p.trace)
        for (int idx = tid; idx < 256; idx += NTHR) p.trace[(size_t)blockIdx.x * 256 + idx] = tl[idx];
#endif
#undef FASTLSTM_TP
}

}  // namespace fastlstm

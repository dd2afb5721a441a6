// Persistent forward kernel: the whole time loop of one LSTM layer in one launch.
//
// Replaces persistent_fwd_kernel (fastlstm/kernels.py:414-663) and, for H <= 64,
// fully_fused_persistent_fwd_kernel's barrier-free single-tile form
// (fastlstm/kernels.py:672-819).  Per step t, for the workgroup's tile of
// bt batch rows x ht hidden units:
//     p      = ifgo[t] (holds x_t.Wx^T + b) + h_{t-1} . Wh_slice^T      fp32 accumulate
//     ifgo[t] <- p rounded to T (kept for the backward pass, kernels.py:631-640)
//     c      = sigmoid(p_f)*c + sigmoid(p_i)*tanh(p_g)                   c stays in fp32 registers
//     h      = sigmoid(p_o)*tanh(c);  cell[t+1] <- c, out[t+1] <- h      (kernels.py:647-657)
//
// MI355X mapping
//  * The workgroup's slice of W_h (4*ht rows x H) is copied ONCE into LDS, already in
//    MFMA operand order, and stays there for all T steps (the reference re-reads it from
//    L2 every step when H > 128, kernels.py:550-578).
//  * Rows of an M tile are ordered (unit, gate) so that the 4 accumulator registers of a
//    lane are exactly i,f,g,o of one (unit, batch row): the gate maths needs no shuffles.
//  * h_t travels between workgroups through a small double-buffered exchange buffer that
//    is laid out in MFMA operand order too: a consumer wave fetches a whole 16 x KSTEP
//    operand block with one fully coalesced 1 KiB load, straight into registers.
//  * The 4 waves split K (small batch tiles), the batch tiles (large ones) or the W rows
//    (barrier-free small-H form); partial sums meet in LDS.
#pragma once
#include <type_traits>

#include "recurrent_common.hpp"

namespace fastlstm {

struct FwdParams {
    void *ifgo;        // [T,B,4H]
    void *out;         // [T+1,B,H]
    void *cell;        // [T+1,B,H]
    const void *Wh;    // [4H,H]
    WsHeader *hdr;
    int *flags;        // [n_bt][flag_stride]
    unsigned char *xbuf;  // [2 slots][n_bt][NT][KS] operand blocks
    int T, B, H;
    int b_base;        // first batch row covered by this launch
    int n_bt, n_ht, flag_stride;
    int KS;            // k-steps covering H
    int vec_io;        // 1: move the ifgo / out / cell tiles through LDS with 16-byte accesses
    int w_regs;        // > 0: k-steps per wave of the W_h slice held in registers (NKW instantiation)
    int keep;          // 1: store the gate pre-activations and every cell state (what the reverse pass reads);
                       // 0: inference, ifgo stays the input projection and only cell[T] is written
    long long spin_limit;
    long long *trace;  // optional diagnostics: 4 accumulated phase times per workgroup, else nullptr
    // SPLIT 2 only (no exchange between workgroups): n_rec > 1 independent recurrences of this shape share the launch,
    // recurrence r on the workgroups r * n_bt_launch ...; operands of recurrences 1 ... in the arrays
    int n_rec, n_bt_launch;
    int rs;            // 2, 4: batch tiles of 16 / rs rows (RS instantiation; b_base and n_bt_launch count in those), else 0
    void *ifgo_x[3], *out_x[3], *cell_x[3];
    const void *Wh_x[3];
};

// SPLIT 0: waves split K   (MT m-tiles, NTW n-tiles per WG, 4 partial sums)
// SPLIT 1: waves split N   (MT m-tiles per WG, NTW n-tiles per wave, 4*NTW per WG)
// SPLIT 2: waves split M   (MT m-tiles per wave, 4*MT per WG, one n-tile; no cross-WG sync)
// NKW > 0 (SPLIT 0 only): every wave keeps its share of the W_h slice -- MT x NKW operand
// fragments, k-steps wave, wave+4, ... -- in registers instead of re-reading it from LDS every
// timestep (the LDS reads of a 128 KiB slice alone take ~0.4 us per step).  Needs KS <= 4*NKW.
// SPLIT 2 with tile I/O runs CW computing waves and four more that only move the tiles between global
// memory and LDS (the gates of the step after next in, the results of the last step out).  In one wave the
// two jobs queue behind each other in a step that is one chain of dependent latencies; side by side they
// overlap (H = 64, B = 256, fp16: 1.00 -> 0.78 us per step; the reverse kernel 1.10 -> 0.98).
// CW (that form only): the number of computing waves, 4 or 8, each with MT of the workgroup's CW * MT row tiles;
// the four tile-moving waves come behind them.  Eight waves of 2 cells per lane instead of four waves of 4 shorten
// the step of 64 units by 11 % (two waves per SIMD overlap each other's LDS and MFMA latencies; it showed only
// once the tile-moving waves had stopped being the bound, see their loop below).
template <int SPLIT, bool VIO, int CW = 4> constexpr int fwd_threads() {
    return (SPLIT == 2 && VIO) ? (CW + 4) * kWave : kThreads;
}

// RS = 2 (8 computing waves of 2 row tiles) or 4 (4 computing waves of 4 row tiles), 64 units: a workgroup takes
// 16 / RS batch rows, i.e. the batch spreads over RS times the CUs.  The MFMAs still produce 16 columns (the operand
// rows that do not exist are zeros); the RS accumulator tiles of a lane are folded into one -- the lanes of the
// columns that do not exist take the columns 0 .. 16 / RS - 1 of the lane's other tiles through DPP rotations
// within the row of 16 lanes -- so that every lane computes ONE cell per step instead of two or four.  The step of
// the 16-row kernel is bound by the vector ALU, not by a latency: per wave and step 20 exp / rcp at a quarter of the
// rate and 70 other instructions for two cells, two such waves per SIMD, is 1200 of the step's 1170 cycles
// (T = 1024, B = 256, fp16: 0.556 us per step with 16 rows, 0.401 with 8, 0.339 with 4).
template <typename T, int MT, int NTW, int SPLIT, bool VIO, int NKW = 0, int CW = 4, int RS = 1>
__global__ __launch_bounds__((fwd_threads<SPLIT, VIO, CW>())) void lstm_fwd_persistent_kernel(const FwdParams p) {
    using E = Elem<T>;
    constexpr bool SYNC = SPLIT != 2;
    constexpr bool IOW = SPLIT == 2 && VIO;   // tile-moving waves CW..CW+3 behind the computing waves 0..CW-1
    static_assert(CW == 4 || (IOW && CW == 8), "8 computing waves: the one-tile form with tile I/O");
    constexpr int CT = CW * kWave;            // threads of the computing waves
    constexpr bool ACC = (E::DT == FASTLSTM_FP32);
    constexpr int MTT = SPLIT == 2 ? CW * MT : MT;    // m-tiles per workgroup
    constexpr int NT = SPLIT == 1 ? 4 * NTW : NTW;   // n-tiles per workgroup
    constexpr int P = SPLIT == 0 ? 4 : 1;            // partial sums per output tile
    constexpr int TILES = MTT * NT;
    static_assert(RS == 1 || (IOW && NTW == 1 && ((RS == 2 && CW == 8 && MT == 2) || (RS == 4 && CW == 4 && MT == 4))),
                  "batch tiles of 16 / RS rows: RS row tiles per wave, folded into one cell per lane");
    constexpr int IPT = RS > 1 ? 1 : (TILES + CW - 1) / CW;   // (tile, lane) items per thread
    constexpr int HT = 4 * MTT, BT = 16 * NT / RS;
    constexpr int CH = 8 / NTW;                      // k-steps fetched per batch of loads
    constexpr bool WREG = NKW > 0;
    static_assert(!WREG || SPLIT == 0, "register-resident weights: K-split kernels only");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const bool cw = !IOW || tid < CT;                    // a computing wave
    const int wave = IOW ? (tid >> 6) & (CW - 1) : tid >> 6;   // (a tile-moving wave mirrors the set-up of a computing wave and never uses it)
    const int q = lane >> 4, n = lane & 15;
    const int KS = p.KS, H = p.H, B = p.B, T_ = p.T;
    const bool keep = p.keep != 0;   // training: gate pre-activations and every cell state are stored

    int g, j;
    if constexpr (SYNC) {
        const int lin = xcd_major_id(blockIdx.x, gridDim.x);
        g = lin / p.n_ht;
        j = lin % p.n_ht;
    } else {
        g = blockIdx.x;
        j = 0;
    }
    int rec = 0;   // which recurrence of the launch
    if constexpr (!SYNC) {
        if (p.n_rec > 1) {
            rec = blockIdx.x / p.n_bt_launch;
            g = blockIdx.x - rec * p.n_bt_launch;
        }
    }
    // (constant indices only: a run-time index into the kernel's arguments would move them all to scratch memory)
    auto pick = [&](auto a0, auto a1, auto a2, auto a3) {
        if constexpr (SYNC) return a0;
        else return rec == 0 ? a0 : rec == 1 ? a1 : rec == 2 ? a2 : a3;
    };
    const int u0 = j * HT;                  // first hidden unit of this workgroup
    const int b0 = p.b_base + g * BT;       // first batch row

    unsigned char *Wl = smem;                                  // [MTT][KS] blocks + one all-zero block
    const unsigned zero_off = (unsigned)MTT * KS * kFragBytes;
    f32x4 *red = reinterpret_cast<f32x4 *>(smem + zero_off + kFragBytes);  // [P][TILES][64]
    unsigned char *xl = reinterpret_cast<unsigned char *>(red + P * TILES * kWave);  // SPLIT 2: [2][KS] blocks

    // Coalesced tile I/O: the workgroup's tile of ifgo[t] (bt rows x 4 gates x ht units) and of
    // out / cell (bt x ht) lies in global memory as row segments of ht elements.  Moving them
    // element by element costs one scattered 2-byte access per gate and item; instead the tile
    // is moved with 16-byte pieces between global memory and padded LDS tiles, and the items
    // work on LDS.  Needs 16-byte aligned, complete segments (host decides: p.vec_io).
    constexpr int GSEG = HT * E::BYTES;                 // bytes of one gate segment of a row
    constexpr bool VEC_OK = GSEG >= 16;
    constexpr int GROW = 4 * GSEG + 16, SROW = GSEG + 16;   // padded LDS rows (bank spread)
    constexpr int PPSEG = VEC_OK ? GSEG / 16 : 1;       // 16-byte pieces per segment
    constexpr int GPIECES = BT * 4 * PPSEG, SPIECES = BT * PPSEG;
    // wave 0 polls the flags and must not queue its polls behind bulk loads/stores of its own:
    // the tiles are moved by waves 1..3 only
    // (one hidden tile per workgroup: by the four waves that do nothing else)
    constexpr int IOT = IOW ? kThreads : kThreads - kWave;
    constexpr int GPT = (GPIECES + IOT - 1) / IOT, SPT = (SPIECES + IOT - 1) / IOT;
    const int io_tid = IOW ? tid - CT : tid - kWave;   // < 0: not an I/O thread
    constexpr int TILE_BYTES = BT * GROW + 2 * BT * SROW;   // gates tile + h tile + c tile
    static_assert(!VIO || VEC_OK, "tile I/O needs 16-byte gate segments");
    unsigned char *tiles = xl + (SYNC ? 0 : 2 * (size_t)KS * kFragBytes);  // SYNC: 1 set, else 2 (step parity)

    // Diagnostic build (-DFASTLSTM_TIMELINE): lane 0 of every wave stamps the 100 MHz clock at fixed
    // points of timesteps 200..203 into LDS; the stamps go to p.trace (256 words per workgroup:
    // [step][wave][16 events]) when the kernel ends.  The host adds 4 KiB of LDS for it.
#ifdef FASTLSTM_TIMELINE
    long long *tl = reinterpret_cast<long long *>(tiles + (SYNC ? 1 : 2) * TILE_BYTES + 64);
    for (int idx = tid; idx < 256; idx += kThreads) tl[idx] = 0;
    __syncthreads();
    if (tid == 0) {   // event 15 of (step 200, wave 0): the XCD this workgroup runs on
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        tl[15] = (long long)(xcc & 15u);
    }
#define FASTLSTM_TP(ev)                                                                              \
    do {                                                                                             \
        if (lane == 0 && t >= 200 && t < 204) tl[((t - 200) * 4 + wave) * 16 + (ev)] = (long long)wall_clock64(); \
    } while (0)
#else
#define FASTLSTM_TP(ev) do {} while (0)
#endif
    T *ifgo = static_cast<T *>(pick(p.ifgo, p.ifgo_x[0], p.ifgo_x[1], p.ifgo_x[2]));
    T *out = static_cast<T *>(pick(p.out, p.out_x[0], p.out_x[1], p.out_x[2]));
    T *cell = static_cast<T *>(pick(p.cell, p.cell_x[0], p.cell_x[1], p.cell_x[2]));
    const T *Wh = static_cast<const T *>(pick(p.Wh, p.Wh_x[0], p.Wh_x[1], p.Wh_x[2]));

    // ---- prologue 1: W_h slice -> LDS in operand order (zero padded) ----------------
    {
        const int chunks_per_row = KS * 4;  // 16-byte chunks along K
        const int total = MTT * 16 * chunks_per_row;
        const bool vec = (H % E::EPL) == 0;
        for (int idx = tid; cw && idx < total; idx += CT) {
            const int row = idx / chunks_per_row, kc = idx % chunks_per_row;
            const int mt = row >> 4, r = row & 15;
            // row r of an m-tile is gate r % 4 of the tile's unit r / 4.  One hidden tile per workgroup:
            // the MT tiles of a wave interleave, so that a lane's MT results are MT consecutive units
            const int unit = u0 + (SPLIT == 2 ? (mt / MT) * 4 * MT + (r >> 2) * MT + mt % MT : mt * 4 + (r >> 2));
            const int gate = r & 3;
            const int k0 = kc * E::EPL;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (unit < H && k0 < H) {
                const T *src = Wh + ((size_t)gate * H + unit) * H + k0;
                if (vec) {
                    v = *reinterpret_cast<const u32x4 *>(src);
                } else {
                    T tmp[E::EPL];
#pragma unroll
                    for (int e = 0; e < E::EPL; ++e) tmp[e] = (k0 + e < H) ? src[e] : E::from_f32(0.f);
                    v = *reinterpret_cast<u32x4 *>(tmp);
                }
            }
            const int ks = kc >> 2, qq = kc & 3;
            *reinterpret_cast<u32x4 *>(Wl + ((size_t)(mt * KS + ks) * kWave + qq * 16 + r) * 16) = v;
        }
        if (tid < kWave) reinterpret_cast<u32x4 *>(Wl + zero_off)[tid] = u32x4{0u, 0u, 0u, 0u};
        if constexpr (!SYNC) {
            for (int idx = tid; cw && idx < 2 * KS * kWave; idx += CT)
                reinterpret_cast<u32x4 *>(xl)[idx] = u32x4{0u, 0u, 0u, 0u};
        }
    }
    __syncthreads();
    u32x4 wreg[WREG ? MT : 1][WREG ? NKW : 1];   // this wave's fragments of the slice (zero past KS)
    if constexpr (WREG) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int ki = 0; ki < NKW; ++ki) {
                const int ks = wave + 4 * ki;
                const unsigned woff = ks < KS ? (unsigned)((a * KS + ks) * kWave + lane) * 16u : zero_off + lane * 16u;
                wreg[a][ki] = *reinterpret_cast<const u32x4 *>(Wl + woff);
            }
    }

    // One hidden tile per workgroup (SPLIT == 2, H <= 64): the wave's MT row tiles x all k-steps are
    // few enough to stay in registers too (the LDS copy was a chain of dependent round trips per step).
    constexpr int KS2 = 64 / E::KSTEP;   // k-steps that cover H = 64
    u32x4 w2[SPLIT == 2 ? MT : 1][SPLIT == 2 ? KS2 : 1];
    if constexpr (SPLIT == 2) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) {
                const unsigned woff = ks < KS ? (unsigned)(((wave * MT + a) * KS + ks) * kWave + lane) * 16u
                                              : zero_off + lane * 16u;
                w2[a][ks] = *reinterpret_cast<const u32x4 *>(Wl + woff);
            }
    }

    // ---- per-thread items: (tile = wave + 4m, lane) -> (unit, batch row) -------------
    float c_state[IPT];
    size_t off_h[IPT];    // b*H + unit
    size_t off_p[IPT];    // b*4H + unit
    int xoff[IPT];        // byte offset of (unit, row) inside one exchange slot of this group
    int goff[IPT], soff[IPT];  // byte offsets of the item inside the LDS gates / state tiles
    bool valid[IPT];
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        // SPLIT 2: the item is the lane's own accumulator of the wave's m-tile m (see the weight rows above)
        const int tl = SPLIT == 2 ? wave * MT + m : wave + 4 * m;
        const int mt = tl / NT, nt = tl % NT;
        // (RS 2, 4: the lane's one item is row n % (16 / RS) of the wave's row tile n / (16 / RS))
        const int ul = RS > 1 ? wave * 4 * MT + q * MT + n / (16 / RS)
                              : SPLIT == 2 ? wave * 4 * MT + q * MT + m : mt * 4 + q;   // unit inside the hidden tile
        const int row = RS > 1 ? n % (16 / RS) : nt * 16 + n;
        const int unit = u0 + ul, b = b0 + row;
        valid[m] = (tl < TILES) && unit < H && b < B;
        // invalid items point at the tile's first element: their loads stay in bounds, nothing is stored
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        off_p[m] = valid[m] ? (size_t)b * 4 * H + unit : (size_t)b0 * 4 * H + u0;
        xoff[m] = RS > 1 ? frag_offset<T>(row, unit) : nt * KS * kFragBytes + frag_offset<T>(n, unit);
        goff[m] = row * GROW + ul * E::BYTES;
        soff[m] = row * SROW + ul * E::BYTES;
        c_state[m] = valid[m] ? E::to_f32(cell[off_h[m]]) : 0.f;
    }

    // exchange buffer: [2 slots][batch tile][NT][KS] operand blocks (global) or [2][KS] (LDS)
    using Xchg = typename std::conditional<SYNC, XchgGlobal, XchgLds>::type;
    const unsigned xslot = SYNC ? (unsigned)p.n_bt * NT * KS * kFragBytes : (unsigned)KS * kFragBytes;
    const unsigned xgrp = SYNC ? (unsigned)g * NT * KS * kFragBytes : 0u;
    constexpr int n_slots = 2;   // h_v lives in slot v % 2; the loads are device-scope (the address is reused)
    const Xchg xch(SYNC ? p.xbuf : xl, (unsigned)n_slots * xslot);
    int *my_flag = SYNC ? p.flags + (size_t)g * p.flag_stride + j : nullptr;
    const int *grp_flags = SYNC ? p.flags + (size_t)g * p.flag_stride : nullptr;

    // ---- prologue 2: publish h_0 (version 1) ------------------------------------------
#pragma unroll
    for (int m = 0; m < IPT; ++m)
        if (cw && valid[m]) xch.store_elem(xgrp + xoff[m], out[off_h[m]]);
    if constexpr (SYNC) publish_version(my_flag, 1);
    else __syncthreads();

    const size_t BH = (size_t)B * H, B4H = (size_t)B * 4 * H;

    // x_t.Wx^T + b does not depend on the recurrence: it is requested PD steps ahead (an HBM round
    // trip is ~2 us).  The loads are unconditional -- invalid items / pieces read a valid dummy
    // address -- so that their results stay in the registers they were loaded into: a
    // conditional load ends in a register copy, and the copy in a wait for the load.
    constexpr int PD = SYNC ? 2 : 4;
    constexpr int PRE_N = VIO ? 1 : PD, GPRE_N = VIO ? PD : 1;
    T pre[PRE_N][IPT][4];
    auto fetch_pre = [&](int t, T(&dst)[IPT][4]) {
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const T *src = ifgo + (size_t)t * B4H + off_p[m];
#pragma unroll
            for (int gt = 0; gt < 4; ++gt) dst[m][gt] = src[(size_t)gt * H];
        }
    };
    u32x4 gpre[GPRE_N][GPT];  // VIO: 16-byte pieces of the gates tile, in flight
    const size_t tile_org = (size_t)b0 * 4 * H + u0;   // first element of the tile inside ifgo[t]
    auto fetch_tile = [&](int t, u32x4(&dst)[GPT]) {
        if (io_tid < 0) return;
#pragma unroll
        for (int i = 0; i < GPT; ++i) {
            const int pc = io_tid + IOT * i;
            const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG);
            const int seg = rem / PPSEG, k = rem % PPSEG;
            const bool ok = pc < GPIECES && b0 + row < B;
            const size_t off = ok ? (size_t)row * 4 * H + (size_t)seg * H + k * (16 / E::BYTES) : 0;
            dst[i] = *reinterpret_cast<const u32x4 *>(ifgo + (size_t)t * B4H + tile_org + off);
        }
    };
    auto tile_to_lds = [&](const u32x4(&src)[GPT], unsigned char *gt) {
#pragma unroll
        for (int i = 0; i < GPT; ++i) {
            const int pc = io_tid + IOT * i;
            const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG);
            if (io_tid >= 0 && pc < GPIECES)
                *reinterpret_cast<u32x4 *>(gt + row * GROW + (rem / PPSEG) * GSEG + (rem % PPSEG) * 16) = src[i];
        }
    };
    // LDS tiles -> ifgo[t], out[t+1], cell[t+1] with 16-byte row-contiguous stores
    auto tiles_to_global = [&](int t, const unsigned char *gt) {
        const unsigned char *sth = gt + BT * GROW, *stc = sth + BT * SROW;
#pragma unroll
        for (int i = 0; i < GPT; ++i) {
            const int pc = io_tid + IOT * i;
            const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG);
            const int seg = rem / PPSEG, k = rem % PPSEG;
            if (keep && io_tid >= 0 && pc < GPIECES && b0 + row < B)
                *reinterpret_cast<u32x4 *>(ifgo + ((size_t)t * B + b0 + row) * 4 * H + (size_t)seg * H + u0 +
                                           k * (16 / E::BYTES)) =
                    *reinterpret_cast<const u32x4 *>(gt + row * GROW + seg * GSEG + k * 16);
        }
#pragma unroll
        for (int i = 0; i < SPT; ++i) {
            const int pc = io_tid + IOT * i;
            const int row = pc / PPSEG, k = pc % PPSEG;
            if (io_tid >= 0 && pc < SPIECES && b0 + row < B) {
                const size_t go = ((size_t)(t + 1) * B + b0 + row) * H + u0 + k * (16 / E::BYTES);
                *reinterpret_cast<u32x4 *>(out + go) = *reinterpret_cast<const u32x4 *>(sth + row * SROW + k * 16);
                if (keep || t + 1 == T_)
                    *reinterpret_cast<u32x4 *>(cell + go) = *reinterpret_cast<const u32x4 *>(stc + row * SROW + k * 16);
            }
        }
    };
    auto prefetch = [&](int t, auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        if constexpr (IOW) return;   // (the tile-moving waves have a loop of their own, below)
        if (t < T_) {
            if constexpr (VIO) fetch_tile(t, gpre[u]);
            else fetch_pre(t, pre[u]);
        }
    };
    // ---- the tile-moving waves of the one-tile form: their own time loop --------------------------------
    // Every vector-memory instruction of this loop is unconditional -- a piece that does not exist, a row past
    // the batch, a timestep past the end, a store that is not wanted get an offset outside the buffer
    // descriptor (loads return zeros, stores are dropped) -- and four steps are unrolled without a branch
    // between them.  The compiler can then count: its s_waitcnt vmcnt(N) in front of "tile t + 1 into LDS"
    // names exactly the loads of that tile and leaves the 12 younger operations -- the stores of the last two
    // steps, the tiles of steps t + 2 and t + 3 -- in flight.  With conditional stores and loads in between
    // (and the roles of the waves decided by a branch around them) it could only wait for everything: every
    // step then paid the round trip of the loads it had just requested four steps ahead, and of its stores
    // (T = 1024, B = 256, H = 64: 0.78 -> 0.63 us per step).
    if constexpr (IOW) {
        if (!cw) {
            constexpr unsigned kOut = 0xfffffff0u;
            constexpr int EPC = 16 / E::BYTES;
            const u32x4 zero = {0u, 0u, 0u, 0u};
            unsigned gv[GPT], gvs[GPT], sv[SPT];   // byte offsets inside ifgo[t] (loads / stores) and out[t]; kOut: none
            int gl[GPT], sl[SPT];                  // byte offsets inside the LDS tiles; -1: no such piece
#pragma unroll
            for (int i = 0; i < GPT; ++i) {
                const int pc = io_tid + IOT * i;
                const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG), seg = rem / PPSEG, k = rem % PPSEG;
                const bool ok = pc < GPIECES && b0 + row < B;
                gv[i] = ok ? (unsigned)((((size_t)(b0 + row) * 4 + seg) * H + u0 + k * EPC) * E::BYTES) : kOut;
                gvs[i] = keep ? gv[i] : kOut;
                gl[i] = ok ? row * GROW + seg * GSEG + k * 16 : -1;
            }
#pragma unroll
            for (int i = 0; i < SPT; ++i) {
                const int pc = io_tid + IOT * i;
                const int row = pc / PPSEG, k = pc % PPSEG;
                const bool ok = pc < SPIECES && b0 + row < B;
                sv[i] = ok ? (unsigned)(((size_t)(b0 + row) * H + u0 + k * EPC) * E::BYTES) : kOut;
                sl[i] = ok ? row * SROW + k * 16 : -1;
            }
            const unsigned g_bytes = (unsigned)(B4H * E::BYTES), s_bytes = (unsigned)(BH * E::BYTES);
            auto rsrc_g = [&](int t) {   // ifgo[t]; past the last timestep: an empty buffer
                return __builtin_amdgcn_make_buffer_rsrc(ifgo + (size_t)min(t, T_ - 1) * B4H, 0, t < T_ ? g_bytes : 0u, 0x00020000);
            };
            u32x4 ring[PD][GPT];
            auto load_tile = [&](int t, auto uc) __attribute__((always_inline)) {
                constexpr int u = decltype(uc)::value;
                const __amdgpu_buffer_rsrc_t rg = rsrc_g(t);
#pragma unroll
                for (int i = 0; i < GPT; ++i) ring[u][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rg, gv[i], 0, 0));
            };
            auto dropped_stores = [&](unsigned group) __attribute__((always_inline)) {   // as many as a step issues
                const __amdgpu_buffer_rsrc_t rg = rsrc_g(0);   // (each at an offset of its own, or the compiler keeps one of them)
#pragma unroll
                for (int i = 0; i < GPT + 2 * SPT; ++i)
                    __builtin_amdgcn_raw_buffer_store_b128(zero, rg, kOut - 16u * (group * (GPT + 2 * SPT) + i), 0, 0);
            };
            auto to_lds = [&](auto uc, unsigned char *gt) __attribute__((always_inline)) {
                constexpr int u = decltype(uc)::value;
#pragma unroll
                for (int i = 0; i < GPT; ++i)
                    if (gl[i] >= 0) *reinterpret_cast<u32x4 *>(gt + gl[i]) = ring[u][i];
            };
            auto to_global = [&](int t, const unsigned char *gt) __attribute__((always_inline)) {
                const unsigned char *sth = gt + BT * GROW, *stc = sth + BT * SROW;
                const __amdgpu_buffer_rsrc_t rg = rsrc_g(t);
                const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(out + (size_t)(t + 1) * BH, 0, s_bytes, 0x00020000);
                const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(cell + (size_t)(t + 1) * BH, 0, s_bytes, 0x00020000);
                const bool cell_wanted = keep || t + 1 == T_;
#pragma unroll
                for (int i = 0; i < GPT; ++i)
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(gt + max(gl[i], 0)), rg, gvs[i], 0, 0);
#pragma unroll
                for (int i = 0; i < SPT; ++i) {
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(sth + max(sl[i], 0)), rh, sv[i], 0, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(stc + max(sl[i], 0)), rc,
                                                           cell_wanted ? sv[i] : kOut, 0, 0);
                }
            };
            // step t: tile t + 1 (ring entry (u + 1) % PD) into the other tile set before the barrier, this step's
            // results out of this one behind it, tile t + PD requested into the entry that tile t left
            auto io_step = [&](int t, auto uc) __attribute__((always_inline)) {
                constexpr int u = decltype(uc)::value;
                to_lds(std::integral_constant<int, (u + 1) % PD>{}, tiles + ((t + 1) & 1) * TILE_BYTES);
                __syncthreads();
                to_global(t, tiles + (t & 1) * TILE_BYTES);
                load_tile(t + PD, uc);
            };
            // (the loop is entered with what every later pass finds in flight: between the tiles, as many stores as a step issues)
            static_for<0, PD>([&](auto uc) __attribute__((always_inline)) {
                load_tile(decltype(uc)::value, uc);
                if constexpr (decltype(uc)::value + 1 < PD) dropped_stores(decltype(uc)::value);
            });
            to_lds(std::integral_constant<int, 0>{}, tiles);
            __syncthreads();
            int t0 = 0;
            for (; t0 + PD <= T_; t0 += PD)
                static_for<0, PD>([&](auto uc) __attribute__((always_inline)) { io_step(t0 + decltype(uc)::value, uc); });
            static_for<0, PD - 1>([&](auto uc) __attribute__((always_inline)) {
                if (t0 + decltype(uc)::value < T_) io_step(t0 + decltype(uc)::value, uc);
            });
            return;
        }
    }
    prefetch(0, std::integral_constant<int, 0>{});
    prefetch(1, std::integral_constant<int, 1>{});
    if constexpr (PD > 2) {
        prefetch(2, std::integral_constant<int, 2>{});
        prefetch(3, std::integral_constant<int, 3>{});
    }

    int slot_r = 0;  // ring slot that holds h_{t-1}
    if constexpr (IOW) __syncthreads();   // the gates tile of step 0 is in LDS (every later one is moved a step ahead)
    // One timestep; u = t % PD selects the prefetch ring entry at compile time.
    auto step = [&](const int t, auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        const int slot_w = (slot_r + 1 == n_slots) ? 0 : slot_r + 1;
        unsigned char *gt = tiles + (SYNC ? 0 : (t & 1) * TILE_BYTES);
        if constexpr (SPLIT == 2) {
            // One hidden tile per workgroup.  A lane's accumulators ARE its items: accumulator m holds the
            // four gates of unit (first unit of the lane) + m for batch row n, so nothing is reduced and
            // nothing but h_t crosses waves; the lane moves its MT consecutive units of every tile row
            // with one LDS access.  One workgroup barrier per step: behind it h_t (operand blocks), this
            // step's result tiles and the next step's gates tile are all in LDS.
            constexpr int NI = RS > 1 ? 1 : MT;   // cells per lane
            using V = typename VecBytes<NI * E::BYTES>::type;
            const unsigned xb = (unsigned)slot_r * xslot, xn = (unsigned)slot_w * xslot;
            if (cw) {
            f32x4 acc[MT];
            V xv[4];
            {
                u32x4 bq[KS2];
#pragma unroll
                for (int ks = 0; ks < KS2; ++ks)   // past the end: any valid block (its weights are zero)
                    bq[ks] = xch.template load16<false>(xb + (unsigned)(min(ks, KS - 1) * kWave + lane) * 16u);
                if constexpr (VIO) {   // the lane's gates of this step: requested with the operand blocks
#pragma unroll
                    for (int gg = 0; gg < 4; ++gg) xv[gg] = *reinterpret_cast<const V *>(gt + goff[0] + gg * GSEG);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int a = 0; a < MT; ++a) acc[a] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
                    for (int a = 0; a < MT; ++a) acc[a] = mfma_kstep<T>(w2[a][ks], bq[ks], acc[a]);
            }
            if constexpr (RS == 2) {
                // lanes 8..15 of every row of 16: columns 0..7 of the second tile (row_ror:8 into banks 2 and 3)
                // (element by element on scalars: written as a loop over the vectors' elements, the compiler emitted
                // the first element's move four times)
                const float lo0 = acc[0][0], lo1 = acc[0][1], lo2 = acc[0][2], lo3 = acc[0][3];
                const float hi0 = acc[1][0], hi1 = acc[1][1], hi2 = acc[1][2], hi3 = acc[1][3];
                acc[0] = f32x4{fold_upper_half(lo0, hi0), fold_upper_half(lo1, hi1), fold_upper_half(lo2, hi2), fold_upper_half(lo3, hi3)};
            }
            if constexpr (RS == 4) {   // lanes 4j .. 4j + 3: columns 0..3 of the wave's tile j
                float f[4][4];
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    f[a][0] = acc[a][0]; f[a][1] = acc[a][1]; f[a][2] = acc[a][2]; f[a][3] = acc[a][3];
                }
                acc[0] = f32x4{fold_quarters(f[0][0], f[1][0], f[2][0], f[3][0]), fold_quarters(f[0][1], f[1][1], f[2][1], f[3][1]),
                               fold_quarters(f[0][2], f[1][2], f[2][2], f[3][2]), fold_quarters(f[0][3], f[1][3], f[2][3], f[3][3])};
            }
            T x4[4][NI], st_p[IPT][4], st_h[IPT], st_c[IPT];
#pragma unroll
            for (int gg = 0; gg < 4; ++gg) {
                if constexpr (VIO) {
                    __builtin_memcpy(x4[gg], &xv[gg], sizeof(V));
                } else {
#pragma unroll
                    for (int m = 0; m < NI; ++m) x4[gg][m] = pre[u][m][gg];
                }
            }
#pragma unroll
            for (int m = 0; m < NI; ++m) {
                const float pi = E::to_f32(x4[0][m]) + acc[m][0];
                const float pf = E::to_f32(x4[1][m]) + acc[m][1];
                const float pg = E::to_f32(x4[2][m]) + acc[m][2];
                const float po = E::to_f32(x4[3][m]) + acc[m][3];
                const float c1 = sigmoidf_<ACC>(pf) * c_state[m] + sigmoidf_<ACC>(pi) * tanhf_<ACC>(pg);
                const float h1 = sigmoidf_<ACC>(po) * tanhf_<ACC>(c1);
                c_state[m] = c1;
                // units past H and rows past B stay zero in the operand blocks (their weights are zero,
                // but 0 x NaN is not)
                st_h[m] = E::from_f32(valid[m] ? h1 : 0.f);
                st_p[m][0] = E::from_f32(pi);
                st_p[m][1] = E::from_f32(pf);
                st_p[m][2] = E::from_f32(pg);
                st_p[m][3] = E::from_f32(po);
                st_c[m] = E::from_f32(c1);
            }
            V vh, vc;
            __builtin_memcpy(&vh, st_h, sizeof(V));
            __builtin_memcpy(&vc, st_c, sizeof(V));
            *reinterpret_cast<V *>(xl + xn + xoff[0]) = vh;
            if constexpr (VIO) {
#pragma unroll
                for (int gg = 0; gg < 4; ++gg) {
                    T pk[NI];
#pragma unroll
                    for (int m = 0; m < NI; ++m) pk[m] = st_p[m][gg];
                    V vp;
                    __builtin_memcpy(&vp, pk, sizeof(V));
                    *reinterpret_cast<V *>(gt + goff[0] + gg * GSEG) = vp;
                }
                *reinterpret_cast<V *>(gt + BT * GROW + soff[0]) = vh;
                *reinterpret_cast<V *>(gt + BT * GROW + BT * SROW + soff[0]) = vc;
            } else {
#pragma unroll
                for (int m = 0; m < NI; ++m) {
                    if (valid[m]) {
                        if (keep) {
                            T *dst = ifgo + (size_t)t * B4H + off_p[m];
                            dst[0] = st_p[m][0];
                            dst[(size_t)H] = st_p[m][1];
                            dst[(size_t)2 * H] = st_p[m][2];
                            dst[(size_t)3 * H] = st_p[m][3];
                        }
                        out[(size_t)(t + 1) * BH + off_h[m]] = st_h[m];
                        if (keep || t + 1 == T_) cell[(size_t)(t + 1) * BH + off_h[m]] = st_c[m];
                    }
                }
            }
            }   // computing waves
            // tile-moving waves (with tile I/O; without it nobody): the next step's gates into the other
            // tile set before the barrier, this step's results out of this one behind it
            __syncthreads();   // (with tile I/O: the tile-moving waves meet it in their own loop)
            prefetch(t + PD, uc);
            slot_r = slot_w;
            return;
        }
        long long tr0 = 0, tr1 = 0, tr2 = 0, tr3 = 0;
        if (p.trace) tr0 = (long long)wall_clock64();
        FASTLSTM_TP(0);
        if constexpr (SYNC) {
            if (wave == 0) wait_versions(grp_flags, p.n_ht, t + 1, p.hdr, p.spin_limit, g, t);
            FASTLSTM_TP(1);
            __syncthreads();
        }
        FASTLSTM_TP(2);
        if (p.trace) tr1 = (long long)wall_clock64();

        // ---- acc[mt][i] += Wslice(mt) . h_{t-1}(nt)^T over this wave's k-steps ----------
        const unsigned xb = xgrp + (unsigned)slot_r * xslot;
        f32x4 acc[MT][NTW];
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int i = 0; i < NTW; ++i) acc[a][i] = f32x4{0.f, 0.f, 0.f, 0.f};

        const int kfirst = SPLIT == 0 ? wave : 0, kstride = SPLIT == 0 ? 4 : 1;
        const int nk = SPLIT == 0 ? (KS - wave + 3) / 4 : KS;  // k-steps of this wave
        const int nt_base = SPLIT == 1 ? wave * NTW : 0;
        const int mt_base = SPLIT == 2 ? wave * MT : 0;

        // Straight-line chunks of CH k-steps: the operand loads of a chunk are issued back to
        // back (one round trip for all of them) and there is not a single branch inside: a k-step
        // past the end of this wave's share re-reads the last valid block and multiplies it with
        // the all-zero weight block instead.
        auto kloop = [&](auto coh) {
            constexpr bool COH = decltype(coh)::value;
            auto load_b = [&](u32x4(&bq)[CH][NTW], int ki0) {
#pragma unroll
                for (int cc = 0; cc < CH; ++cc) {
                    const int ki = min(ki0 + cc, nk - 1);
                    const int ks = kfirst + ki * kstride;
#pragma unroll
                    for (int i = 0; i < NTW; ++i)
                        bq[cc][i] = xch.template load16<COH>(
                            xb + (unsigned)(((nt_base + i) * KS + ks) * kWave + lane) * 16u);
                }
            };
            auto compute = [&](const u32x4(&bq)[CH][NTW], int ki0) {
#pragma unroll
                for (int cc = 0; cc < CH; ++cc) {
                    const int ki = ki0 + cc;
                    const int ks = kfirst + ki * kstride;
#pragma unroll
                    for (int a = 0; a < MT; ++a) {
                        const unsigned woff = ki < nk ? (unsigned)(((mt_base + a) * KS + ks) * kWave + lane) * 16u
                                                      : zero_off + lane * 16u;
                        const u32x4 af = *reinterpret_cast<const u32x4 *>(Wl + woff);
#pragma unroll
                        for (int i = 0; i < NTW; ++i) acc[a][i] = mfma_kstep<T>(af, bq[cc][i], acc[a][i]);
                    }
                }
            };
            u32x4 bqA[CH][NTW], bqB[CH][NTW];
            const int nchunks = (nk + CH - 1) / CH;
            if (nchunks > 0) load_b(bqA, 0);
            for (int ci = 0; ci < nchunks; ci += 2) {
                if (ci + 1 < nchunks) load_b(bqB, (ci + 1) * CH);
                compute(bqA, ci * CH);
                if (ci + 1 < nchunks) {
                    if (ci + 2 < nchunks) load_b(bqA, (ci + 2) * CH);
                    compute(bqB, (ci + 1) * CH);
                }
            }
        };
        // register-resident weights: all NKW operand blocks of this wave are requested at once
        auto kloop_wreg = [&](auto coh) {
            constexpr bool COH = decltype(coh)::value;
            u32x4 bq[WREG ? NKW : 1][NTW];
#pragma unroll
            for (int ki = 0; ki < (WREG ? NKW : 0); ++ki) {
                const int ks = min(wave + 4 * ki, KS - 1);   // past the end: any valid block (its weights are zero)
#pragma unroll
                for (int i = 0; i < NTW; ++i)
                    bq[ki][i] = xch.template load16<COH>(xb + (unsigned)((i * KS + ks) * kWave + lane) * 16u);
            }
            __builtin_amdgcn_sched_barrier(0);   // all loads are issued before the first MFMA: one round trip, not NKW
#pragma unroll
            for (int ki = 0; ki < (WREG ? NKW : 0); ++ki)
#pragma unroll
                for (int a = 0; a < MT; ++a)
#pragma unroll
                    for (int i = 0; i < NTW; ++i) acc[a][i] = mfma_kstep<T>(wreg[a][ki], bq[ki][i], acc[a][i]);
        };
        if constexpr (WREG) kloop_wreg(std::true_type{});
        else kloop(std::true_type{});
#ifdef FASTLSTM_TIMELINE
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#endif
        FASTLSTM_TP(3);
        if (p.trace) {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // attribute the operand fetch to this phase
            tr2 = (long long)wall_clock64();
        }
        // ---- partial sums -> LDS, then every (tile, lane) item sums its P partials ------
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int i = 0; i < NTW; ++i) {
                const int tl = (mt_base + a) * NT + nt_base + i;
                const int pp = SPLIT == 0 ? wave : 0;
                red[(pp * TILES + tl) * kWave + lane] = acc[a][i];
            }
        if constexpr (VIO) tile_to_lds(gpre[u], gt);
        FASTLSTM_TP(4);
        __syncthreads();
        FASTLSTM_TP(5);

        const unsigned xn = xgrp + (unsigned)slot_w * xslot;
        // Results of this step.  Only the exchange copy of h_t is on the critical path: it is
        // stored first and alone, the workgroup publishes, and the bulk stores (pre-activations,
        // c_t, h_t for the caller) are issued after the flag so that nobody waits for them.
        T st_p[IPT][4], st_h[IPT], st_c[IPT];
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const int tl = wave + 4 * m;
            if (tl < TILES) {
                f32x4 s = red[tl * kWave + lane];
#pragma unroll
                for (int pp = 1; pp < P; ++pp) s += red[(pp * TILES + tl) * kWave + lane];
                if (valid[m]) {
                    T *gl = reinterpret_cast<T *>(gt + goff[m]);   // the item's 4 gates in the LDS tile
                    T x4[4];
#pragma unroll
                    for (int gg = 0; gg < 4; ++gg) {
                        if constexpr (VIO) x4[gg] = gl[gg * HT];
                        else x4[gg] = pre[u][m][gg];
                    }
                    const float pi = E::to_f32(x4[0]) + s[0];
                    const float pf = E::to_f32(x4[1]) + s[1];
                    const float pg = E::to_f32(x4[2]) + s[2];
                    const float po = E::to_f32(x4[3]) + s[3];
                    const float c1 = sigmoidf_<ACC>(pf) * c_state[m] + sigmoidf_<ACC>(pi) * tanhf_<ACC>(pg);
                    const float h1 = sigmoidf_<ACC>(po) * tanhf_<ACC>(c1);
                    c_state[m] = c1;
                    st_h[m] = E::from_f32(h1);
                    xch.store_elem(xn + xoff[m], st_h[m]);
                    st_p[m][0] = E::from_f32(pi);
                    st_p[m][1] = E::from_f32(pf);
                    st_p[m][2] = E::from_f32(pg);
                    st_p[m][3] = E::from_f32(po);
                    st_c[m] = E::from_f32(c1);
                    if constexpr (VIO) {
#pragma unroll
                        for (int gg = 0; gg < 4; ++gg) gl[gg * HT] = st_p[m][gg];
                        *reinterpret_cast<T *>(gt + BT * GROW + soff[m]) = st_h[m];
                        *reinterpret_cast<T *>(gt + BT * GROW + BT * SROW + soff[m]) = st_c[m];
                    }
                }
            }
        }
        if (p.trace) tr3 = (long long)wall_clock64();
        FASTLSTM_TP(6);
        auto bulk_store = [&]() {
#pragma unroll
            for (int m = 0; m < IPT; ++m) {
                if (valid[m]) {
                    if (keep) {
                        T *dst = ifgo + (size_t)t * B4H + off_p[m];
                        dst[0] = st_p[m][0];
                        dst[(size_t)H] = st_p[m][1];
                        dst[(size_t)2 * H] = st_p[m][2];
                        dst[(size_t)3 * H] = st_p[m][3];
                    }
                    out[(size_t)(t + 1) * BH + off_h[m]] = st_h[m];
                    if (keep || t + 1 == T_) cell[(size_t)(t + 1) * BH + off_h[m]] = st_c[m];
                }
            }
        };
        if constexpr (SYNC) {
#ifdef FASTLSTM_TIMELINE
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            FASTLSTM_TP(7);
#endif
            if (t + 1 < T_) publish_version(my_flag, t + 2);
            else if constexpr (VIO) __syncthreads();   // last step: the tiles still have to be complete
            FASTLSTM_TP(8);
            if constexpr (VIO) tiles_to_global(t, gt);
            else bulk_store();
        } else {
            if constexpr (VIO) {
                __syncthreads();
                tiles_to_global(t, gt);
            } else {
                bulk_store();
                __syncthreads();
            }
        }
        prefetch(t + PD, uc);
        FASTLSTM_TP(9);
        slot_r = slot_w;
#ifndef FASTLSTM_TIMELINE
        if (p.trace && tid == 0) {  // accumulated wait / fetch+mfma / reduce+gates / publish times
            long long *tr = p.trace + (size_t)blockIdx.x * 4;
            tr[0] += tr1 - tr0;
            tr[1] += tr2 - tr1;
            tr[2] += tr3 - tr2;
            tr[3] += (long long)wall_clock64() - tr3;
        }
#endif
    };
    for (int t0 = 0; t0 < T_; t0 += PD) {
        step(t0, std::integral_constant<int, 0>{});
        if (t0 + 1 < T_) step(t0 + 1, std::integral_constant<int, 1>{});
        if constexpr (PD > 2) {
            if (t0 + 2 < T_) step(t0 + 2, std::integral_constant<int, 2>{});
            if (t0 + 3 < T_) step(t0 + 3, std::integral_constant<int, 3>{});
        }
    }
#ifdef FASTLSTM_TIMELINE
    __syncthreads();
    if (p.trace)
        for (int idx = tid; idx < 256; idx += kThreads) p.trace[(size_t)blockIdx.x * 256 + idx] = tl[idx];
#endif
#undef FASTLSTM_TP
}

}  // namespace fastlstm

// Persistent reverse-time kernel: d_ifgo[t], dh_0, dc_0 for one LSTM layer in one launch.
//
// Replaces lstm_persistent_seq_bwd (fastlstm/kernels.py:1201-1409).  Per step
// t = T-1 .. 0, for the workgroup's tile of bt batch rows x ht hidden units:
//     dh  = dh_rec + dout[t]
//     dc += dh * sigmoid(o) * (1 - tanh(c_t)^2)
//     d_o = dh * tanh(c_t) * sigmoid(o) * (1 - sigmoid(o))
//     d_f = dc * c_{t-1} * sigmoid(f) * (1 - sigmoid(f))
//     d_i = dc * tanh(g) * sigmoid(i) * (1 - sigmoid(i))
//     d_g = dc * sigmoid(i) * (1 - tanh(g)^2)
//     dc  = dc * sigmoid(f)                                   (kernels.py:1301-1316)
//     d_ifgo[t] <- (d_i, d_f, d_g, d_o);  barrier over the hidden tiles of the batch tile
//     dh_rec = d_ifgo[t][rows, 0:4H] . Wh[0:4H, units]        (kernels.py:1362-1383)
// The gates are re-evaluated from the stored (rounded) pre-activations and cell
// states, as the reference does.  Unlike the reference (kernels.py:1286-1291,
// 1337-1342, 1388-1390) dc and dh_rec never leave fp32 registers: both are local
// to the (unit, batch row) a thread owns.
//
// MI355X mapping: the column slice Wh[:, units] is transposed ONCE into LDS in MFMA
// operand order (K = (unit', gate) pairs, 4H long) and stays resident; d_ifgo[t]
// travels between workgroups through a double-buffered exchange buffer in operand
// order, so the K = 4H contraction reads fully coalesced 1 KiB blocks.
#pragma once
#include <type_traits>

#include "recurrent_common.hpp"

namespace fastlstm {

struct BwdParams {
    const void *dout;   // [T,B,H]
    void *dh, *dc;      // [B,H] in: grads of h_T, c_T; out: grads of h_0, c_0
    const void *ifgo;   // [T,B,4H]
    const void *cell;   // [T+1,B,H]
    void *d_ifgo;       // [T,B,4H]
    const void *Wh;     // [4H,H]
    WsHeader *hdr;
    int *flags;
    unsigned char *xbuf;   // [2 slots][n_bt][NT][KSB] operand blocks
    int T, B, H;
    int b_base;
    int n_bt, n_ht, flag_stride;
    int KSB;            // k-steps covering 4H
    int ht;             // hidden units per workgroup (SPLIT 0/1: 4, 8 or 16)
    long long spin_limit;
    int vec_io;         // 1: the VIO instantiation is launched (complete, 16-byte aligned tile segments)
    long long *trace;   // optional diagnostics: 4 accumulated phase times per workgroup, else nullptr
    // SPLIT 2 only: n_rec > 1 independent recurrences of this shape share the launch (see FwdParams)
    int n_rec, n_bt_launch;
    int rs;             // 2, 4: batch tiles of 16 / rs rows (RS instantiation; b_base and n_bt_launch count in those), else 0
    const void *dout_x[3], *ifgo_x[3], *cell_x[3], *Wh_x[3];
    void *dh_x[3], *dc_x[3], *d_ifgo_x[3];
};

// SPLIT 0: waves split K (NTW n-tiles per WG); SPLIT 1: waves split N (NTW n-tiles per wave);
// SPLIT 2: barrier-free small-H form, wave w owns unit tile w (up to 64 units), one n-tile.
// VIO: the workgroup's tiles of ifgo[t], cell[t], dout[t] and d_ifgo[t] move between global memory
// and LDS in 16-byte pieces (waves 1..3) instead of element by element; see the forward kernel.
// SPLIT 2 with tile I/O runs CW computing waves and four that move the tiles, as the forward kernel does.  CW = 8:
// the waves 2w and 2w + 1 both multiply unit tile w (8 MFMAs each, on different SIMDs) and each takes two of the
// four units that a lane's accumulator holds: half the gate arithmetic per wave, two waves per SIMD that overlap
// each other's latencies.
template <int SPLIT, bool VIO, int CW = 4> constexpr int bwd_threads() {
    return (SPLIT == 2 && VIO) ? (CW + 4) * kWave : kThreads;
}

// RS = 2 (with CW = 8) or 4 (with CW = 4): batch tiles of 16 / RS rows -- RS times the workgroups -- and ONE cell
// per lane instead of two or four: the lanes of the columns that do not exist take over the lane's other units
// through DPP rotations of the accumulator within the row of 16 lanes (the operand rows that do not exist are
// zeros).  See the forward kernel: the step of the 16-row form is bound by the vector ALU (T = 1024, B = 256, fp16:
// 0.82 us per step with 16 rows, 0.593 with 8, 0.458 with 4).
template <typename T, int NTW, int SPLIT, bool VIO, int CW = 4, int RS = 1>
__global__ __launch_bounds__((bwd_threads<SPLIT, VIO, CW>())) void lstm_bwd_persistent_kernel(const BwdParams p) {
    using E = Elem<T>;
    constexpr bool SYNC = SPLIT != 2;
    constexpr bool IOW = SPLIT == 2 && VIO;   // tile-moving waves CW..CW+3 behind the computing waves 0..CW-1
    static_assert(CW == 4 || (IOW && CW == 8), "8 computing waves: the one-tile form with tile I/O");
    constexpr int CT = CW * kWave;            // threads of the computing waves
    constexpr int UPL = 16 / CW;              // SPLIT 2: units of a lane (of the four its accumulator holds)
    constexpr bool ACC = (E::DT == FASTLSTM_FP32);
    constexpr int NT = SPLIT == 1 ? 4 * NTW : NTW;
    constexpr int P = SPLIT == 0 ? 4 : 1;
    constexpr int MTB = SPLIT == 2 ? 4 : 1;          // unit tiles (16 rows each) per workgroup
    static_assert(RS == 1 || (IOW && NTW == 1 && ((RS == 2 && CW == 8) || (RS == 4 && CW == 4))),
                  "batch tiles of 16 / RS rows: the one-tile form, RS units per lane folded into one cell");
    constexpr int NI = RS > 1 ? 1 : UPL;             // SPLIT 2: cells per lane
    constexpr int IPT = SPLIT == 2 ? NI : NT;        // (unit, batch row) items per thread, upper bound
    constexpr int BT = 16 * NT / RS;
    constexpr int CH = 16 / NTW;                     // k-steps fetched per batch of loads (2 batches in flight)

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const bool cw = !IOW || tid < CT;                    // a computing wave
    const int wave = IOW ? (tid >> 6) & (CW - 1) : tid >> 6;   // (a tile-moving wave mirrors the set-up of a computing wave and never uses it)
    const int ut = CW == 8 ? wave >> 1 : wave, mh = CW == 8 ? (wave & 1) : 0;   // SPLIT 2: the wave's unit tile, and which units of it
    const int KSB = p.KSB, H = p.H, B = p.B, T_ = p.T;
    const int HT = SYNC ? p.ht : 16 * MTB;           // unit slots per workgroup
    const int RPT = SYNC ? p.ht : 16;                // weight rows stored per unit tile
    const int n_utiles = SYNC ? 1 : cdiv(H, 16);     // unit tiles actually used

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
    auto pick = [&](auto a0, auto a1, auto a2, auto a3) {   // (constant indices only, see the forward kernel)
        if constexpr (SYNC) return a0;
        else return rec == 0 ? a0 : rec == 1 ? a1 : rec == 2 ? a2 : a3;
    };
    const int u0 = j * HT;
    const int b0 = p.b_base + g * BT;

    const size_t wbytes = (size_t)MTB * KSB * 4 * RPT * 16;
    unsigned char *Wl = smem;                                                // + one all-zero operand block
    const size_t zero_off = wbytes;
    f32x4 *red = reinterpret_cast<f32x4 *>(smem + wbytes + kFragBytes);      // [P][MTB][NT][64]
    unsigned char *xl = reinterpret_cast<unsigned char *>(red + P * MTB * NT * kWave);  // SPLIT 2

    // ---- tile I/O geometry (VIO) ---------------------------------------------------------
    // gates tile [BT][4 gates][HT] with rows padded to GROW bytes, then two state tiles
    // [BT][HT] (c_{t-1} and dout[t]) with rows of SROW bytes.  HT is a run-time value here.
    constexpr int HTMAX = SYNC ? 16 : 64;
    constexpr int PPSEG_MAX = HTMAX * E::BYTES / 16 > 0 ? HTMAX * E::BYTES / 16 : 1;
    constexpr int IOT = IOW ? kThreads : kThreads - kWave;   // wave 0 polls the flags and moves nothing; IOW: waves 4..7
    constexpr int GPT = (BT * 4 * PPSEG_MAX + IOT - 1) / IOT, SPT = (BT * PPSEG_MAX + IOT - 1) / IOT;
    const int GSEG = HT * E::BYTES, GROW = 4 * GSEG + 16, SROW = GSEG + 16;
    const int PPSEG = GSEG / 16;            // 16-byte pieces per segment (>= 1 when VIO)
    const int TILE_BYTES = BT * GROW + 2 * BT * SROW;
    unsigned char *tiles = xl + (SYNC ? 0 : 2 * (size_t)KSB * kFragBytes);   // SYNC: 1 set, else 2 (step parity)
    const int io_tid = IOW ? tid - CT : tid - kWave;   // < 0: not an I/O thread

    const T *dout = static_cast<const T *>(pick(p.dout, p.dout_x[0], p.dout_x[1], p.dout_x[2]));
    const T *ifgo = static_cast<const T *>(pick(p.ifgo, p.ifgo_x[0], p.ifgo_x[1], p.ifgo_x[2]));
    const T *cell = static_cast<const T *>(pick(p.cell, p.cell_x[0], p.cell_x[1], p.cell_x[2]));
    T *d_ifgo = static_cast<T *>(pick(p.d_ifgo, p.d_ifgo_x[0], p.d_ifgo_x[1], p.d_ifgo_x[2]));
    const T *Wh = static_cast<const T *>(pick(p.Wh, p.Wh_x[0], p.Wh_x[1], p.Wh_x[2]));
    T *dh_io = static_cast<T *>(pick(p.dh, p.dh_x[0], p.dh_x[1], p.dh_x[2]));
    T *dc_io = static_cast<T *>(pick(p.dc, p.dc_x[0], p.dc_x[1], p.dc_x[2]));

    // ---- prologue: Wh[:, units] -> LDS, transposed into operand order ------------------
    {
        const int Kpad = KSB * E::KSTEP;
        const int total = Kpad * HT;
        for (int idx = tid; cw && idx < total; idx += CT) {
            const int ul = idx % HT, k = idx / HT;
            const int uk = k >> 2, gate = k & 3;
            T v = E::from_f32(0.f);
            if (uk < H && u0 + ul < H) v = Wh[((size_t)gate * H + uk) * H + u0 + ul];
            const int mtile = SYNC ? 0 : (ul >> 4);
            const int r = SYNC ? ul : (ul & 15);
            const int ks = k / E::KSTEP, kk = k % E::KSTEP;
            const size_t off = ((((size_t)mtile * KSB + ks) * 4 + kk / E::EPL) * RPT + r) * 16 +
                               (kk % E::EPL) * E::BYTES;
            *reinterpret_cast<T *>(Wl + off) = v;
        }
        if (tid < kWave) reinterpret_cast<u32x4 *>(Wl + zero_off)[tid] = u32x4{0u, 0u, 0u, 0u};
        if constexpr (!SYNC) {
            for (int idx = tid; cw && idx < 2 * KSB * kWave; idx += CT)
                reinterpret_cast<u32x4 *>(xl)[idx] = u32x4{0u, 0u, 0u, 0u};
        }
    }
    __syncthreads();
    // One hidden tile per workgroup: this wave's unit tile of Wh^T, all k-steps, in registers (the LDS
    // copy was a chain of dependent round trips per step).  Waves without a unit tile hold zeros.
    constexpr int KSB2 = 256 / E::KSTEP;   // k-steps that cover 4H for H = 64
    u32x4 wb2[SPLIT == 2 ? KSB2 : 1];
    if constexpr (SPLIT == 2) {
        const int q_ = lane >> 4, r_ = lane & 15;
#pragma unroll
        for (int ks = 0; ks < KSB2; ++ks) {
            const bool ok = ks < KSB && ut < n_utiles;
            const unsigned char *wp = ok ? Wl + ((((size_t)ut * KSB + ks) * 4 + q_) * RPT + (r_ % RPT)) * 16
                                         : Wl + zero_off + lane * 16;
            wb2[ks] = *reinterpret_cast<const u32x4 *>(wp);
        }
    }

    // ---- per-thread items: it = tid + 256 m -> (row n, unit ul, n-tile nt) --------------
    float dc_state[IPT], dh_rec[IPT], c1v[IPT];
    size_t off_h[IPT], off_p[IPT];
    int xoff[IPT], roff[IPT];
    int goff[IPT], soff[IPT];   // VIO: byte offsets of the item inside the LDS gates / state tiles
    bool valid[IPT], pair_lead[IPT];
    const size_t BH = (size_t)B * H, B4H = (size_t)B * 4 * H;
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        // SPLIT 2: the item is element mh * UPL + m of the lane's own accumulator -- that unit of 4 * (lane / 16) .. + 3
        // of the wave's unit tile, batch row lane % 16 -- so the product of a step lands where it is used
        const int it = tid + kThreads * m;
        // (RS 2, 4: row lane % (16 / RS), and of the wave's RS units per lane group the one that lane % 16 / (16 / RS) names)
        const int n = RS > 1 ? (lane & 15) % (16 / RS) : SPLIT == 2 ? (lane & 15) : (it & 15), rest = it >> 4;
        const int ul = RS > 1 ? ut * 16 + (lane >> 4) * 4 + mh * UPL + (lane & 15) / (16 / RS)
                              : SPLIT == 2 ? ut * 16 + (lane >> 4) * 4 + mh * UPL + m : rest % HT;
        const int nt = SPLIT == 2 ? 0 : rest / HT;
        const int unit = u0 + ul, b = b0 + nt * 16 + n;
        valid[m] = nt < NT && unit < H && b < B;
        // invalid items point at the tile's first element: their loads stay in bounds, nothing is stored
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        off_p[m] = valid[m] ? (size_t)b * 4 * H + unit : (size_t)b0 * 4 * H + u0;
        xoff[m] = nt * KSB * kFragBytes + frag_offset<T>(n, unit * 4);
        pair_lead[m] = valid[m] && ((ul & 1) == 0);  // u0 is a multiple of 4: even ul <=> low half of a slot
        goff[m] = (nt * 16 + n) * GROW + ul * E::BYTES;
        soff[m] = (nt * 16 + n) * SROW + ul * E::BYTES;
        const int mtile = ul >> 4, ur = ul & 15;
        roff[m] = ((mtile * NT + (nt < NT ? nt : 0)) * kWave + (ur >> 2) * 16 + n) * 4 + (ur & 3);
        dh_rec[m] = valid[m] ? E::to_f32(dh_io[off_h[m]]) : 0.f;
        dc_state[m] = valid[m] ? E::to_f32(dc_io[off_h[m]]) : 0.f;
        c1v[m] = valid[m] ? E::to_f32(cell[(size_t)T_ * BH + off_h[m]]) : 0.f;
    }

    using Xchg = typename std::conditional<SYNC, XchgGlobal, XchgLds>::type;
    const unsigned xslot = SYNC ? (unsigned)p.n_bt * NT * KSB * kFragBytes : (unsigned)KSB * kFragBytes;
    const unsigned xgrp = SYNC ? (unsigned)g * NT * KSB * kFragBytes : 0u;
    constexpr int n_slots = 2;   // reverse step s uses slot s % 2; the loads are device-scope (the address is reused)
    const Xchg xch(SYNC ? p.xbuf : xl, (unsigned)n_slots * xslot);
    int *my_flag = SYNC ? p.flags + (size_t)g * p.flag_stride + j : nullptr;
    const int *grp_flags = SYNC ? p.flags + (size_t)g * p.flag_stride : nullptr;

    // Stored activations and dout do not depend on the recurrence: they are requested PD steps
    // ahead (an HBM round trip is ~2 us).  The loads are unconditional -- invalid items read a valid
    // dummy address -- so that their results stay in the registers they were loaded into: a
    // conditional load ends in a register copy, and the copy in a wait for the load.
    constexpr int PD = SYNC ? 2 : 4;
    constexpr int PRE_N = VIO ? 1 : PD, GPRE_N = VIO ? PD : 1;
    T pre[PRE_N][IPT][4], c0r[PRE_N][IPT], dor[PRE_N][IPT];
    auto fetch = [&](int t, T(&dp)[IPT][4], T(&dc0)[IPT], T(&dd)[IPT]) {
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const T *src = ifgo + (size_t)t * B4H + off_p[m];
#pragma unroll
            for (int gt = 0; gt < 4; ++gt) dp[m][gt] = src[(size_t)gt * H];
            dc0[m] = cell[(size_t)t * BH + off_h[m]];
            dd[m] = dout[(size_t)t * BH + off_h[m]];
        }
    };
    // VIO: the 16-byte pieces this thread moves.  Piece pc of the gates tile = (row, gate, k-th
    // piece of the segment); pieces that do not exist or lie past the batch read the tile origin.
    unsigned g_glb[GPT], s_glb[SPT];   // element offsets inside ifgo[t] / cell[t]
    int g_lds[GPT], s_lds[SPT];        // byte offsets inside the LDS tiles
    bool g_ok[GPT], s_ok[SPT];
    u32x4 gpre[GPRE_N][GPT], cpre[GPRE_N][SPT], dpre[GPRE_N][SPT];
    if constexpr (VIO) {
        const int gpieces = BT * 4 * PPSEG, spieces = BT * PPSEG;
#pragma unroll
        for (int i = 0; i < GPT; ++i) {
            const int pc = io_tid + IOT * i;
            const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG);
            const int seg = rem / PPSEG, k = rem % PPSEG;
            g_ok[i] = io_tid >= 0 && pc < gpieces && b0 + row < B;
            g_lds[i] = g_ok[i] ? row * GROW + seg * GSEG + k * 16 : 0;
            g_glb[i] = (unsigned)((size_t)b0 * 4 * H + u0) +
                       (g_ok[i] ? (unsigned)(row * 4 * H + seg * H + k * (16 / E::BYTES)) : 0u);
        }
#pragma unroll
        for (int i = 0; i < SPT; ++i) {
            const int pc = io_tid + IOT * i;
            const int row = pc / PPSEG, k = pc % PPSEG;
            s_ok[i] = io_tid >= 0 && pc < spieces && b0 + row < B;
            s_lds[i] = s_ok[i] ? row * SROW + k * 16 : 0;
            s_glb[i] = (unsigned)((size_t)b0 * H + u0) + (s_ok[i] ? (unsigned)(row * H + k * (16 / E::BYTES)) : 0u);
        }
    }
    auto fetch_tiles = [&](int t, u32x4(&gp)[GPT], u32x4(&cp)[SPT], u32x4(&dp)[SPT]) {
        if (io_tid < 0) return;
#pragma unroll
        for (int i = 0; i < GPT; ++i) gp[i] = *reinterpret_cast<const u32x4 *>(ifgo + (size_t)t * B4H + g_glb[i]);
#pragma unroll
        for (int i = 0; i < SPT; ++i) {
            cp[i] = *reinterpret_cast<const u32x4 *>(cell + (size_t)t * BH + s_glb[i]);
            dp[i] = *reinterpret_cast<const u32x4 *>(dout + (size_t)t * BH + s_glb[i]);
        }
    };
    auto tiles_to_lds = [&](const u32x4(&gp)[GPT], const u32x4(&cp)[SPT], const u32x4(&dp)[SPT], unsigned char *gt) {
        unsigned char *stc = gt + BT * GROW, *std_ = stc + BT * SROW;
#pragma unroll
        for (int i = 0; i < GPT; ++i)
            if (g_ok[i]) *reinterpret_cast<u32x4 *>(gt + g_lds[i]) = gp[i];
#pragma unroll
        for (int i = 0; i < SPT; ++i)
            if (s_ok[i]) {
                *reinterpret_cast<u32x4 *>(stc + s_lds[i]) = cp[i];
                *reinterpret_cast<u32x4 *>(std_ + s_lds[i]) = dp[i];
            }
    };
    // LDS gates tile (now d_i, d_f, d_g, d_o) -> d_ifgo[t]
    auto tile_to_global = [&](int t, const unsigned char *gt) {
#pragma unroll
        for (int i = 0; i < GPT; ++i)
            if (g_ok[i])
                *reinterpret_cast<u32x4 *>(d_ifgo + (size_t)t * B4H + g_glb[i]) =
                    *reinterpret_cast<const u32x4 *>(gt + g_lds[i]);
    };
    // inputs of reverse step s (timestep T-1-s) into ring entry s % PD
    auto prefetch = [&](int s, auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        if constexpr (IOW) return;   // (the tile-moving waves have a loop of their own, below)
        if (s < T_) {
            if constexpr (VIO) fetch_tiles(T_ - 1 - s, gpre[u], cpre[u], dpre[u]);
            else fetch(T_ - 1 - s, pre[u], c0r[u], dor[u]);
        }
    };
    // ---- the tile-moving waves of the one-tile form: their own time loop, every vector-memory instruction
    // unconditional and four steps unrolled without a branch between them, so that the compiler's counted waits
    // name the loads of the tiles that go into LDS next and leave everything younger in flight (see the forward
    // kernel; T = 1024, B = 256, H = 64: 0.98 -> 0.87 us per step)
    if constexpr (IOW) {
        if (!cw) {
            constexpr unsigned kOut = 0xfffffff0u;
            const u32x4 zero = {0u, 0u, 0u, 0u};
            unsigned gv[GPT], sv[SPT];   // byte offsets inside ifgo[t] / d_ifgo[t] and cell[t] / dout[t]; kOut: no such piece
#pragma unroll
            for (int i = 0; i < GPT; ++i) gv[i] = g_ok[i] ? g_glb[i] * (unsigned)E::BYTES : kOut;
#pragma unroll
            for (int i = 0; i < SPT; ++i) sv[i] = s_ok[i] ? s_glb[i] * (unsigned)E::BYTES : kOut;
            const unsigned g_bytes = (unsigned)(B4H * E::BYTES), s_bytes = (unsigned)(BH * E::BYTES);
            u32x4 rg_[PD][GPT], rc_[PD][SPT], rd_[PD][SPT];
            // the input tiles of reverse step s2 (timestep T - 1 - s2; past the first timestep: empty buffers, zeros)
            auto load_tiles = [&](int s2, auto uc) __attribute__((always_inline)) {
                constexpr int u = decltype(uc)::value;
                const int t2 = T_ - 1 - s2, tc = max(t2, 0);
                const bool live = t2 >= 0;
                const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(ifgo) + (size_t)tc * B4H, 0, live ? g_bytes : 0u, 0x00020000);
                const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(cell) + (size_t)tc * BH, 0, live ? s_bytes : 0u, 0x00020000);
                const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(dout) + (size_t)tc * BH, 0, live ? s_bytes : 0u, 0x00020000);
#pragma unroll
                for (int i = 0; i < GPT; ++i) rg_[u][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rg, gv[i], 0, 0));
#pragma unroll
                for (int i = 0; i < SPT; ++i) {
                    rc_[u][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rc, sv[i], 0, 0));
                    rd_[u][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rd, sv[i], 0, 0));
                }
            };
            auto dropped_stores = [&](unsigned group) __attribute__((always_inline)) {   // as many as a step issues, each at an offset of its own
                const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(d_ifgo, 0, g_bytes, 0x00020000);
#pragma unroll
                for (int i = 0; i < GPT; ++i) __builtin_amdgcn_raw_buffer_store_b128(zero, rg, kOut - 16u * (group * GPT + i), 0, 0);
            };
            auto io_step = [&](int s2, auto uc) __attribute__((always_inline)) {
                constexpr int u = decltype(uc)::value, un = (u + 1) % PD;
                tiles_to_lds(rg_[un], rc_[un], rd_[un], tiles + ((s2 + 1) & 1) * TILE_BYTES);   // the next step's inputs
                __syncthreads();
                const unsigned char *gt = tiles + (s2 & 1) * TILE_BYTES;   // this step's d_ifgo tile
                const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(d_ifgo + (size_t)(T_ - 1 - s2) * B4H, 0, g_bytes, 0x00020000);
#pragma unroll
                for (int i = 0; i < GPT; ++i)
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(gt + g_lds[i]), ro, gv[i], 0, 0);
                load_tiles(s2 + PD, uc);
            };
            static_assert(PD == 4, "four steps per pass of the loop");
            // (the loop is entered with what every later pass finds in flight: between the tiles, as many stores as a step issues)
            load_tiles(0, std::integral_constant<int, 0>{});
            dropped_stores(0);
            load_tiles(1, std::integral_constant<int, 1>{});
            dropped_stores(1);
            load_tiles(2, std::integral_constant<int, 2>{});
            dropped_stores(2);
            load_tiles(3, std::integral_constant<int, 3>{});
            tiles_to_lds(rg_[0], rc_[0], rd_[0], tiles);
            __syncthreads();
            int s0 = 0;
            for (; s0 + PD <= T_; s0 += PD) {
                io_step(s0, std::integral_constant<int, 0>{});
                io_step(s0 + 1, std::integral_constant<int, 1>{});
                io_step(s0 + 2, std::integral_constant<int, 2>{});
                io_step(s0 + 3, std::integral_constant<int, 3>{});
            }
            if (s0 < T_) io_step(s0, std::integral_constant<int, 0>{});
            if (s0 + 1 < T_) io_step(s0 + 1, std::integral_constant<int, 1>{});
            if (s0 + 2 < T_) io_step(s0 + 2, std::integral_constant<int, 2>{});
            return;
        }
    }
    prefetch(0, std::integral_constant<int, 0>{});
    if constexpr (IOW) {
        __syncthreads();   // the tiles of step 0 are in LDS (the tile-moving waves' loop)
    } else if constexpr (VIO) {   // step 0 works on the LDS tiles right away; its ring entry is refilled in step 0
        tiles_to_lds(gpre[0], cpre[0], dpre[0], tiles);
        __syncthreads();
    }
    prefetch(1, std::integral_constant<int, 1>{});
    if constexpr (PD > 2) {
        prefetch(2, std::integral_constant<int, 2>{});
        prefetch(3, std::integral_constant<int, 3>{});
    }

    int slot = 0;  // ring slot of this step's d_ifgo
    // One hidden tile per workgroup: the lane's UPL units of the current step's tile rows (4 gates,
    // c_{t-1}, dout), read a step ahead
    using NxV = typename VecBytes<(SPLIT == 2 ? NI : 4) * E::BYTES>::type;
    NxV nx[6];
    auto load_items = [&](const unsigned char *gt_) __attribute__((always_inline)) {
#pragma unroll
        for (int gg = 0; gg < 4; ++gg) nx[gg] = *reinterpret_cast<const NxV *>(gt_ + goff[0] + gg * GSEG);
        nx[4] = *reinterpret_cast<const NxV *>(gt_ + BT * GROW + soff[0]);
        nx[5] = *reinterpret_cast<const NxV *>(gt_ + BT * GROW + BT * SROW + soff[0]);
    };
    if constexpr (SPLIT == 2 && VIO) {
        if (cw) load_items(tiles);
    }
    // One reverse step; u = s % PD selects the prefetch ring entry at compile time.
    auto step = [&](const int s, auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        const int t = T_ - 1 - s;
        const unsigned xw = xgrp + (unsigned)slot * xslot;
        slot = (slot + 1 == n_slots) ? 0 : slot + 1;

        long long tr0 = 0, tr1 = 0, tr2 = 0, tr3 = 0;
        if (p.trace) tr0 = (long long)wall_clock64();
        unsigned char *gt = tiles + (SYNC ? 0 : (s & 1) * TILE_BYTES);         // VIO: this step's tiles
        unsigned char *gt_next = tiles + (SYNC ? 0 : ((s + 1) & 1) * TILE_BYTES);
        if constexpr (SPLIT == 2) {
            // One hidden tile per workgroup.  The lane's four items are four consecutive units of one batch
            // row: every tile row is touched with one LDS access per gate, the lane writes whole operand
            // slots of the exchange copy, and the product comes back in the lane's own accumulator (nothing
            // is reduced).  One workgroup barrier per step: behind it the exchange copy, the d_ifgo tile
            // and the next step's input tiles are all in LDS.
            using V = typename VecBytes<NI * E::BYTES>::type;
            if (cw) {
            T xg[4][NI], xc[NI], xd[NI], st_d[NI][4];
            if constexpr (VIO) {   // read behind the previous step's barrier (or in the prologue)
#pragma unroll
                for (int gg = 0; gg < 4; ++gg) __builtin_memcpy(xg[gg], &nx[gg], NI * E::BYTES);
                __builtin_memcpy(xc, &nx[4], NI * E::BYTES);
                __builtin_memcpy(xd, &nx[5], NI * E::BYTES);
            } else {
#pragma unroll
                for (int m = 0; m < NI; ++m) {
#pragma unroll
                    for (int gg = 0; gg < 4; ++gg) xg[gg][m] = pre[u][m][gg];
                    xc[m] = c0r[u][m];
                    xd[m] = dor[u][m];
                }
            }
#pragma unroll
            for (int m = 0; m < NI; ++m) {
                const float si = sigmoidf_<ACC>(E::to_f32(xg[0][m]));
                const float sf = sigmoidf_<ACC>(E::to_f32(xg[1][m]));
                const float tg = tanhf_<ACC>(E::to_f32(xg[2][m]));
                const float so = sigmoidf_<ACC>(E::to_f32(xg[3][m]));
                const float tc = tanhf_<ACC>(c1v[m]);
                const float c0 = E::to_f32(xc[m]);
                const float dh = dh_rec[m] + E::to_f32(xd[m]);
                const float dc1 = dc_state[m] + dh * so * (1.f - tc * tc);
                const float d_o = dh * tc * so * (1.f - so);
                const float d_f = dc1 * c0 * sf * (1.f - sf);
                const float d_i = dc1 * tg * si * (1.f - si);
                const float d_g = dc1 * si * (1.f - tg * tg);
                dc_state[m] = dc1 * sf;
                c1v[m] = c0;  // c_{t-1} is the next step's c_t
                // items past H or B: zeros (they are operands of the product below)
                st_d[m][0] = E::from_f32(valid[m] ? d_i : 0.f);
                st_d[m][1] = E::from_f32(valid[m] ? d_f : 0.f);
                st_d[m][2] = E::from_f32(valid[m] ? d_g : 0.f);
                st_d[m][3] = E::from_f32(valid[m] ? d_o : 0.f);
            }
            // exchange copy: k = 4 * unit + gate, whole 16-byte operand slots (two units of a 16-bit
            // type, one of fp32); slots past 4H do not exist in the blocks and are left alone
            if constexpr (RS > 1 && E::BYTES == 2) {   // one unit: half an operand slot
                if (valid[0]) {
                    u32x2 v;
                    __builtin_memcpy(&v, st_d[0], 8);
                    xch.store8(xw + xoff[0], v);
                }
            } else if constexpr (E::BYTES == 2) {
#pragma unroll
                for (int m = 0; m < NI; m += 2)
                    if (valid[m]) {
                        u32x4 v;
                        __builtin_memcpy(&v, st_d[m], 16);
                        xch.store16(xw + xoff[m], v);
                    }
            } else {
#pragma unroll
                for (int m = 0; m < NI; ++m)
                    if (valid[m]) {
                        u32x4 v;
                        __builtin_memcpy(&v, st_d[m], 16);
                        xch.store16(xw + xoff[m], v);
                    }
            }
            if constexpr (VIO) {
#pragma unroll
                for (int gg = 0; gg < 4; ++gg) {
                    T pk[NI];
#pragma unroll
                    for (int m = 0; m < NI; ++m) pk[m] = st_d[m][gg];
                    V v;
                    __builtin_memcpy(&v, pk, sizeof(V));
                    *reinterpret_cast<V *>(gt + goff[0] + gg * GSEG) = v;
                }
            } else {
#pragma unroll
                for (int m = 0; m < NI; ++m)
                    if (valid[m]) {
                        T *dst = d_ifgo + (size_t)t * B4H + off_p[m];
                        dst[0] = st_d[m][0];
                        dst[(size_t)H] = st_d[m][1];
                        dst[(size_t)2 * H] = st_d[m][2];
                        dst[(size_t)3 * H] = st_d[m][3];
                    }
            }
            }   // computing waves
            // tile-moving waves: the next step's inputs into the other tile set before the barrier, this
            // step's d_ifgo tile out of this one behind it
            __syncthreads();   // (with tile I/O: the tile-moving waves meet it in their own loop)
            prefetch(s + PD, uc);
            if (!cw) return;
            // dh_rec(units of this wave, rows) = Wh[:, units]^T . d_ifgo[t](rows, :)^T over K = 4H
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
            u32x4 bq[KSB2];
#pragma unroll
            for (int ks = 0; ks < KSB2; ++ks)   // past the end: any valid block (its weights are zero)
                bq[ks] = xch.template load16<false>(xw + (unsigned)(min(ks, KSB - 1) * kWave + lane) * 16u);
            if constexpr (VIO) {   // the next step's tile rows (in LDS since the barrier above)
                if (s + 1 < T_) load_items(gt_next);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < KSB2; ++ks) acc = mfma_kstep<T>(wb2[ks], bq[ks], acc);
            if constexpr (RS == 2) {
                // (scalars, not elements of the vector inside the builtin: see the forward kernel)
                const float a0 = acc[0], a1 = acc[1], a2 = acc[2], a3 = acc[3];
                dh_rec[0] = fold_upper_half(mh ? a2 : a0, mh ? a3 : a1);
            } else if constexpr (RS == 4) {
                const float a0 = acc[0], a1 = acc[1], a2 = acc[2], a3 = acc[3];
                dh_rec[0] = fold_quarters(a0, a1, a2, a3);
            } else {
#pragma unroll
                for (int m = 0; m < UPL; ++m) dh_rec[m] = (CW == 8 && mh) ? acc[UPL + m] : acc[m];
            }
            return;
        }
        // ---- point-wise gate backward for this thread's items --------------------------
        T st_d[IPT][4];
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            if (valid[m]) {
                T x4[4], xc, xd;
                T *gl = reinterpret_cast<T *>(gt + goff[m]);   // VIO: the item's 4 gates in the LDS tile
                if constexpr (VIO) {
#pragma unroll
                    for (int gg = 0; gg < 4; ++gg) x4[gg] = gl[gg * HT];
                    xc = *reinterpret_cast<const T *>(gt + BT * GROW + soff[m]);
                    xd = *reinterpret_cast<const T *>(gt + BT * GROW + BT * SROW + soff[m]);
                } else {
#pragma unroll
                    for (int gg = 0; gg < 4; ++gg) x4[gg] = pre[u][m][gg];
                    xc = c0r[u][m];
                    xd = dor[u][m];
                }
                const float si = sigmoidf_<ACC>(E::to_f32(x4[0]));
                const float sf = sigmoidf_<ACC>(E::to_f32(x4[1]));
                const float tg = tanhf_<ACC>(E::to_f32(x4[2]));
                const float so = sigmoidf_<ACC>(E::to_f32(x4[3]));
                const float tc = tanhf_<ACC>(c1v[m]);
                const float c0 = E::to_f32(xc);
                const float dh = dh_rec[m] + E::to_f32(xd);
                const float dc1 = dc_state[m] + dh * so * (1.f - tc * tc);
                const float d_o = dh * tc * so * (1.f - so);
                const float d_f = dc1 * c0 * sf * (1.f - sf);
                const float d_i = dc1 * tg * si * (1.f - si);
                const float d_g = dc1 * si * (1.f - tg * tg);
                dc_state[m] = dc1 * sf;
                c1v[m] = c0;  // c_{t-1} is the next step's c_t
                st_d[m][0] = E::from_f32(d_i);
                st_d[m][1] = E::from_f32(d_f);
                st_d[m][2] = E::from_f32(d_g);
                st_d[m][3] = E::from_f32(d_o);
                if constexpr (VIO) {
#pragma unroll
                    for (int gg = 0; gg < 4; ++gg) gl[gg * HT] = st_d[m][gg];
                }
            } else {
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) st_d[m][gt] = E::from_f32(0.f);
            }
            // Exchange copy now (critical path): 4 consecutive k = (unit, gate 0..3); the copy for
            // the GEMMs is stored after the flag has been raised.  A 16-byte operand slot holds two
            // units of the 16-bit types: lanes l and l+16 own units u and u+1 of the same batch row,
            // so the even-unit lane fetches its neighbour's half and writes the whole slot -- the
            // write-through stores then cover full 32-byte sectors instead of halves.
            if constexpr (E::BYTES == 2) {
                const u32x2 mine = *reinterpret_cast<u32x2 *>(st_d[m]);
                u32x2 other;
                other[0] = (unsigned)__shfl_down((int)mine[0], 16);
                other[1] = (unsigned)__shfl_down((int)mine[1], 16);
                if (pair_lead[m]) xch.store16(xw + xoff[m], u32x4{mine[0], mine[1], other[0], other[1]});
            } else {
                if (valid[m]) xch.store16(xw + xoff[m], *reinterpret_cast<u32x4 *>(st_d[m]));
            }
        }
        auto bulk_store = [&]() {
#pragma unroll
            for (int m = 0; m < IPT; ++m) {
                if (valid[m]) {
                    T *dst = d_ifgo + (size_t)t * B4H + off_p[m];
                    dst[0] = st_d[m][0];
                    dst[(size_t)H] = st_d[m][1];
                    dst[(size_t)2 * H] = st_d[m][2];
                    dst[(size_t)3 * H] = st_d[m][3];
                }
            }
        };
        constexpr int un = (u + 1) % PD;   // ring entry of the next step's inputs
        if constexpr (SYNC) {
            publish_version(my_flag, s + 1);
            if (p.trace) tr1 = (long long)wall_clock64();
            if constexpr (VIO) tile_to_global(t, gt);
            else bulk_store();
        } else {
            if constexpr (VIO) {
                __syncthreads();
                tile_to_global(t, gt);
                if (s + 1 < T_) tiles_to_lds(gpre[un], cpre[un], dpre[un], gt_next);
            } else {
                bulk_store();
                __syncthreads();
            }
        }

        // recurrence-independent operands of a later step: issue before waiting
        prefetch(s + PD, uc);

        if (p.trace) tr2 = (long long)wall_clock64();
        if constexpr (SYNC) {
            if (wave == 0) wait_versions(grp_flags, p.n_ht, s + 1, p.hdr, p.spin_limit, g, s);
            __syncthreads();
            // the tile has been drained: the next step's inputs may take its place
            if constexpr (VIO) {
                if (s + 1 < T_) tiles_to_lds(gpre[un], cpre[un], dpre[un], gt_next);
            }
        }
        if (p.trace) tr3 = (long long)wall_clock64();

        // ---- dh_rec(units, rows) = Wh[:, units]^T . d_ifgo[t](rows, :)^T over K = 4H ----
        f32x4 acc[NTW];
#pragma unroll
        for (int i = 0; i < NTW; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        const int kfirst = SPLIT == 0 ? wave : 0, kstride = SPLIT == 0 ? 4 : 1;
        const int nk = (SPLIT == 2 && wave >= n_utiles) ? 0 : (SPLIT == 0 ? (KSB - wave + 3) / 4 : KSB);
        const int nt_base = SPLIT == 1 ? wave * NTW : 0;
        const int mtile = SPLIT == 2 ? wave : 0;
        const int q = lane >> 4, r = lane & 15;
        const unsigned char *wrow = Wl + (((size_t)mtile * KSB * 4 + q) * RPT + (r % RPT)) * 16;
        const unsigned xb = xw;

        // straight-line chunks of CH k-steps, no branch inside (see the forward kernel)
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
                            xb + (unsigned)(((nt_base + i) * KSB + ks) * kWave + lane) * 16u);
                }
            };
            auto compute = [&](const u32x4(&bq)[CH][NTW], int ki0) {
#pragma unroll
                for (int cc = 0; cc < CH; ++cc) {
                    const int ki = ki0 + cc;
                    const int ks = kfirst + ki * kstride;
                    const unsigned char *wp = ki < nk ? wrow + (size_t)ks * 4 * RPT * 16 : Wl + zero_off + lane * 16;
                    const u32x4 af = *reinterpret_cast<const u32x4 *>(wp);
#pragma unroll
                    for (int i = 0; i < NTW; ++i) acc[i] = mfma_kstep<T>(af, bq[cc][i], acc[i]);
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
        kloop(std::true_type{});
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
            const int pp = SPLIT == 0 ? wave : 0;
            red[((pp * MTB + mtile) * NT + nt_base + i) * kWave + lane] = acc[i];
        }
        __syncthreads();
        const float *redf = reinterpret_cast<const float *>(red);
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            float v = redf[roff[m]];
#pragma unroll
            for (int pp = 1; pp < P; ++pp) v += redf[roff[m] + pp * MTB * NT * kWave * 4];
            dh_rec[m] = v;
        }
        if (p.trace && tid == 0) {  // accumulated gate maths / publish+stores / wait / fetch+mfma+reduce
            long long *tr = p.trace + (size_t)blockIdx.x * 4;
            tr[0] += tr1 - tr0;
            tr[1] += tr2 - tr1;
            tr[2] += tr3 - tr2;
            tr[3] += (long long)wall_clock64() - tr3;
        }
        // the next iteration's publish (or block barrier) orders these reads before the
        // next writes to `red`
    };
    for (int s0 = 0; s0 < T_; s0 += PD) {
        step(s0, std::integral_constant<int, 0>{});
        if (s0 + 1 < T_) step(s0 + 1, std::integral_constant<int, 1>{});
        if constexpr (PD > 2) {
            if (s0 + 2 < T_) step(s0 + 2, std::integral_constant<int, 2>{});
            if (s0 + 3 < T_) step(s0 + 3, std::integral_constant<int, 3>{});
        }
    }

    T *dh_out = dh_io, *dc_out = dc_io;
#pragma unroll
    for (int m = 0; m < IPT; ++m)
        if (cw && valid[m]) {
            dh_out[off_h[m]] = E::from_f32(dh_rec[m]);
            dc_out[off_h[m]] = E::from_f32(dc_state[m]);
        }
}

}  // namespace fastlstm

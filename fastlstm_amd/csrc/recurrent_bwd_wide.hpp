// Persistent reverse-time kernel for hidden sizes whose W_h does not fit the CUs of one XCD
// (H = 1536, 2048 with 16-bit elements): the counterpart of lstm_fwd_wide_kernel.  Same mathematics
// and results as lstm_bwd_persistent_kernel (which replaces fastlstm/kernels.py:1201-1409).
//
// A workgroup of 8 waves owns 16 hidden units and up to 64 batch rows and keeps Wh[:, units]^T (K = 4H
// rows of (unit, gate) pairs, 256 KiB for H = 2048) in registers: the waves split K eight ways.
// A barrier group has H / 16 workgroups on xpg = H / 512 whole XCDs (placement, flags and exchange
// ring as in the forward kernel).  Per step every workgroup has to read the d_ifgo[t] of its group,
// 64 rows x 4H (1 MiB for H = 2048): the step is bound by that stream.  Registers cannot hold enough
// of it in flight next to the weights, so the operand blocks travel L2 -> LDS with LDS-direct loads
// into a ring of kRing blocks per wave (nobody else touches a wave's ring: no workgroup barrier, the
// wave waits for its own loads with counted s_waitcnt vmcnt) and reach the MFMA through 16-byte LDS
// reads issued two blocks ahead.  Those reads are inline assembly: the compiler would put
// s_waitcnt vmcnt(0) before every LDS access it knows of while LDS-direct loads are in flight.
#pragma once
#include <type_traits>

#include "recurrent_bwd_xcd.hpp"

namespace fastlstm {

constexpr int kWideRing = 12;   // LDS blocks (1 KiB) per wave for operand blocks in flight (8 and 14: same step time)

// number of k-steps per wave NKW = 4H / KSTEP / 8 (20, 24, 28, 32 for H = 1280, 1536, 1792, 2048)
// NT batch tiles of 16 rows per group: 4, 2 or 1 (see lstm_fwd_wide_kernel; H = 2048, B = 16: 5.9 instead of
// 13.3 us per step)
template <typename T, int NKW, int NT>
__global__ __launch_bounds__(kWave * 8) void lstm_bwd_wide_kernel(const BwdXcdParams p) {
    using E = Elem<T>;
    constexpr bool ACC = E::BYTES == 4;                // fp32: refined reciprocal in the gates
    constexpr int NWV = 8, NTHR = kWave * NWV;
    constexpr int HT = 16, BT = 16 * NT;
    constexpr int IPT = (HT * BT + NTHR - 1) / NTHR;   // (unit, batch row) items per thread
    constexpr int GSEG = HT * E::BYTES;
    constexpr int GROW = 4 * GSEG + 16, SROW = GSEG + 16;
    constexpr int PPSEG = GSEG / 16;
    constexpr int GPIECES = BT * 4 * PPSEG, SPIECES = BT * PPSEG;
    constexpr int IOT = NTHR - kWave;                  // wave 0 polls, the others move the tiles
    constexpr int GPT = (GPIECES + IOT - 1) / IOT, SPT = (SPIECES + IOT - 1) / IOT;
    constexpr int S = kWideRing, NB = NT * NKW;        // ring slots; operand blocks per wave and step
    static_assert(NB % 4 == 0 && S > 4, "fragment registers rotate by 4; the ring is deeper than the read-ahead");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // (uniform: in a scalar register)
    const int q = lane >> 4, r = lane & 15;
    const int KSB = p.KSB, H = p.H, B = p.B, T_ = p.T;

    // ---- placement: group g on XCDs g*xpg .. (hardware deals workgroup i to XCD i % 8) --------
    const int xpg = p.gpx;
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    // several independent recurrences of one shape may share the launch (p.n_layers; NT <= 2), as in the forward kernel
    const int n_rec = NT <= 2 ? max(1, min(p.n_layers, kMaxSideBySide)) : 1;
    const int vg = xcd / xpg, j = (xcd % xpg) * 32 + slot;
    if (vg >= n_rec * p.n_groups || j >= p.n_ht) return;
    const int rec = vg / p.n_groups, g = vg - rec * p.n_groups;
    auto pick = [&](auto a0, auto a1, auto a2, auto a3) {   // (constant indices only, see the forward kernel)
        if constexpr (NT > 2) return a0;
        else return rec == 0 ? a0 : rec == 1 ? a1 : rec == 2 ? a2 : a3;
    };
    check_xcd_placement(p.hdr);
    const int u0 = j * HT, b0 = p.b_base + g * BT;   // b_base: first batch row of this launch

    f32x4 *red = reinterpret_cast<f32x4 *>(smem);                                      // [8][NT][64]
    unsigned char *tiles = reinterpret_cast<unsigned char *>(red + NWV * NT * kWave);   // gates, c, dout tiles
    unsigned char *ring = tiles + BT * GROW + 2 * BT * SROW + (size_t)wave * S * kFragBytes;   // this wave's blocks
    const int io_tid = tid - kWave;

    const T *dout = static_cast<const T *>(pick(p.dout, static_cast<const void *>(p.k5.C), p.dout_more[0], p.dout_more[1]));
    const T *ifgo = static_cast<const T *>(pick(p.ifgo, p.ifgo_lo, p.ifgo_more[0], p.ifgo_more[1]));
    const T *cell = static_cast<const T *>(pick(p.cell, p.cell_lo, p.cell_more[0], p.cell_more[1]));
    T *d_ifgo = static_cast<T *>(pick(p.d_ifgo, p.d_ifgo_lo, p.d_ifgo_more[0], p.d_ifgo_more[1]));
    const T *Wh = static_cast<const T *>(pick(p.Wh, p.Wh_lo, p.Wh_more[0], p.Wh_more[1]));
    T *dh_state = static_cast<T *>(pick(p.dh, p.dh_lo, p.dh_more[0], p.dh_more[1]));
    T *dc_state_buf = static_cast<T *>(pick(p.dc, p.dc_lo, p.dc_more[0], p.dc_more[1]));

    // ---- prologue: this wave's fragments of Wh[:, units]^T, gathered from global memory ----
    // fragment k-step ks = wave + 8 ki: lane (q, r) holds row r = unit u0 + r and
    // k = ks*KSTEP + q*EPL + e, e < EPL, with k = 4 * source unit + gate
    u32x4 wreg[NKW];
#pragma unroll
    for (int ki = 0; ki < NKW; ++ki) {
        const int ks = wave + NWV * ki;
        T tmp[E::EPL];
#pragma unroll
        for (int e = 0; e < E::EPL; ++e) {
            const int k = ks * E::KSTEP + q * E::EPL + e;
            tmp[e] = Wh[((size_t)(k & 3) * H + (k >> 2)) * H + u0 + r];
        }
        wreg[ki] = *reinterpret_cast<u32x4 *>(tmp);
    }

    // ---- per-thread items: it = tid + NTHR*m -> (row n, unit ul, n-tile nt) ----------------
    float dc_state[IPT], dh_rec[IPT], c1v[IPT];
    size_t off_h[IPT];
    int xoff[IPT], roff[IPT], goff[IPT], soff[IPT];
    bool valid[IPT], pair_lead[IPT];
    const size_t BH = (size_t)B * H, B4H = (size_t)B * 4 * H;
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        const int it = tid + NTHR * m;
        const int n = it & 15, rest = it >> 4;
        const int ul = rest % HT, nt = rest / HT;
        const int unit = u0 + ul, b = b0 + nt * 16 + n;
        valid[m] = nt < NT && b < B;   // (16-row groups: items for half of the threads)
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        xoff[m] = nt * KSB * kFragBytes + frag_offset<T>(n, unit * 4);
        pair_lead[m] = valid[m] && ((ul & 1) == 0);
        roff[m] = ((nt < NT ? nt : 0) * kWave + (ul >> 2) * 16 + n) * 4 + (ul & 3);
        goff[m] = (nt * 16 + n) * GROW + ul * E::BYTES;
        soff[m] = (nt * 16 + n) * SROW + ul * E::BYTES;
        dh_rec[m] = valid[m] ? E::to_f32(dh_state[off_h[m]]) : 0.f;
        dc_state[m] = valid[m] ? E::to_f32(dc_state_buf[off_h[m]]) : 0.f;
        c1v[m] = valid[m] ? E::to_f32(cell[(size_t)T_ * BH + off_h[m]]) : 0.f;
    }

    const unsigned xgrp = (unsigned)vg * NT * KSB * kFragBytes;
    const size_t xslot = (size_t)n_rec * p.n_groups * NT * KSB * kFragBytes;
    int *grp_flags = p.counters + (size_t)vg * kXcdGroupStride;   // one flag per workgroup of the group

    // ---- coalesced tile I/O: ifgo[t], cell[t], dout[t] in, d_ifgo[t] out (two sets in flight) ----
    u32x4 gpre[2][GPT], cpre[2][SPT], dpre[2][SPT];
    unsigned g_glb[GPT], s_glb[SPT];
    int g_lds[GPT], s_lds[SPT];
    bool g_ok[GPT], s_ok[SPT];
#pragma unroll
    for (int i = 0; i < GPT; ++i) {
        const int pc = io_tid + IOT * i;
        const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG);
        const int seg = rem / PPSEG, k = rem % PPSEG;
        g_ok[i] = io_tid >= 0 && pc < GPIECES && b0 + row < B;
        g_lds[i] = g_ok[i] ? row * GROW + seg * GSEG + k * 16 : 0;
        g_glb[i] = (unsigned)((size_t)b0 * 4 * H + u0) +
                   (g_ok[i] ? (unsigned)(row * 4 * H + seg * H + k * (16 / E::BYTES)) : 0u);
    }
#pragma unroll
    for (int i = 0; i < SPT; ++i) {
        const int pc = io_tid + IOT * i;
        const int row = pc / PPSEG, k = pc % PPSEG;
        s_ok[i] = io_tid >= 0 && pc < SPIECES && b0 + row < B;
        s_lds[i] = s_ok[i] ? row * SROW + k * 16 : 0;
        s_glb[i] = (unsigned)((size_t)b0 * H + u0) + (s_ok[i] ? (unsigned)(row * H + k * (16 / E::BYTES)) : 0u);
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
    auto tiles_to_lds = [&](const u32x4(&gp)[GPT], const u32x4(&cp)[SPT], const u32x4(&dp)[SPT]) {
        unsigned char *stc = tiles + BT * GROW, *std_ = stc + BT * SROW;
#pragma unroll
        for (int i = 0; i < GPT; ++i)
            if (g_ok[i]) *reinterpret_cast<u32x4 *>(tiles + g_lds[i]) = gp[i];
#pragma unroll
        for (int i = 0; i < SPT; ++i)
            if (s_ok[i]) {
                *reinterpret_cast<u32x4 *>(stc + s_lds[i]) = cp[i];
                *reinterpret_cast<u32x4 *>(std_ + s_lds[i]) = dp[i];
            }
    };
    auto tile_to_global = [&](int t) {
#pragma unroll
        for (int i = 0; i < GPT; ++i)
            if (g_ok[i])
                *reinterpret_cast<u32x4 *>(d_ifgo + (size_t)t * B4H + g_glb[i]) =
                    *reinterpret_cast<const u32x4 *>(tiles + g_lds[i]);
    };
    fetch_tiles(T_ - 1, gpre[0], cpre[0], dpre[0]);
    if (T_ > 1) fetch_tiles(T_ - 2, gpre[1], cpre[1], dpre[1]);
    tiles_to_lds(gpre[0], cpre[0], dpre[0]);   // step 0 works on the LDS tiles right away
    __syncthreads();

    // operand block b of this wave: batch tile b / NKW, k-step wave + 8 (b % NKW); byte offset in the slot
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto block_off = [&](int b) {
        const int bb = b < NB ? b : NB - 1;   // behind the last block: any block again (fixed wait counts)
        return xgrp + (unsigned)(((bb / NKW) * KSB + wave_u + NWV * (bb % NKW)) * kFragBytes);
    };

    // one reverse step; PAR = s % 2 picks the tile register sets at compile time
    auto step = [&](const int s, auto par) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par)::value;
        const int t = T_ - 1 - s;
        const XchgGlobal xch(p.xbuf + (size_t)(s & 1) * xslot, (unsigned)xslot);

        // ---- point-wise gate backward for this thread's items --------------------------
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            T st_d[4];
            if (valid[m]) {
                T *gl_ = reinterpret_cast<T *>(tiles + goff[m]);   // the item's 4 gates in the LDS tile
                const float si = sigmoidf_<ACC>(E::to_f32(gl_[0]));
                const float sf = sigmoidf_<ACC>(E::to_f32(gl_[HT]));
                const float tg = tanhf_<ACC>(E::to_f32(gl_[2 * HT]));
                const float so = sigmoidf_<ACC>(E::to_f32(gl_[3 * HT]));
                const float tc = tanhf_<ACC>(c1v[m]);
                const float c0 = E::to_f32(*reinterpret_cast<const T *>(tiles + BT * GROW + soff[m]));
                const float dh = dh_rec[m] + E::to_f32(*reinterpret_cast<const T *>(tiles + BT * GROW + BT * SROW + soff[m]));
                const float dc1 = dc_state[m] + dh * so * (1.f - tc * tc);
                const float d_o = dh * tc * so * (1.f - so);
                const float d_f = dc1 * c0 * sf * (1.f - sf);
                const float d_i = dc1 * tg * si * (1.f - si);
                const float d_g = dc1 * si * (1.f - tg * tg);
                dc_state[m] = dc1 * sf;
                c1v[m] = c0;   // c_{t-1} is the next step's c_t
                st_d[0] = E::from_f32(d_i);
                st_d[1] = E::from_f32(d_f);
                st_d[2] = E::from_f32(d_g);
                st_d[3] = E::from_f32(d_o);
                gl_[0] = st_d[0];
                gl_[HT] = st_d[1];
                gl_[2 * HT] = st_d[2];
                gl_[3 * HT] = st_d[3];
            } else {
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) st_d[gt] = E::from_f32(0.f);
            }
            // exchange copy: 4 consecutive k = (unit, gate 0..3), 16 bytes per unit with fp32; with 16-bit
            // elements lanes l and l+16 own units u and u+1 of the same batch row and the even-unit lane
            // writes both (16 bytes, write-through)
            if constexpr (E::BYTES == 4) {
                if (valid[m]) xch.store16(xgrp + xoff[m], *reinterpret_cast<u32x4 *>(st_d));
            } else {
                const u32x2 mine = *reinterpret_cast<u32x2 *>(st_d);
                u32x2 other;
                other[0] = (unsigned)__shfl_down((int)mine[0], 16);
                other[1] = (unsigned)__shfl_down((int)mine[1], 16);
                if (pair_lead[m]) xch.store16(xgrp + xoff[m], u32x4{mine[0], mine[1], other[0], other[1]});
            }
        }
        publish_version(grp_flags + j, s + 1);   // waits for the stores, workgroup barrier, raises the flag
        tile_to_global(t);
        if (s + 2 < T_) fetch_tiles(t - 2, gpre[PAR], cpre[PAR], dpre[PAR]);

        if (wave == 0) wait_versions(grp_flags, p.n_ht, s + 1, p.hdr, p.spin_limit, vg, s);
        __syncthreads();

        // ---- dh_rec(units, rows) = Wh[:, units]^T . d_ifgo[t](rows, :)^T over this wave's k-steps ----
        // Block b goes L2 -> ring slot b % S with an LDS-direct load; its 16-byte fragment is read two
        // blocks ahead of its MFMA; slot b % S is refilled with block b + S right after block b's MFMA.
        f32x4 acc[NT];
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        const unsigned lane_off = (unsigned)lane * 16u;
        auto request = [&](int b) {
            load_block_to_lds_device(xch.rsrc, ring + (b % S) * kFragBytes, lane_off, block_off(b));   // (the slot's address is reused)
        };
#pragma unroll
        for (int b = 0; b < S; ++b) request(b);
        u32x4 fr[4];
        // blocks 0 and 1: everything but the S - 1 resp. S - 2 youngest loads has landed
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S - 1) : "memory");
        fr[0] = lds_read_b128_asm<0>(ring + lane_off);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S - 2) : "memory");
        fr[1] = lds_read_b128_asm<0>(ring + kFragBytes + lane_off);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            // block b + 2 has landed when at most the S - 3 loads behind it are in flight
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S - 3) : "memory");
            fr[(b + 2) & 3] = lds_read_b128_asm<0>(ring + ((b + 2) % S) * kFragBytes + lane_off);
            lds_reads_landed_but<1>(fr[b & 3]);   // all but the read just issued: block b's fragment is here
            acc[b / NKW] = mfma_kstep<T>(wreg[b % NKW], fr[b & 3], acc[b / NKW]);
            request(b + S);                       // its fragment is in a register: the slot is free
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // the refills behind the last block
#pragma unroll
        for (int i = 0; i < NT; ++i) red[(wave * NT + i) * kWave + lane] = acc[i];
        // the tile was drained before the barrier above: the next step's inputs take its place
        if (s + 1 < T_) tiles_to_lds(gpre[PAR ^ 1], cpre[PAR ^ 1], dpre[PAR ^ 1]);
        __syncthreads();
        const float *redf = reinterpret_cast<const float *>(red);
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            float v = redf[roff[m]];
#pragma unroll
            for (int pp = 1; pp < NWV; ++pp) v += redf[roff[m] + pp * NT * kWave * 4];
            dh_rec[m] = v;
        }
        // the next step's publish barrier orders these reads before the next writes to `red`
    };
    for (int s = 0; s < T_; s += 2) {
        step(s, std::integral_constant<int, 0>{});
        if (s + 1 < T_) step(s + 1, std::integral_constant<int, 1>{});
    }

    T *dh_out = dh_state, *dc_out = dc_state_buf;
#pragma unroll
    for (int m = 0; m < IPT; ++m)
        if (valid[m]) {
            dh_out[off_h[m]] = E::from_f32(dh_rec[m]);
            dc_out[off_h[m]] = E::from_f32(dc_state[m]);
        }
}

}  // namespace fastlstm

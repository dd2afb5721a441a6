// Persistent forward kernel for hidden sizes whose W_h does not fit the CUs of one XCD
// (H = 1536, 2048 with 16-bit elements): weight slice in registers, barrier groups of H / 16
// workgroups that span several whole XCDs.
//
// Same mathematics and the same results as lstm_fwd_persistent_kernel (which replaces
// fastlstm/kernels.py:414-663).  The general kernel keeps a workgroup's slice of W_h in LDS, which
// for H = 2048 leaves room for 8 hidden units per CU only: one barrier group of 256 workgroups, each
// of which has to read the h_t of ALL batch rows every step (512 KiB per CU and step for B = 128).
// Here a workgroup of 8 waves holds 16 units x 4 gates x H (256 KiB for H = 2048) in registers, as
// the XCD-local kernel does, so a group needs H / 16 workgroups (128) and the launch has room for two
// groups of up to 64 batch rows: half the operand volume per CU.
//  * placement: group g takes the workgroups of XCDs [g * xpg, (g + 1) * xpg), xpg = H / 16 / 32, so
//    an XCD's L2 only ever holds the exchange data of one group;
//  * exchange: device-scope (write-through) stores into two slots (h_s lives in slot s % 2) and
//    device-scope loads (past the CU's L1, served by the XCD's L2; the 32 CUs of an XCD share one fetch);
//  * barrier: one flag per workgroup, raised with a device-scope store, polled by wave 0 of every
//    member (wait_versions); h_t goes from the LDS tile to the exchange slot in whole 16-byte pieces;
//  * the 8 waves split K eight ways (no wave loads an operand block that another wave of the
//    workgroup loads too); the NT batch tiles of 16 rows are multiplied one after the other, the operand
//    blocks of the next one in flight meanwhile: weights (128 registers), two sets of operand blocks
//    (64) and accumulators (16) stay within 256 registers.
// Requirements (host): 16-bit elements, H = 256 * NKW (1280 ... 2048), groups * xpg <= 8 with xpg = ceil(H / 512).
#pragma once
#include <type_traits>

#include "recurrent_fwd_xcd.hpp"

namespace fastlstm {

// NT batch tiles of 16 rows per group: 4 (64 rows; groups x XCDs-per-group <= 8 limits a launch to 128 rows at
// H = 2048), or 2 or 1 where the batch fits the launch that way: a small batch then spreads over more groups,
// i.e. more CUs, and a CU fetches a half or a quarter of the operand bytes per step (H = 2048, B = 16:
// 3.3 instead of 5.8 us per step).
template <typename T, int NKW, int NT>
__global__ __launch_bounds__(kWave * 8) void lstm_fwd_wide_kernel(const FwdXcdParams p) {
    using E = Elem<T>;
    constexpr bool ACC = E::BYTES == 4;                      // fp32: refined reciprocal in the gates
    constexpr int NWV = 8, NTHR = kWave * NWV;
    constexpr int MT = 4, TILES = MT * NT;                   // unit tiles, batch tiles of 16 rows
    constexpr int IPT = (TILES + NWV - 1) / NWV;             // (tile, lane) items per thread
    constexpr int HT = 4 * MT, BT = 16 * NT;
    constexpr int GSEG = HT * E::BYTES;                      // bytes of one gate segment of a row
    constexpr int GROW = 4 * GSEG + 16, SROW = GSEG + 16;
    constexpr int PPSEG = GSEG / 16;
    constexpr int GPIECES = BT * 4 * PPSEG, SPIECES = BT * PPSEG;
    constexpr int IOT = NTHR - kWave;                        // waves 1.. move the tiles, wave 0 polls
    constexpr int GPT = (GPIECES + IOT - 1) / IOT, SPT = (SPIECES + IOT - 1) / IOT;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // (uniform: in a scalar register)
    const int q = lane >> 4, n = lane & 15;
    const int KS = p.KS, H = p.H, B = p.B, T_ = p.T;
    const bool keep = p.keep != 0;   // training: gate pre-activations and every cell state are stored

    // ---- placement: group g on XCDs g*xpg .. (hardware deals workgroup i to XCD i % 8) --------
    const int xpg = p.gpx;   // XCDs per group
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    // several independent recurrences of one shape may share the launch (p.n_layers; NT <= 2): recurrence r takes the
    // groups r * n_groups ... of the launch, with its own operands, flags and exchange blocks
    const int n_rec = NT <= 2 ? max(1, min(p.n_layers, kMaxSideBySide)) : 1;
    const int vg = xcd / xpg, j = (xcd % xpg) * 32 + slot;
    if (vg >= n_rec * p.n_groups || j >= p.n_ht) return;
    check_xcd_placement(p.hdr);
    const int rec = vg / p.n_groups, g = vg - rec * p.n_groups;
    // (constant indices only: a run-time index into the kernel's arguments would move them all to scratch memory)
    auto pick = [&](auto a0, auto a1, auto a2, auto a3) {
        if constexpr (NT > 2) return a0;
        else return rec == 0 ? a0 : rec == 1 ? a1 : rec == 2 ? a2 : a3;
    };
    const int u0 = j * HT, b0 = p.b_base + g * BT;   // b_base: first batch row of this launch

    f32x4 *red = reinterpret_cast<f32x4 *>(smem);                                       // [8][TILES][64]
    unsigned char *tiles = reinterpret_cast<unsigned char *>(red + NWV * TILES * kWave);   // gates, h, c tiles
    const int io_tid = tid - kWave;

    T *ifgo = static_cast<T *>(pick(p.ifgo, p.ifgo2, p.ifgo_more[0], p.ifgo_more[1]));
    T *out = static_cast<T *>(pick(p.out, p.out2, p.out_more[0], p.out_more[1]));
    T *cell = static_cast<T *>(pick(p.cell, p.cell2, p.cell_more[0], p.cell_more[1]));
    const T *Wh = static_cast<const T *>(pick(p.Wh, p.Wh2, p.Wh_more[0], p.Wh_more[1]));

    // ---- prologue 1: this wave's fragments of the W_h slice, global -> registers ---------
    // fragment (m-tile a, k-step ks = wave + 8 ki): lane (q, r) holds row r = (unit a*4 + r/4, gate r%4),
    // k = ks*KSTEP + q*EPL .. + EPL-1, i.e. 16 contiguous bytes of W_h
    u32x4 wreg[MT][NKW];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int ki = 0; ki < NKW; ++ki) {
            const int ks = wave + NWV * ki;
            const int unit = u0 + a * 4 + (n >> 2), gate = n & 3;
            const int k0 = ks * E::KSTEP + q * E::EPL;
            wreg[a][ki] = *reinterpret_cast<const u32x4 *>(Wh + ((size_t)gate * H + unit) * H + k0);
        }

    // ---- per-thread items: (tile = wave + 8m, lane) -> (unit, batch row) -------------
    float c_state[IPT];
    size_t off_h[IPT];
    int xoff[IPT], goff[IPT], soff[IPT];   // xoff: prologue only
    bool valid[IPT];
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        const int tile = wave + NWV * m;
        const int mt = tile / NT, nt = tile % NT;
        const int unit = u0 + mt * 4 + q, b = b0 + nt * 16 + n;
        valid[m] = tile < TILES && b < B;
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        xoff[m] = nt * KS * kFragBytes + frag_offset<T>(n, unit);
        goff[m] = (nt * 16 + n) * GROW + (mt * 4 + q) * E::BYTES;
        soff[m] = (nt * 16 + n) * SROW + (mt * 4 + q) * E::BYTES;
        c_state[m] = valid[m] ? E::to_f32(cell[off_h[m]]) : 0.f;
    }

    // two exchange slots: h_s lives in slot s % 2
    const unsigned xgrp = (unsigned)vg * NT * KS * kFragBytes;
    const size_t xslot = (size_t)n_rec * p.n_groups * NT * KS * kFragBytes;
    int *grp_flags = p.counters + (size_t)vg * kXcdGroupStride;   // n_ht <= kXcdGroupStride flags per group
    auto publish = [&](int version) { publish_version(grp_flags + j, version); };

    // ---- prologue 2: publish h_0 (slot 0) as version 1 -------------------------------------
    {
        const XchgGlobal x0(p.xbuf, (unsigned)xslot);
#pragma unroll
        for (int m = 0; m < IPT; ++m)
            if (valid[m]) x0.store_elem(xgrp + xoff[m], out[off_h[m]]);
        publish(1);
    }

    const size_t B4H = (size_t)B * 4 * H, BH = (size_t)B * H;

    // ---- coalesced tile I/O (see lstm_fwd_persistent_kernel) --------------------------------
    // The gates tile of a step (x_t.Wx^T + b, BT rows x 4 gates x 16 units) travels global -> LDS tile with
    // LDS-direct loads, a step ahead of its use, by waves 1..7: no register holds it meanwhile.  (Held in
    // registers next to the 128 weight registers and two sets of operand blocks it was spilled right behind
    // its load, and the spill waited for the load: a memory round trip on every step's critical path,
    // 9.1 instead of 6.9 us per step at H = 2048.)  A tile row is GROW = 4 * GSEG + 16 bytes = 9 slots of 16
    // bytes, so lane l of wave instruction i fills slot 64 i + l; the pad slot of a row and rows past B stay
    // untouched (lanes switched off).
    constexpr int SPR = GROW / 16, SLOTS = BT * SPR;       // slots per row, per tile
    constexpr int DMA_N = (SLOTS + kWave - 1) / kWave;     // wave instructions per tile
    constexpr int DPW = (DMA_N + NWV - 2) / (NWV - 1);     // per moving wave
    const size_t tile_org = (size_t)b0 * 4 * H + u0;
    unsigned dma_off[DPW];
    bool dma_ok[DPW];
#pragma unroll
    for (int d = 0; d < DPW; ++d) {
        const int i = (wave - 1) + (NWV - 1) * d, sl = i * kWave + lane;
        const int row = sl / SPR, idx = sl % SPR;
        dma_ok[d] = wave >= 1 && i < DMA_N && sl < SLOTS && idx < 4 * PPSEG && b0 + row < B;
        dma_off[d] = dma_ok[d] ? (unsigned)(((size_t)row * 4 * H + (size_t)(idx / PPSEG) * H + (idx % PPSEG) * (16 / E::BYTES)) * E::BYTES) : 0u;
    }
    auto request_tile = [&](int t) {
        if (t >= T_) return;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<T *>(ifgo) + (size_t)t * B4H + tile_org, 0, (unsigned)((size_t)BT * 4 * H * E::BYTES), 0x00020000);
#pragma unroll
        for (int d = 0; d < DPW; ++d)
            if (dma_ok[d]) load_block_to_lds(rs, tiles + (size_t)((wave - 1) + (NWV - 1) * d) * kFragBytes, dma_off[d], 0);
    };
    // LDS tiles -> ifgo[t], out[t+1], cell[t+1]: buffer stores with a per-step base in scalar registers and per-lane
    // byte offsets that never change (the gates tile slot by slot, as it came in; the state tiles in 16-byte pieces)
    unsigned st_off[SPT];
    int st_lds[SPT];
    bool st_ok[SPT];
#pragma unroll
    for (int i = 0; i < SPT; ++i) {
        const int pc = io_tid + IOT * i;
        const int row = pc / PPSEG, k = pc % PPSEG;
        st_ok[i] = io_tid >= 0 && pc < SPIECES && b0 + row < B;
        st_off[i] = st_ok[i] ? (unsigned)(((size_t)row * H + k * (16 / E::BYTES)) * E::BYTES) : 0u;
        st_lds[i] = st_ok[i] ? row * SROW + k * 16 : 0;
    }
    const size_t state_org = (size_t)b0 * H + u0;
    auto tiles_to_global = [&](int t, const unsigned char *gt) {
        const unsigned char *sth = gt + BT * GROW, *stc = sth + BT * SROW;
        if (keep) {
            const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(
                ifgo + (size_t)t * B4H + tile_org, 0, (unsigned)((size_t)BT * 4 * H * E::BYTES), 0x00020000);
#pragma unroll
            for (int d = 0; d < DPW; ++d)
                if (dma_ok[d])
                    __builtin_amdgcn_raw_buffer_store_b128(
                        *reinterpret_cast<const u32x4 *>(gt + (size_t)((wave - 1) + (NWV - 1) * d) * kFragBytes + lane * 16), rg,
                        dma_off[d], 0, 0);
        }
        const unsigned sbytes = (unsigned)((size_t)BT * H * E::BYTES);
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(out + (size_t)(t + 1) * BH + state_org, 0, sbytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(cell + (size_t)(t + 1) * BH + state_org, 0, sbytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < SPT; ++i)
            if (st_ok[i]) {
                __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(sth + st_lds[i]), rh, st_off[i], 0, 0);
                if (keep || t + 1 == T_)
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(stc + st_lds[i]), rc, st_off[i], 0, 0);
            }
    };
    request_tile(0);

    auto step = [&](const int t) __attribute__((always_inline)) {
        unsigned char *gt = tiles;
        if (wave == 0) wait_versions(grp_flags, p.n_ht, t + 1, p.hdr, p.spin_limit, vg, t);
        __syncthreads();

        // ---- partial(a, i) = Wslice(a, this wave's k-steps) . h_{t-1}(i)^T, one batch tile i per pass.
        // The operand blocks of pass i + 1 are requested before pass i is multiplied (two register
        // sets): one exposed round trip per step, the others hide behind the MFMAs.
        const XchgGlobal xr(p.xbuf + (size_t)(t & 1) * xslot, (unsigned)xslot);
        u32x4 bq[2][NKW];
        auto request = [&](auto ic) __attribute__((always_inline)) {
            constexpr int i = decltype(ic)::value;
#pragma unroll
            for (int ki = 0; ki < NKW; ++ki)   // device-scope loads: the slot's address is reused every other step
                bq[i & 1][ki] = xr.template load16<true>(xgrp + (unsigned)((i * KS + wave + NWV * ki) * kWave + lane) * 16u);
        };
        auto pass = [&](auto ic) __attribute__((always_inline)) {
            constexpr int i = decltype(ic)::value;
            if constexpr (i + 1 < NT) request(std::integral_constant<int, i + 1>{});
            __builtin_amdgcn_sched_barrier(0);   // the next pass's loads are issued before this pass's first MFMA
            f32x4 acc[MT];
#pragma unroll
            for (int a = 0; a < MT; ++a) acc[a] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ki = 0; ki < NKW; ++ki)
#pragma unroll
                for (int a = 0; a < MT; ++a) acc[a] = mfma_kstep<T>(wreg[a][ki], bq[i & 1][ki], acc[a]);
#pragma unroll
            for (int a = 0; a < MT; ++a) red[(wave * TILES + a * NT + i) * kWave + lane] = acc[a];
            __builtin_amdgcn_sched_barrier(0);
        };
        request(std::integral_constant<int, 0>{});
        static_for<0, NT>(pass);
        __syncthreads();   // (the gates tile of this step was requested a step ago: the compiler's wait for it, before
                           // the first LDS access behind the request, fell in the first multiplication pass)

        // ---- every (tile, lane) item sums the 8 partials and applies the gates -------------------
        const XchgGlobal xw(p.xbuf + (size_t)((t + 1) & 1) * xslot, (unsigned)xslot);
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const int tile = wave + NWV * m;
            if (tile >= TILES) continue;   // (16-row groups: four tiles for eight waves)
            f32x4 s = red[tile * kWave + lane];
#pragma unroll
            for (int pp = 1; pp < NWV; ++pp) s += red[(pp * TILES + tile) * kWave + lane];
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
                gl_[0] = E::from_f32(pi);
                gl_[HT] = E::from_f32(pf);
                gl_[2 * HT] = E::from_f32(pg);
                gl_[3 * HT] = E::from_f32(po);
                *reinterpret_cast<T *>(gt + BT * GROW + soff[m]) = hv;
                *reinterpret_cast<T *>(gt + BT * GROW + BT * SROW + soff[m]) = E::from_f32(c1);
            }
        }
        __syncthreads();   // the h tile is complete in LDS
        if (t + 1 < T_) {
            // h_t to the exchange slot in 16-byte pieces (8 consecutive units of one batch row are 16
            // contiguous bytes of an operand block): write-through stores of whole pieces, not of elements
            const unsigned char *sth = gt + BT * GROW;
            for (int pc = io_tid; io_tid >= 0 && pc < BT * PPSEG; pc += IOT) {
                const int row = pc / PPSEG, c = pc % PPSEG;
                if (b0 + row < B)
                    xw.store16(xgrp + (unsigned)((row >> 4) * KS * kFragBytes + frag_offset<T>(row & 15, u0 + c * E::EPL)),
                               *reinterpret_cast<const u32x4 *>(sth + row * SROW + c * 16));
            }
            publish(t + 2);
        }
        tiles_to_global(t, gt);
        // the stores are acknowledged while the workgroup would wait for its peers anyway; the tile
        // requests below and the next step's operand requests then queue behind nothing (measured: 0.2-0.3 us
        // per step at H = 2048)
        if (keep) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // the stores above have their data (the tile's rows were read out of LDS): the next step's gates may land there
        request_tile(t + 1);
    };
    for (int t = 0; t < T_; ++t) step(t);
}

}  // namespace fastlstm

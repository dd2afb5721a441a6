// Persistent forward / reverse kernels for hidden sizes whose W_h does not fit on chip: the weight slice
// of a workgroup is STREAMED from memory every timestep instead of staying resident.
//
// The reference does the same above H = 64 (fp32) / 128 (16-bit): RELOAD_WEIGHTS, fastlstm/lstm.py:70-72,
// fastlstm/kernels.py:464, 550-626 (forward) and 1362-1383 (reverse, always).  Here the resident kernels
// cover everything up to 32 MiB of W_h (H = 2048 in 16 bits, 1024 in fp32); these kernels take over beyond
// that, so that no hidden size is refused.  Mathematics, stored values and rounding points are those of
// lstm_fwd_persistent_kernel / lstm_bwd_persistent_kernel.
//
// What bounds a step here is the stream itself: all of W_h (4H x H elements) crosses the memory system once
// per timestep and direction (H = 4096 in fp16: 128 MiB, 16 us at 8 TB/s), so the design keeps that stream
// clean and everything else small:
//  * a pack kernel writes W_h once per call into MFMA operand order (1 KiB blocks, zero padded), slice by
//    slice, so that a wave's loads are full, contiguous 1 KiB blocks;
//  * one workgroup per slice of `HT` hidden units and ALL batch rows of the launch it can hold (up to 64):
//    the weights are read once per step, not once per batch tile;
//  * the 4 waves split K; every wave keeps two chunks of weight and operand blocks in flight;
//  * h_t / d_ifgo[t] travel through a two-slot exchange buffer with write-through stores, device-scope loads
//    and one flag per workgroup (recurrent_common.hpp).  (Measured alternative: invalidating the
//    non-coherent cache lines once per step with `buffer_inv sc1` and reading the exchange data through the
//    caches, one fetch per XCD instead of one per CU, is slower: 32.7 instead of 26.4 us per step at
//    H = 4096, B = 64 in fp16.)
#pragma once
#include <type_traits>

#include "recurrent_common.hpp"

namespace fastlstm {

constexpr int kStreamCK = 2;                 // k-steps per chunk of loads
constexpr int kStreamKPad = 4 * kStreamCK * 2;   // k-steps are padded to a multiple of this: no branch in the K loop

struct FwdStreamParams {
    void *ifgo;        // [T,B,4H]
    void *out, *cell;  // [T+1,B,H]
    const unsigned char *wpack;   // [n_ht][MT][KSP] operand blocks, rows (unit, gate), zero past H
    WsHeader *hdr;
    int *flags;        // [n_bt][flag_stride]
    unsigned char *xbuf;   // [2 slots][n_bt][NT][KSP] operand blocks
    int T, B, H;
    int b_base, n_bt, n_ht, flag_stride;
    int KS, KSP;       // k-steps covering H, padded
    int keep;
    long long spin_limit;
};

struct BwdStreamParams {
    const void *dout;   // [T,B,H]
    void *dh, *dc;      // [B,H]
    const void *ifgo, *cell;
    void *d_ifgo;
    const unsigned char *wpack;   // [n_ht][MTB][KSBP] operand blocks of Wh[:, units]^T, K = (unit', gate)
    WsHeader *hdr;
    int *flags;
    unsigned char *xbuf;   // [2 slots][n_bt][NT][KSBP]
    int T, B, H;
    int b_base, n_bt, n_ht, flag_stride;
    int KSB, KSBP;
    long long spin_limit;
};

// ---- packing: W_h -> operand blocks, once per call -----------------------------------------------
// forward: block (j, a, ks), lane (q, r): row r = (unit j*4*MT + a*4 + r/4, gate r%4), k = ks*KSTEP + q*EPL ..
template <typename T>
__global__ void pack_wh_fwd_kernel(const T *Wh, unsigned char *wpack, int H, int KS, int KSP, int MT, int n_ht) {
    using E = Elem<T>;
    const size_t total = (size_t)n_ht * MT * KSP * kWave;
    for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
        const int lane = (int)(idx % kWave);
        const size_t blk = idx / kWave;
        const int ks = (int)(blk % KSP), a = (int)((blk / KSP) % MT), j = (int)(blk / ((size_t)KSP * MT));
        const int q = lane >> 4, r = lane & 15;
        const int unit = (j * MT + a) * 4 + (r >> 2), gate = r & 3;
        const int k0 = ks * E::KSTEP + q * E::EPL;
        T tmp[E::EPL];
#pragma unroll
        for (int e = 0; e < E::EPL; ++e)
            tmp[e] = (ks < KS && unit < H && k0 + e < H) ? Wh[((size_t)gate * H + unit) * H + k0 + e] : E::from_f32(0.f);
        *reinterpret_cast<u32x4 *>(wpack + idx * 16) = *reinterpret_cast<u32x4 *>(tmp);
    }
}
// reverse: block (j, mt, ks), lane (q, r): row r = unit j*16*MTB + mt*16 + r, k = ks*KSTEP + q*EPL + e = 4*unit' + gate
template <typename T>
__global__ void pack_wh_bwd_kernel(const T *Wh, unsigned char *wpack, int H, int KSB, int KSBP, int MTB, int n_ht) {
    using E = Elem<T>;
    const size_t total = (size_t)n_ht * MTB * KSBP * kWave;
    for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
        const int lane = (int)(idx % kWave);
        const size_t blk = idx / kWave;
        const int ks = (int)(blk % KSBP), mt = (int)((blk / KSBP) % MTB), j = (int)(blk / ((size_t)KSBP * MTB));
        const int q = lane >> 4, r = lane & 15;
        const int unit = (j * MTB + mt) * 16 + r;
        T tmp[E::EPL];
#pragma unroll
        for (int e = 0; e < E::EPL; ++e) {
            const int k = ks * E::KSTEP + q * E::EPL + e, uk = k >> 2, gate = k & 3;
            tmp[e] = (ks < KSB && unit < H && uk < H) ? Wh[((size_t)gate * H + uk) * H + unit] : E::from_f32(0.f);
        }
        *reinterpret_cast<u32x4 *>(wpack + idx * 16) = *reinterpret_cast<u32x4 *>(tmp);
    }
}

// acc[a][i] += A(a, ks) . B(i, ks) over the calling wave's k-steps ks = wave, wave + 4, ... < KSP.
// A blocks come from `wp` (this workgroup's slice, [MT][KSP] blocks), B blocks from the exchange slot `xb`
// ([NT][KSP] blocks).  KSP is a multiple of kStreamKPad, so every wave runs the same, branch-free schedule:
// two chunks of kStreamCK k-steps in flight.  Blocks past KS hold zero weights; their operand loads are
// clamped to the last real block.
template <typename T, int MT, int NT>
__device__ __forceinline__ void stream_kloop(f32x4 (&acc)[MT][NT], const unsigned char *wp, const XchgGlobal &xch,
                                             unsigned xb, int KS, int KSP, int wave, int lane) {
    constexpr int CK = kStreamCK;
    const int nchunks = KSP / (4 * CK);   // even
    auto load = [&](u32x4(&a)[CK][MT], u32x4(&b)[CK][NT], int c) {
#pragma unroll
        for (int cc = 0; cc < CK; ++cc) {
            const int ks = wave + 4 * (c * CK + cc);
            const int kb = min(ks, KS - 1);
#pragma unroll
            for (int m = 0; m < MT; ++m)
                a[cc][m] = *reinterpret_cast<const u32x4 *>(wp + ((size_t)(m * KSP + ks) * kWave + lane) * 16);
#pragma unroll
            for (int i = 0; i < NT; ++i) b[cc][i] = xch.template load16<true>(xb + (unsigned)((i * KSP + kb) * kWave + lane) * 16u);
        }
    };
    auto compute = [&](const u32x4(&a)[CK][MT], const u32x4(&b)[CK][NT]) {
#pragma unroll
        for (int cc = 0; cc < CK; ++cc)
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int i = 0; i < NT; ++i) acc[m][i] = mfma_kstep<T>(a[cc][m], b[cc][i], acc[m][i]);
    };
    u32x4 aA[CK][MT], bA[CK][NT], aB[CK][MT], bB[CK][NT];
    load(aA, bA, 0);
    for (int c = 0; c < nchunks; c += 2) {
        load(aB, bB, c + 1);
        compute(aA, bA);
        if (c + 2 < nchunks) load(aA, bA, c + 2);
        compute(aB, bB);
    }
}

// One workgroup (4 waves): HT = 4*MT hidden units x BT = 16*NT batch rows x 4 gates; MT*NT <= 16 tiles.
template <typename T, int MT, int NT>
__global__ __launch_bounds__(kThreads) void lstm_fwd_stream_kernel(const FwdStreamParams p) {
    using E = Elem<T>;
    constexpr bool ACC = (E::DT == FASTLSTM_FP32);
    constexpr int TILES = MT * NT, IPT = (TILES + 3) / 4;
    constexpr int HT = 4 * MT, BT = 16 * NT;
    static_assert(TILES <= 16, "at most 16 output tiles per workgroup");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    f32x4 *red = reinterpret_cast<f32x4 *>(smem);   // [4][TILES][64]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane >> 4, n = lane & 15;
    const int KS = p.KS, KSP = p.KSP, H = p.H, B = p.B, T_ = p.T;
    const bool keep = p.keep != 0;
    const int lin = xcd_major_id(blockIdx.x, gridDim.x);
    const int g = lin / p.n_ht, j = lin % p.n_ht;
    const int u0 = j * HT, b0 = p.b_base + g * BT;
    T *ifgo = static_cast<T *>(p.ifgo);
    T *out = static_cast<T *>(p.out);
    T *cell = static_cast<T *>(p.cell);
    const unsigned char *wp = p.wpack + (size_t)j * MT * KSP * kFragBytes;

    float c_state[IPT];
    size_t off_h[IPT], off_p[IPT];
    int xoff[IPT];
    bool valid[IPT];
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        const int tl = wave + 4 * m, mt = tl / NT, nt = tl % NT;
        const int unit = u0 + mt * 4 + q, b = b0 + nt * 16 + n;
        valid[m] = tl < TILES && unit < H && b < B;
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        off_p[m] = valid[m] ? (size_t)b * 4 * H + unit : (size_t)b0 * 4 * H + u0;
        xoff[m] = nt * KSP * kFragBytes + frag_offset<T>(n, unit);
        c_state[m] = valid[m] ? E::to_f32(cell[off_h[m]]) : 0.f;
    }
    const unsigned xslot = (unsigned)p.n_bt * NT * KSP * kFragBytes;
    const unsigned xgrp = (unsigned)g * NT * KSP * kFragBytes;
    const XchgGlobal xch(p.xbuf, 2u * xslot);
    int *my_flag = p.flags + (size_t)g * p.flag_stride + j;
    const int *grp_flags = p.flags + (size_t)g * p.flag_stride;

    // h_0 is version 1 in slot 0
#pragma unroll
    for (int m = 0; m < IPT; ++m)
        if (valid[m]) xch.store_elem(xgrp + xoff[m], out[off_h[m]]);
    publish_version(my_flag, 1);

    const size_t BH = (size_t)B * H, B4H = (size_t)B * 4 * H;
    // the input projection of a step does not depend on the recurrence: requested two steps ahead
    // (unconditional loads: invalid items read the tile origin)
    T pre[2][IPT][4];
    auto fetch_pre = [&](int t, T(&dst)[IPT][4]) {
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const T *src = ifgo + (size_t)t * B4H + off_p[m];
#pragma unroll
            for (int gt = 0; gt < 4; ++gt) dst[m][gt] = src[(size_t)gt * H];
        }
    };
    fetch_pre(0, pre[0]);
    if (T_ > 1) fetch_pre(1, pre[1]);

    auto step = [&](const int t, auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        const unsigned xb = xgrp + (unsigned)(t & 1) * xslot, xn = xgrp + (unsigned)((t + 1) & 1) * xslot;
        if (wave == 0) wait_versions(grp_flags, p.n_ht, t + 1, p.hdr, p.spin_limit, g, t);
        __syncthreads();
        f32x4 acc[MT][NT];
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int i = 0; i < NT; ++i) acc[a][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        stream_kloop<T, MT, NT>(acc, wp, xch, xb, KS, KSP, wave, lane);
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int i = 0; i < NT; ++i) red[(wave * TILES + a * NT + i) * kWave + lane] = acc[a][i];
        __syncthreads();
        T st_p[IPT][4], st_h[IPT], st_c[IPT];
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const int tl = wave + 4 * m;
            if (tl < TILES) {
                f32x4 s = red[tl * kWave + lane];
#pragma unroll
                for (int pp = 1; pp < 4; ++pp) s += red[(pp * TILES + tl) * kWave + lane];
                if (valid[m]) {
                    const float pi = E::to_f32(pre[u][m][0]) + s[0];
                    const float pf = E::to_f32(pre[u][m][1]) + s[1];
                    const float pg = E::to_f32(pre[u][m][2]) + s[2];
                    const float po = E::to_f32(pre[u][m][3]) + s[3];
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
                }
            }
        }
        if (t + 1 < T_) publish_version(my_flag, t + 2);   // (its barrier also orders the reads of `red` before the next step's writes)
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
        if (t + 2 < T_) fetch_pre(t + 2, pre[u]);
    };
    for (int t0 = 0; t0 < T_; t0 += 2) {
        step(t0, std::integral_constant<int, 0>{});
        if (t0 + 1 < T_) step(t0 + 1, std::integral_constant<int, 1>{});
    }
}

// One workgroup (4 waves): HT = 16*MTB hidden units x BT = 16*NT batch rows; MTB*NT <= 4 output tiles
// (each thread owns MTB*NT (unit, row) items: tile m, unit tid/16, row tid%16).
template <typename T, int MTB, int NT>
__global__ __launch_bounds__(kThreads) void lstm_bwd_stream_kernel(const BwdStreamParams p) {
    using E = Elem<T>;
    constexpr bool ACC = (E::DT == FASTLSTM_FP32);
    constexpr int TILES = MTB * NT, IPT = TILES;
    constexpr int HT = 16 * MTB, BT = 16 * NT;
    static_assert(TILES <= 4, "at most 4 output tiles per workgroup");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    f32x4 *red = reinterpret_cast<f32x4 *>(smem);   // [4][TILES][64]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int KSB = p.KSB, KSBP = p.KSBP, H = p.H, B = p.B, T_ = p.T;
    const int lin = xcd_major_id(blockIdx.x, gridDim.x);
    const int g = lin / p.n_ht, j = lin % p.n_ht;
    const int u0 = j * HT, b0 = p.b_base + g * BT;
    const T *dout = static_cast<const T *>(p.dout);
    const T *ifgo = static_cast<const T *>(p.ifgo);
    const T *cell = static_cast<const T *>(p.cell);
    T *d_ifgo = static_cast<T *>(p.d_ifgo);
    const unsigned char *wp = p.wpack + (size_t)j * MTB * KSBP * kFragBytes;

    // item m of a thread: output tile m = (unit tile mt, batch tile nt), unit row ur = tid / 16, batch row n = tid % 16.
    // The product of a step leaves tile (mt, nt) in MFMA layout: lane (q', n) holds units 4q' .. 4q'+3 of row n.
    float dc_state[IPT], dh_rec[IPT], c1v[IPT];
    size_t off_h[IPT], off_p[IPT];
    int xoff[IPT], roff[IPT];
    bool valid[IPT];
    const size_t BH = (size_t)B * H, B4H = (size_t)B * 4 * H;
    const int n = tid & 15, ur = tid >> 4;
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        const int mt = m / NT, nt = m % NT;
        const int unit = u0 + mt * 16 + ur, b = b0 + nt * 16 + n;
        valid[m] = unit < H && b < B;
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        off_p[m] = valid[m] ? (size_t)b * 4 * H + unit : (size_t)b0 * 4 * H + u0;
        xoff[m] = nt * KSBP * kFragBytes + frag_offset<T>(n, unit * 4);
        roff[m] = ((m * kWave) + (ur >> 2) * 16 + n) * 4 + (ur & 3);   // float index inside one partial-sum set
        dh_rec[m] = valid[m] ? E::to_f32(static_cast<const T *>(p.dh)[off_h[m]]) : 0.f;
        dc_state[m] = valid[m] ? E::to_f32(static_cast<const T *>(p.dc)[off_h[m]]) : 0.f;
        c1v[m] = valid[m] ? E::to_f32(cell[(size_t)T_ * BH + off_h[m]]) : 0.f;
    }
    const unsigned xslot = (unsigned)p.n_bt * NT * KSBP * kFragBytes;
    const unsigned xgrp = (unsigned)g * NT * KSBP * kFragBytes;
    const XchgGlobal xch(p.xbuf, 2u * xslot);
    int *my_flag = p.flags + (size_t)g * p.flag_stride + j;
    const int *grp_flags = p.flags + (size_t)g * p.flag_stride;

    T pre[2][IPT][4], c0r[2][IPT], dor[2][IPT];
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
    fetch(T_ - 1, pre[0], c0r[0], dor[0]);
    if (T_ > 1) fetch(T_ - 2, pre[1], c0r[1], dor[1]);

    auto step = [&](const int s, auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        const int t = T_ - 1 - s;
        const unsigned xw = xgrp + (unsigned)(s & 1) * xslot;
        T st_d[IPT][4];
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            if (valid[m]) {
                const float si = sigmoidf_<ACC>(E::to_f32(pre[u][m][0]));
                const float sf = sigmoidf_<ACC>(E::to_f32(pre[u][m][1]));
                const float tg = tanhf_<ACC>(E::to_f32(pre[u][m][2]));
                const float so = sigmoidf_<ACC>(E::to_f32(pre[u][m][3]));
                const float tc = tanhf_<ACC>(c1v[m]);
                const float c0 = E::to_f32(c0r[u][m]);
                const float dh = dh_rec[m] + E::to_f32(dor[u][m]);
                const float dc1 = dc_state[m] + dh * so * (1.f - tc * tc);
                const float d_o = dh * tc * so * (1.f - so);
                const float d_f = dc1 * c0 * sf * (1.f - sf);
                const float d_i = dc1 * tg * si * (1.f - si);
                const float d_g = dc1 * si * (1.f - tg * tg);
                dc_state[m] = dc1 * sf;
                c1v[m] = c0;
                st_d[m][0] = E::from_f32(d_i);
                st_d[m][1] = E::from_f32(d_f);
                st_d[m][2] = E::from_f32(d_g);
                st_d[m][3] = E::from_f32(d_o);
                // exchange copy: 4 consecutive k = (unit, gate 0..3)
                if constexpr (E::BYTES == 2) xch.store8(xw + xoff[m], *reinterpret_cast<u32x2 *>(st_d[m]));
                else xch.store16(xw + xoff[m], *reinterpret_cast<u32x4 *>(st_d[m]));
            }
        }
        publish_version(my_flag, s + 1);
#pragma unroll
        for (int m = 0; m < IPT; ++m)
            if (valid[m]) {
                T *dst = d_ifgo + (size_t)t * B4H + off_p[m];
                dst[0] = st_d[m][0];
                dst[(size_t)H] = st_d[m][1];
                dst[(size_t)2 * H] = st_d[m][2];
                dst[(size_t)3 * H] = st_d[m][3];
            }
        if (s + 2 < T_) fetch(T_ - 3 - s, pre[u], c0r[u], dor[u]);
        if (wave == 0) wait_versions(grp_flags, p.n_ht, s + 1, p.hdr, p.spin_limit, g, s);
        __syncthreads();
        f32x4 acc[MTB][NT];
#pragma unroll
        for (int a = 0; a < MTB; ++a)
#pragma unroll
            for (int i = 0; i < NT; ++i) acc[a][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        stream_kloop<T, MTB, NT>(acc, wp, xch, xw, KSB, KSBP, wave, lane);
#pragma unroll
        for (int a = 0; a < MTB; ++a)
#pragma unroll
            for (int i = 0; i < NT; ++i) red[(wave * TILES + a * NT + i) * kWave + lane] = acc[a][i];
        __syncthreads();
        const float *redf = reinterpret_cast<const float *>(red);
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            float v = redf[roff[m]];
#pragma unroll
            for (int pp = 1; pp < 4; ++pp) v += redf[roff[m] + pp * TILES * kWave * 4];
            dh_rec[m] = v;
        }
        // (the next step's publish barrier orders these reads before the next writes to `red`)
    };
    for (int s0 = 0; s0 < T_; s0 += 2) {
        step(s0, std::integral_constant<int, 0>{});
        if (s0 + 1 < T_) step(s0 + 1, std::integral_constant<int, 1>{});
    }
    T *dh_out = static_cast<T *>(p.dh), *dc_out = static_cast<T *>(p.dc);
#pragma unroll
    for (int m = 0; m < IPT; ++m)
        if (valid[m]) {
            dh_out[off_h[m]] = E::from_f32(dh_rec[m]);
            dc_out[off_h[m]] = E::from_f32(dc_state[m]);
        }
}

}  // namespace fastlstm

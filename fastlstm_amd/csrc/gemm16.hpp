// High-throughput MFMA GEMM for the 16-bit element types (fp16 / bf16, fp32 accumulate):
//     C[m][n] = sum_k A(m,k) * B(n,k)   [+ bias0[n] + bias1[n]]
// the same contraction as gemm.hpp's generic kernel, restricted to the aligned case
// (K a multiple of 64, leading dimensions multiples of 8 elements, operands < 4 GiB)
// that every BASELINE configuration of the LSTM hits.
//
// Design for gfx950
//  * BM x BN x 64 workgroup tile (256 x 256 for large problems), 4 waves in 2 x 2, each
//    wave BM/2 x BN/2 as MFMA 16x16x32 tiles -> up to 256 fp32 accumulators per lane;
//    one LDS byte feeds 128 MACs, so LDS reads run at half the MFMA rate.
//  * K-contiguous operands are stored in LDS directly in MFMA operand order: a fragment is
//    one linear, conflict-free ds_read_b128.
//  * K-major operands (d_ifgo, x and h in the weight-gradient products) stay in memory order
//    in LDS and are transposed on the way to the registers by gfx950's ds_read_b64_tr_b16:
//    within 16 lanes, lane (a, b) supplies the address of 4 consecutive m of k-row a, and
//    lane i receives element i of the 4 rows.  No transposed copy is ever written.
//  * Tiles travel HBM -> LDS with gfx950's 16-byte LDS-direct buffer loads
//    (buffer_load_dwordx4 ... lds): no staging registers, no ds_write instructions; lane l
//    of a wave instruction fills bytes [16 l, 16 l + 16) of a 1 KiB LDS block, and which
//    global chunk a lane fetches is chosen so that the block comes out in the wanted order
//    (operand order, or k-rows with an XOR swizzle of the 16-byte column chunks that keeps
//    the transposing reads free of bank conflicts).  Out-of-range rows read as zero.
//  * Epilogue: the C tile is staged through LDS (padded rows, conflict-free) and written
//    with 16-byte row-contiguous stores; bias is added in fp32 before rounding.
#pragma once
#include "common.hpp"
#include "gemm.hpp"

namespace fastlstm {

#define FASTLSTM_LDS_PTR __attribute__((address_space(3)))

template <typename T> __device__ __forceinline__ u32x2 lds_read_tr16(const unsigned char *p);
template <> __device__ __forceinline__ u32x2 lds_read_tr16<_Float16>(const unsigned char *p) {
    typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 v4;
    auto lp = (FASTLSTM_LDS_PTR v4 *)(p);
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16(lp));
}
template <> __device__ __forceinline__ u32x2 lds_read_tr16<__bf16>(const unsigned char *p) {
    typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 v4;
    auto lp = (FASTLSTM_LDS_PTR v4 *)(p);
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16(lp));
}

// 16 bytes per lane, global -> LDS, destination = lds_block + 16 * lane.  (The 16-byte form
// exists on gfx950 only; the host pass of hipcc must not see the builtin.)
__device__ __forceinline__ void load_block_to_lds(__amdgpu_buffer_rsrc_t rsrc, unsigned char *lds_block,
                                                  unsigned voffset, unsigned soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (FASTLSTM_LDS_PTR void *)lds_block, 16, voffset, soffset, 0, 0);
#else
    (void)rsrc; (void)lds_block; (void)voffset; (void)soffset;
#endif
}

template <int BM, int BN, int NS, int WVM, int WVN, int KSPT> struct Gemm16Cfg {
    static constexpr int NWAVES = WVM * WVN, THREADS = 64 * NWAVES;  // waves form a WVM x WVN grid
    static constexpr int BK = 32 * KSPT;  // KSPT k-steps (MFMA K = 32) per LDS stage
    static constexpr int A_LD = BM * 2, B_LD = BN * 2;  // K-major row strides (bytes), swizzled not padded
    static constexpr int A_BYTES = BM * BK * 2;
    static constexpr int B_BYTES = BN * BK * 2;
    static constexpr int STAGE = A_BYTES + B_BYTES;
    static constexpr int C_LD = BN * 2 + 16;  // padded C-tile row (bytes)
    static constexpr int C_BYTES = BM * C_LD;
    static constexpr int LDS_BYTES = (NS * STAGE > C_BYTES) ? NS * STAGE : C_BYTES;  // NS pipeline stages
    static constexpr int A_LOADS = BM * BK * 2 / kFragBytes / NWAVES;  // 1 KiB LDS-direct loads per wave per k-tile
    static constexpr int B_LOADS = BN * BK * 2 / kFragBytes / NWAVES;
    static constexpr int TM = BM / WVM / 16, TN = BN / WVN / 16;       // 16x16 tiles per wave
};

// s_waitcnt vmcnt(N) lgkmcnt(0): at most N vector-memory operations of this wave still
// in flight, all LDS operations done (gfx9 encoding: vmcnt = bits 3:0 and 15:14).
template <int N> __device__ __forceinline__ void wait_vm_at_most() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8));
}

// acc += A(rows m0.., k in [kb, ke)) . B(columns n0.., same k) for one BM x BN tile, by a workgroup
// of 64*WVM*WVN threads with Gemm16Cfg::LDS_BYTES of LDS at `smem`; ke - kb a multiple of BK.  All
// threads of the workgroup call it together; it ends behind a workgroup barrier (the LDS is free).
template <typename T, bool A_KM, bool B_KM, int BM, int BN, int NS, int WVM, int WVN, int KSPT>
__device__ __forceinline__ void gemm16_mainloop(const GemmParams &p, const int m0, const int n0, const int kb,
                                                const int ke, unsigned char *smem,
                                                f32x4 (&acc)[BM / WVM / 16][BN / WVN / 16]) {
    using C = Gemm16Cfg<BM, BN, NS, WVM, WVN, KSPT>;
    constexpr int NWAVES = C::NWAVES;
    constexpr int BK = C::BK, TM = C::TM, TN = C::TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane >> 4, r = lane & 15;
    const int wm = wave / WVN, wn = wave % WVN;
    const int nkt = (ke - kb) / BK;

    const unsigned a_bytes = (unsigned)((A_KM ? (size_t)p.K : (size_t)p.M) * p.lda * 2);
    const unsigned b_bytes = (unsigned)((B_KM ? (size_t)p.K : (size_t)p.N) * p.ldb * 2);
    const __amdgpu_buffer_rsrc_t ra_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.A), 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.B), 0, b_bytes, 0x00020000);

    // XOR swizzle of the 16-byte column chunk index of a K-major tile, as a function of the
    // k-row: the 4 rows x 32 bytes one 16-lane group of a transposing read touches (k & 3),
    // and the rows of neighbouring lane groups (k & 8), land in different banks.
    auto swz = [](int k) { return ((k & 3) << 1) ^ (((k >> 3) & 1) << 3); };

    // 1 KiB LDS block `blk` of a k-tile is filled by one wave instruction; wave w fills
    // blocks w, w + NWAVES, ...  Lane l of block blk fetches:
    //   K-contiguous operand (operand order): row = 16 (blk / KSPT) + l % 16, k = 32 (blk % KSPT) + 8 (l / 16)
    //   K-major operand: chunk position P = 64 blk + l -> k-row P / CPR, column chunk (P % CPR) ^ swz(k)
    unsigned goff_a[C::A_LOADS], goff_b[C::B_LOADS];
#pragma unroll
    for (int i = 0; i < C::A_LOADS; ++i) {
        const int blk = wave + NWAVES * i;
        if constexpr (!A_KM) {
            const int row = (blk / KSPT) * 16 + r, k = (blk % KSPT) * 32 + q * 8;
            goff_a[i] = (unsigned)(((size_t)(m0 + row) * p.lda + kb + k) * 2);
        } else {
            constexpr int CPR = BM / 8;
            const int P = blk * 64 + lane, k = P / CPR, mc = (P % CPR) ^ swz(k);
            goff_a[i] = (unsigned)(((size_t)(kb + k) * p.lda + m0 + mc * 8) * 2);
        }
    }
#pragma unroll
    for (int i = 0; i < C::B_LOADS; ++i) {
        const int blk = wave + NWAVES * i;
        if constexpr (!B_KM) {
            const int row = (blk / KSPT) * 16 + r, k = (blk % KSPT) * 32 + q * 8;
            goff_b[i] = (unsigned)(((size_t)(n0 + row) * p.ldb + kb + k) * 2);
        } else {
            constexpr int CPR = BN / 8;
            const int P = blk * 64 + lane, k = P / CPR, nc = (P % CPR) ^ swz(k);
            goff_b[i] = (unsigned)(((size_t)(kb + k) * p.ldb + n0 + nc * 8) * 2);
        }
    }
    const unsigned a_kstep = A_KM ? (unsigned)BK * p.lda * 2 : BK * 2;  // byte advance per k-tile
    const unsigned b_kstep = B_KM ? (unsigned)BK * p.ldb * 2 : BK * 2;

    // k-tile kt -> LDS stage; the k-tile advance never leaves the operand: scalar offset
    auto gload = [&](int kt, int stage) {
        unsigned char *sa = smem + stage * C::STAGE, *sb = sa + C::A_BYTES;
#pragma unroll
        for (int i = 0; i < C::A_LOADS; ++i)
            load_block_to_lds(ra_rsrc, sa + (wave + NWAVES * i) * kFragBytes, goff_a[i], kt * a_kstep);
#pragma unroll
        for (int i = 0; i < C::B_LOADS; ++i)
            load_block_to_lds(rb_rsrc, sb + (wave + NWAVES * i) * kFragBytes, goff_b[i], kt * b_kstep);
    };
    // fragment of rows [tile16*16, +16) of the operand tile, k-step ks
    auto frag = [&](const unsigned char *tile, bool km, int ld, int tile16, int ks) -> u32x4 {
        if (!km) {
            return *reinterpret_cast<const u32x4 *>(tile + ((tile16 * KSPT + ks) * 64 + lane) * 16);
        } else {
            // lane (a, b) of a 16-lane group addresses 4 consecutive m of k-row a; rows k and
            // k + 4 (second read) share k & 3 and k & 8, hence the swizzle
            const int a = r >> 2, b = r & 3;
            const int k = ks * 32 + q * 8 + a;
            const unsigned char *base = tile + k * ld + (((tile16 * 2 + (b >> 1)) ^ swz(k)) * 16) + (b & 1) * 8;
            const u32x2 lo = lds_read_tr16<T>(base), hi = lds_read_tr16<T>(base + 4 * ld);
            return u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    };

    // NS-stage pipeline: the loads of k-tiles kt+1 .. kt+NS-1 are in flight while k-tile kt is
    // multiplied (memory latency, not bandwidth, bounds a short loop: ~2 us per round trip).
    // Per iteration: wait for this wave's own loads of tile kt (everything issued later may
    // stay in flight), barrier (every wave's part of tile kt has landed, and every wave is
    // done reading the stage that tile kt+NS-1 is about to overwrite), issue, multiply.
    constexpr int D = NS - 1;                         // prefetch distance in k-tiles
    constexpr int LPT = C::A_LOADS + C::B_LOADS;      // loads per k-tile per wave
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < nkt) gload(d, d);
    for (int kt = 0; kt < nkt; ++kt) {
        if (kt + D <= nkt) wait_vm_at_most<(D - 1) * LPT>();   // D-1 younger tiles may stay in flight
        else wait_vm_at_most<0>();                             // tail: fewer tiles behind this one
        __builtin_amdgcn_s_barrier();
        if (kt + D < nkt) gload(kt + D, (kt + D) % NS);
        const int st = kt % NS;
        const unsigned char *sa = smem + st * C::STAGE, *sb = sa + C::A_BYTES;
#pragma unroll
        for (int ks = 0; ks < KSPT; ++ks) {
            u32x4 fa[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = frag(sa, A_KM, C::A_LD, wm * TM + i, ks);
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const u32x4 fb = frag(sb, B_KM, C::B_LD, wn * TN + j, ks);
#pragma unroll
                for (int i = 0; i < TM; ++i) acc[i][j] = mfma_kstep<T>(fb, fa[i], acc[i][j]);
            }
        }
    }
    __syncthreads();  // all waves are done reading the stages before the LDS is reused
}

// Stores the accumulated tile: fp32 partials of `split` when p.splits > 1, else bias + rounding,
// staged through LDS and written with 16-byte row-contiguous stores.
template <typename T, int BM, int BN, int NS, int WVM, int WVN, int KSPT>
__device__ __forceinline__ void gemm16_epilogue(const GemmParams &p, const int m0, const int n0, const int split,
                                                unsigned char *smem,
                                                const f32x4 (&acc)[BM / WVM / 16][BN / WVN / 16]) {
    using C = Gemm16Cfg<BM, BN, NS, WVM, WVN, KSPT>;
    constexpr int THREADS = C::THREADS, TM = C::TM, TN = C::TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane >> 4, r = lane & 15;
    const int wm = wave / WVN, wn = wave % WVN;
    // ---- epilogue -----------------------------------------------------------------------
    // lane holds C[m = tile row r][n = 4q .. 4q+3] of each 16x16 tile
    if (p.splits > 1) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = m0 + (wm * TM + i) * 16 + r;
            if (m >= p.M) continue;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int nb = n0 + (wn * TN + j) * 16 + q * 4;
                if (nb >= p.N) continue;
                float *dst = p.Cpart + ((size_t)split * p.M + m) * p.N + nb;
                if ((p.N & 3) == 0) {
                    *reinterpret_cast<f32x4 *>(dst) = acc[i][j];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (nb + e < p.N) dst[e] = acc[i][j][e];
                }
            }
        }
        return;
    }
    const T *bias0 = static_cast<const T *>(p.bias0), *bias1 = static_cast<const T *>(p.bias1);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int nl = (wn * TN + j) * 16 + q * 4;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias0) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n0 + nl + e < p.N)
                    bv[e] = Elem<T>::to_f32(bias0[n0 + nl + e]) + (bias1 ? Elem<T>::to_f32(bias1[n0 + nl + e]) : 0.f);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int ml = (wm * TM + i) * 16 + r;
            const f32x4 v = acc[i][j];
            T pk[4] = {Elem<T>::from_f32(v[0] + bv[0]), Elem<T>::from_f32(v[1] + bv[1]),
                       Elem<T>::from_f32(v[2] + bv[2]), Elem<T>::from_f32(v[3] + bv[3])};
            *reinterpret_cast<u32x2 *>(smem + (size_t)ml * C::C_LD + nl * 2) = *reinterpret_cast<u32x2 *>(pk);
        }
    }
    __syncthreads();
    T *Cg = static_cast<T *>(p.C);
    constexpr int CPR = BN / 8;  // 16-byte chunks per C-tile row
    const bool vec_ok = (p.ldc & 7) == 0;
    for (int c = tid; c < BM * CPR; c += THREADS) {
        const int ml = c / CPR, nc = c % CPR;
        const int m = m0 + ml, n = n0 + nc * 8;
        if (m >= p.M || n >= p.N) continue;
        const u32x4 v = *reinterpret_cast<const u32x4 *>(smem + (size_t)ml * C::C_LD + nc * 16);
        T *dst = Cg + (size_t)m * p.ldc + n;
        if (vec_ok && n + 8 <= p.N) {
            *reinterpret_cast<u32x4 *>(dst) = v;
        } else {
            const T *tv = reinterpret_cast<const T *>(&v);
            for (int e = 0; e < 8; ++e)
                if (n + e < p.N) dst[e] = tv[e];
        }
    }
}

// One BM x BN tile of C (rows m0.., columns n0.., K range of `split`): main loop + epilogue.
template <typename T, bool A_KM, bool B_KM, int BM, int BN, int NS, int WVM, int WVN, int KSPT>
__device__ __forceinline__ void gemm16_tile(const GemmParams &p, const int m0, const int n0, const int split,
                                            unsigned char *smem, const int trace_slot) {
    constexpr int TM = BM / WVM / 16, TN = BN / WVN / 16;
    long long t_start = 0, t_epi = 0;
    if (p.trace) t_start = (long long)wall_clock64();
    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int kb = split * p.k_per_split;
    gemm16_mainloop<T, A_KM, B_KM, BM, BN, NS, WVM, WVN, KSPT>(p, m0, n0, kb, min(p.K, kb + p.k_per_split), smem, acc);
    if (p.trace) t_epi = (long long)wall_clock64();
    gemm16_epilogue<T, BM, BN, NS, WVM, WVN, KSPT>(p, m0, n0, split, smem, acc);
    if (p.trace && threadIdx.x == 0) {   // stamps: start, main loop entered (= start), main loop left, done
        long long *t = p.trace + (size_t)trace_slot * 4;
        t[0] = t_start; t[1] = t_start; t[2] = t_epi; t[3] = (long long)wall_clock64();
    }
}

template <typename T, bool A_KM, bool B_KM, int BM, int BN, int NS, int WVM, int WVN, int KSPT>
__global__ __launch_bounds__(64 * WVM * WVN) void gemm16_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tiles_n = cdiv(p.N, BN), tiles_m = cdiv(p.M, BM);
    int bid = blockIdx.x;
    const int split = bid / (tiles_m * tiles_n);
    bid -= split * tiles_m * tiles_n;
    // Tile order: every XCD gets a contiguous range of a grouped order in which 8 x 8 blocks
    // of C tiles are consecutive, so the ~64 workgroups an XCD runs at a time re-use each
    // other's A and B tiles out of that XCD's L2.
    constexpr int GM = 8;
    const int lin = xcd_major_id(bid, tiles_m * tiles_n);
    const int per_group = GM * tiles_n, first_m = (lin / per_group) * GM;
    const int gsz = min(tiles_m - first_m, GM);
    const int m0 = (first_m + (lin % per_group) % gsz) * BM, n0 = ((lin % per_group) / gsz) * BN;
    gemm16_tile<T, A_KM, B_KM, BM, BN, NS, WVM, WVN, KSPT>(p, m0, n0, split, smem, (int)blockIdx.x);
}

}  // namespace fastlstm

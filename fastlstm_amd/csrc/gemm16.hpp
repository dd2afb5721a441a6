// High-throughput MFMA GEMM for the 16-bit element types (fp16 / bf16, fp32 accumulate):
//     C[m][n] = sum_k A(m,k) * B(n,k)   [+ bias0[n] + bias1[n]]
// the same contraction as gemm.hpp's generic kernel, restricted to the aligned case
// (K a multiple of 64, leading dimensions multiples of 8 elements, operands < 4 GiB)
// that every benchmark configuration of the LSTM hits.
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
#include <type_traits>
#include "common.hpp"
#include "gemm.hpp"

namespace fastlstm {

#define FASTLSTM_LDS_PTR __attribute__((address_space(3)))

// Transposing LDS read (ds_read_b64_tr_b16, the same instruction for both 16-bit types) of the
// 8 bytes at `p + OFF`.  Written as inline assembly on purpose: the compiler orders every LDS
// read it knows of behind ALL LDS-direct global loads in flight (s_waitcnt vmcnt(0)), which
// would serialise the prefetch of the next k-tile with the multiplication of this one.  The
// result is valid only behind lds_reads_landed_but() (below), which counts the reads issued since.
template <int OFF> __device__ __forceinline__ u32x2 lds_read_tr16(const unsigned char *p) {
    u32x2 v = {0u, 0u};
#if defined(__HIP_DEVICE_COMPILE__)
    const unsigned addr = (unsigned)(size_t)((FASTLSTM_LDS_PTR const unsigned char *)p);
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
#else
    (void)p;
#endif
    return v;
}
// Plain 16-byte LDS read, as inline assembly for the same reason.
template <int OFF> __device__ __forceinline__ u32x4 lds_read_b128_asm(const unsigned char *p) {
    u32x4 v = {0u, 0u, 0u, 0u};
#if defined(__HIP_DEVICE_COMPILE__)
    const unsigned addr = (unsigned)(size_t)((FASTLSTM_LDS_PTR const unsigned char *)p);
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
#else
    (void)p;
#endif
    return v;
}
// Waits until at most N LDS operations of this wave are in flight (they complete in order, so
// everything but the N youngest has landed); `f` passes through it so that no use of the fragment
// can be scheduled ahead of the wait.  Operations the compiler issued on its own (LDS or scalar
// memory) only make the wait stricter.
template <int N> __device__ __forceinline__ void lds_reads_landed_but(u32x4 &f) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(f) : "n"(N));
#else
    (void)f;
#endif
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

// The same with device scope (sc1): the load misses the non-coherent cache levels.
__device__ __forceinline__ void load_block_to_lds_device(__amdgpu_buffer_rsrc_t rsrc, unsigned char *lds_block,
                                                         unsigned voffset, unsigned soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (FASTLSTM_LDS_PTR void *)lds_block, 16, voffset, soffset, 0, 16);
#else
    (void)rsrc; (void)lds_block; (void)voffset; (void)soffset;
#endif
}

// 16 bytes per lane, global -> LDS at lds_addr + 16 * lane, with or without device scope; voff = the lane's byte offset,
// soff = the block's byte offset (scalar).  Inline assembly, so that the compiler does not know of the load: it waits for every load it knows of before a workgroup barrier and for every LDS-direct load before an LDS access; the wave that uses this counts its own loads (s_waitcnt vmcnt(n)).  The s_nop: a scalar
// operand may have been written by a vector instruction just before (v_readlane of a spilled scalar), and a
// vector memory instruction may read such a register only 5 wait states later, which the compiler sees to for
// its own instructions but not inside inline assembly (m0 needs 1 before the load).
template <bool DEVICE_SCOPE>
__device__ __forceinline__ void dma_block_asm(u32x4 rsrc, unsigned lds_addr, unsigned voff, unsigned soff) {
#if defined(__HIP_DEVICE_COMPILE__)
    // (m0 cannot be named as clobbered: a kernel that uses this sends every LDS-direct load through here, so that nothing else relies on m0)
    if constexpr (DEVICE_SCOPE)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, %3 offen sc1 lds"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                     : "memory");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                     : "memory");
#else
    (void)rsrc; (void)lds_addr; (void)voff; (void)soff;
#endif
}

// acc += a . b with the accumulator pinned to the accumulation registers (AGPRs).  With more
// than 128 accumulators per lane the register allocator otherwise shuttles them between the two
// halves of the register file around every MFMA.
template <typename T> __device__ __forceinline__ void mfma_kstep_agpr(const u32x4 a, const u32x4 b, f32x4 &c) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (Elem<T>::DT == FASTLSTM_BF16)
        asm("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else
        asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
#else
    (void)a; (void)b; (void)c;
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
                                                f32x4 (&acc)[BM / WVM / 16][BN / WVN / 16], const int tid_salt = 0) {
    using C = Gemm16Cfg<BM, BN, NS, WVM, WVN, KSPT>;
    constexpr int NWAVES = C::NWAVES;
    constexpr int BK = C::BK, TM = C::TM, TN = C::TN;
    // tid_salt is zero.  A caller inside a loop passes one the compiler cannot see through, so that the
    // per-lane address arithmetic below is redone per call instead of being kept in registers (or
    // spilled and reloaded inside the k loop) across the caller's loop.
    // (the wave index as a scalar: the LDS destinations of the LDS-direct loads then need no v_readfirstlane)
    const int tid = threadIdx.x + tid_salt, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

    // K-contiguous operand tile in LDS: rows of BK elements (LPR 16-byte chunks), chunk c of row r
    // at position c ^ kswz(r % 16): the 16 lanes of a fragment read (16 rows, one chunk index) hit
    // 16 different 16-byte bank groups.
    constexpr int LPR = 4 * KSPT, RPB = 64 / LPR;   // chunks per row; rows per 1 KiB block
    static_assert(KSPT == 1 || KSPT == 2 || KSPT == 4, "row of a k-tile: 64, 128 or 256 bytes");
    auto kswz = [](int r16) { return (r16 >> (KSPT == 1 ? 2 : KSPT == 2 ? 1 : 0)) & (LPR - 1); };

    // 1 KiB LDS block `blk` of a k-tile is filled by one wave instruction; wave w fills
    // blocks w, w + NWAVES, ...  Lane l of block blk fetches:
    //   K-contiguous operand: row = RPB blk + l / LPR, whole rows of the k-tile (full cache lines),
    //                         chunk (l % LPR) ^ kswz(row)
    //   K-major operand: chunk position P = 64 blk + l -> k-row P / CPR, column chunk (P % CPR) ^ swz(k)
    // Blocks w + NWAVES i, i = 0, 1, ..., of a wave differ by whole groups of rows that leave both
    // swizzles unchanged: one per-lane offset per operand, the rest is a scalar offset.
    static_assert((NWAVES * RPB) % 16 == 0 && (NWAVES * 64) % (BM / 8) == 0 && (NWAVES * 64) % (BN / 8) == 0 &&
                  (NWAVES * 64 / (BM / 8)) % 16 == 0 && (NWAVES * 64 / (BN / 8)) % 16 == 0, "row groups per block");
    unsigned goff_a, goff_b;
    if constexpr (!A_KM) {
        const int row = wave * RPB + lane / LPR, k = ((lane % LPR) ^ kswz(row & 15)) * 8;
        goff_a = (unsigned)(((size_t)(m0 + row) * p.lda + kb + k) * 2);
    } else {
        constexpr int CPR = BM / 8;
        const int P = wave * 64 + lane, k = P / CPR, mc = (P % CPR) ^ swz(k);
        goff_a = (unsigned)(((size_t)(kb + k) * p.lda + m0 + mc * 8) * 2);
    }
    if constexpr (!B_KM) {
        const int row = wave * RPB + lane / LPR, k = ((lane % LPR) ^ kswz(row & 15)) * 8;
        goff_b = (unsigned)(((size_t)(n0 + row) * p.ldb + kb + k) * 2);
    } else {
        constexpr int CPR = BN / 8;
        const int P = wave * 64 + lane, k = P / CPR, nc = (P % CPR) ^ swz(k);
        goff_b = (unsigned)(((size_t)(kb + k) * p.ldb + n0 + nc * 8) * 2);
    }
    const unsigned a_istep = (unsigned)(A_KM ? NWAVES * 64 / (BM / 8) : NWAVES * RPB) * p.lda * 2;  // bytes per block index
    const unsigned b_istep = (unsigned)(B_KM ? NWAVES * 64 / (BN / 8) : NWAVES * RPB) * p.ldb * 2;
    const unsigned a_kstep = A_KM ? (unsigned)BK * p.lda * 2 : BK * 2;  // byte advance per k-tile
    const unsigned b_kstep = B_KM ? (unsigned)BK * p.ldb * 2 : BK * 2;

    // k-tile kt -> LDS stage, loads `part`, part + parts, ... of the wave's A_LOADS + B_LOADS (all of them:
    // part 0 of 1); the k-tile advance never leaves the operand: scalar offset.  Inside the main loop the
    // loads of a k-tile are dealt out among the multiplications, one or two at a time: eight waves that
    // issue all 64 loads of a k-tile at once fill the vector-memory queue and stand in it instead of
    // issuing MFMAs (K1 at T*B = 32768, 4H = 4096, K = 1024: 967 -> 1040 TFLOP/s).
    auto gload = [&](int kt, int stage, int part, int parts) {
        unsigned char *sa = smem + stage * C::STAGE, *sb = sa + C::A_BYTES;
#pragma unroll
        for (int i = 0; i < C::A_LOADS; ++i)
            if (i % parts == part)
                load_block_to_lds(ra_rsrc, sa + (wave + NWAVES * i) * kFragBytes, goff_a, kt * a_kstep + i * a_istep);
#pragma unroll
        for (int i = 0; i < C::B_LOADS; ++i)
            if ((i + C::A_LOADS) % parts == part)
                load_block_to_lds(rb_rsrc, sb + (wave + NWAVES * i) * kFragBytes, goff_b, kt * b_kstep + i * b_istep);
    };
    // fragment of rows [tile16*16, +16) of the operand tile, k-step ks
    auto frag = [&](const unsigned char *tile, auto km_, auto ld_, int tile16, int ks) -> u32x4 {
        constexpr bool km = decltype(km_)::value;
        constexpr int LD = decltype(ld_)::value, ld = LD;
        if constexpr (!km) {
            const unsigned char *src = tile + ((tile16 * 16 + r) * LPR + ((ks * 4 + q) ^ kswz(r))) * 16;
            if constexpr (A_KM || B_KM) return lds_read_b128_asm<0>(src);   // see the streamed loop below
            else return *reinterpret_cast<const u32x4 *>(src);
        } else {
            // lane (a, b) of a 16-lane group addresses 4 consecutive m of k-row a; rows k and
            // k + 4 (second read) share k & 3 and k & 8, hence the swizzle
            const int a = r >> 2, b = r & 3;
            const int k = ks * 32 + q * 8 + a;
            const unsigned char *base = tile + k * ld + (((tile16 * 2 + (b >> 1)) ^ swz(k)) * 16) + (b & 1) * 8;
            const u32x2 lo = lds_read_tr16<0>(base), hi = lds_read_tr16<4 * LD>(base);
            return u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    };

    // NS-stage pipeline: the loads of k-tiles kt+1 .. kt+NS-1 are in flight while k-tile kt is
    // multiplied (memory latency, not bandwidth, bounds a short loop: ~2 us per round trip).
    // The fragments of k-step s+1 are read from LDS while k-step s is multiplied (two register
    // sets).  Where s+1 is the first k-step of the next k-tile, the wave first waits for its own
    // loads of that tile (everything issued later may stay in flight) and meets the others at a
    // barrier (every wave's part of the tile has landed, and every wave has READ the last
    // fragments of the stage that the next global loads overwrite); the multiplications of the
    // k-tile's last k-step then cover the barrier skew and the LDS latency.
    constexpr int D = NS - 1;                         // prefetch distance in k-tiles
    constexpr int LPT = C::A_LOADS + C::B_LOADS;      // loads per k-tile per wave
    static_assert(KSPT % 2 == 0, "fragment register sets alternate by k-step parity");
    // k-tile kt has landed in LDS and the stage of k-tile kt-1 is free: the caller now issues the loads of
    // k-tile kt-1+NS into it, before it calls tile_ready again
    auto tile_ready = [&](int kt) {
        if (kt + D <= nkt) wait_vm_at_most<(D - 1) * LPT>();   // D-1 younger tiles may stay in flight
        else wait_vm_at_most<0>();                             // tail: fewer tiles behind this one
        __builtin_amdgcn_s_barrier();
    };
    if constexpr (A_KM || B_KM) {
        // Products with a K-major operand: all fragment reads are inline assembly (see
        // lds_read_tr16) and this loop counts them itself.  Registers: the B fragments of both
        // k-steps of a k-tile (TN each) and two registers through which the A fragments stream, one
        // ahead of the multiplications.
        //   iteration i of a k-step: read B fragment i / (TM / TN) of the next k-step (first k-step
        //       only, every TM / TN-th i), read the next A fragment, wait for A fragment i
        //       (everything issued behind it may stay in flight), multiply.
        //   The last two A fragments of a k-tile are in registers when iteration TM - 2 of its second
        //       k-step starts: there the wave waits for all its reads, passes the barrier that hands
        //       the stage to the global loads, and requests the next k-tile's first fragments, whose
        //       latency the remaining two iterations' multiplications cover.
        static_assert(KSPT == 2, "two k-steps per k-tile");
        static_assert(TM % TN == 0 && TM >= 4, "B fragments are read every TM / TN-th iteration");
        constexpr int NA = A_KM ? 2 : 1, NB = B_KM ? 2 : 1, EVERY = TM / TN;   // LDS instructions per fragment
        u32x4 fs[2], fb[2][TN];
        auto rd_a = [&](int kt, int ks, int i) {
            return frag(smem + (kt % NS) * C::STAGE, std::bool_constant<A_KM>{}, std::integral_constant<int, C::A_LD>{},
                        wm * TM + i, ks);
        };
        auto rd_b = [&](int kt, int ks, int j) {
            return frag(smem + (kt % NS) * C::STAGE + C::A_BYTES, std::bool_constant<B_KM>{},
                        std::integral_constant<int, C::B_LD>{}, wn * TN + j, ks);
        };
#pragma unroll
        for (int d = 0; d < D; ++d)
            if (d < nkt) gload(d, d, 0, 1);
        tile_ready(0);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[0][j] = rd_b(0, 0, j);
        fs[0] = rd_a(0, 0, 0);
        for (int kt = 0; kt < nkt; ++kt) {
            const bool more = kt + 1 < nkt;
            auto step0 = [&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                constexpr bool rdb = i % EVERY == 0;
                if (kt + D < nkt) gload(kt + D, (kt + D) % NS, i, TM);   // into the stage the last barrier freed
                if constexpr (rdb) fb[1][i / EVERY] = rd_b(kt, 1, i / EVERY);
                if constexpr (i + 1 < TM) fs[(i + 1) & 1] = rd_a(kt, 0, i + 1);
                else fs[(i + 1) & 1] = rd_a(kt, 1, 0);
                lds_reads_landed_but<(rdb ? NB : 0) + NA>(fs[i & 1]);   // behind A fragment i: this iteration's reads
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma_kstep<T>(fb[0][j], fs[i & 1], acc[i][j]);
            };
            auto step1 = [&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                if constexpr (i < TM - 2) {
                    fs[(i + 1) & 1] = rd_a(kt, 1, i + 1);
                    lds_reads_landed_but<NA>(fs[i & 1]);
                } else if constexpr (i == TM - 2) {
                    fs[(i + 1) & 1] = rd_a(kt, 1, i + 1);
                    lds_reads_landed_but<0>(fs[0]);   // every read of this k-tile has landed (fs[1] passes below)
                    lds_reads_landed_but<0>(fs[1]);
                    if (more) {
                        tile_ready(kt + 1);
#pragma unroll
                        for (int j = 0; j < TN; ++j) fb[0][j] = rd_b(kt + 1, 0, j);
                    }
                }
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma_kstep<T>(fb[1][j], fs[i & 1], acc[i][j]);
                // A fragment TM - 2 has been multiplied: its register takes the next k-tile's first A fragment
                if constexpr (i == TM - 2)
                    if (more) fs[0] = rd_a(kt + 1, 0, 0);
            };
            static_assert(TM == 4 || TM == 8, "wave tile rows");
            step0(std::integral_constant<int, 0>{}); step0(std::integral_constant<int, 1>{});
            step0(std::integral_constant<int, 2>{}); step0(std::integral_constant<int, 3>{});
            if constexpr (TM == 8) {
                step0(std::integral_constant<int, 4>{}); step0(std::integral_constant<int, 5>{});
                step0(std::integral_constant<int, 6>{}); step0(std::integral_constant<int, 7>{});
            }
            step1(std::integral_constant<int, 0>{}); step1(std::integral_constant<int, 1>{});
            step1(std::integral_constant<int, 2>{}); step1(std::integral_constant<int, 3>{});
            if constexpr (TM == 8) {
                step1(std::integral_constant<int, 4>{}); step1(std::integral_constant<int, 5>{});
                step1(std::integral_constant<int, 6>{}); step1(std::integral_constant<int, 7>{});
            }
        }
        __syncthreads();   // every wave has read its last fragments (waited for above)
        return;
    }
    u32x4 fa[2][TM], fb[2][TN];
    auto read_a = [&](int kt, int ks, int i) {
        fa[ks & 1][i] = frag(smem + (kt % NS) * C::STAGE, std::bool_constant<A_KM>{},
                             std::integral_constant<int, C::A_LD>{}, wm * TM + i, ks);
    };
    auto read_b = [&](int kt, int ks, int j) {
        fb[ks & 1][j] = frag(smem + (kt % NS) * C::STAGE + C::A_BYTES, std::bool_constant<B_KM>{},
                             std::integral_constant<int, C::B_LD>{}, wn * TN + j, ks);
    };
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < nkt) gload(d, d, 0, 1);
    tile_ready(0);
    if (D < nkt) gload(D, D % NS, 0, 1);
#pragma unroll
    for (int i = 0; i < TM; ++i) read_a(0, 0, i);
#pragma unroll
    for (int j = 0; j < TN; ++j) read_b(0, 0, j);
    for (int kt = 0; kt < nkt; ++kt) {
#pragma unroll
        for (int ks = 0; ks < KSPT; ++ks) {
            const bool last = ks + 1 == KSPT;
            const bool more = !last || kt + 1 < nkt;
            const int nkt_ = last ? kt + 1 : kt, nks = last ? 0 : ks + 1;   // the k-step after this one
            if (last && more) tile_ready(kt + 1);
            // column j of the wave tile is multiplied while the next k-step's fragments stream in
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                // behind tile_ready(kt + 1): the stage of k-tile kt is free (its fragments are in registers)
                if (last && kt + 1 + D < nkt) gload(kt + 1 + D, (kt + 1 + D) % NS, j, TN);
                if (more) {
                    read_b(nkt_, nks, j);
#pragma unroll
                    for (int i = j; i < TM; i += TN) read_a(nkt_, nks, i);
                }
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    if constexpr (TM * TN > 32) mfma_kstep_agpr<T>(fb[ks & 1][j], fa[ks & 1][i], acc[i][j]);
                    else acc[i][j] = mfma_kstep<T>(fb[ks & 1][j], fa[ks & 1][i], acc[i][j]);
                }
            }
        }
    }
    __syncthreads();  // all waves are done reading the stages before the LDS is reused
}

// LDS reads on LDS byte addresses, as inline assembly (see lds_read_tr16): the wave that uses them waits for
// them itself (FragSet::landed).
template <int OFF> __device__ __forceinline__ u32x4 lds_rd128(unsigned addr) {
    u32x4 v = {0u, 0u, 0u, 0u};
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
#else
    (void)addr;
#endif
    return v;
}
template <int OFF> __device__ __forceinline__ u32x4 lds_rd_tr16x2(unsigned addr) {
    u32x2 lo = {0u, 0u}, hi = {0u, 0u};
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(addr), "n"(OFF));
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(OFF + 2048));
#else
    (void)addr;
#endif
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
}

// The fp32 fragment of a K-major tile (k-rows of 1 KiB): the lane's 4 consecutive k of one column, four 4-byte reads
// 1 KiB apart.  (No transposing read exists for 32-bit elements, and none is needed: with true-fp32 MFMA a phase of
// the loop below is 4096 matrix cycles, next to which 48 such reads per wave do not show.)
template <int OFF> __device__ __forceinline__ u32x4 lds_rd32x4(unsigned addr) {
    unsigned e0 = 0u, e1 = 0u, e2 = 0u, e3 = 0u;
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(e0) : "v"(addr), "n"(OFF));
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(e1) : "v"(addr), "n"(OFF + 1024));
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(e2) : "v"(addr), "n"(OFF + 2048));
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(e3) : "v"(addr), "n"(OFF + 3072));
#else
    (void)addr;
#endif
    return u32x4{e0, e1, e2, e3};
}

// The same contraction as gemm16_mainloop for the 256 x 256 x 64 tile with 8 waves (2 x 4) and two LDS
// stages, scheduled as a ping-pong between the two waves of each SIMD.  Waves 0..3 (the upper half of the
// C tile) and waves 4..7 (the lower half) run the same sequence of phases one phase apart:
//     memory phase of k-step j:   read the 12 fragments of the k-step from LDS (and, once per k-tile,
//                                 request this wave's 8 blocks of the k-tile after next), wait for the
//                                 fragments
//     compute phase of k-step j:  32 MFMAs from registers, nothing else
// with a workgroup barrier between phases, so that on every SIMD one wave issues MFMAs back to back
// while the other one issues the LDS and vector-memory instructions and absorbs their waits.  (With
// both waves in the same phase at the same time, as in gemm16_mainloop, the matrix pipe idles at
// every barrier and behind every queued memory instruction: 1180 -> 1500 TFLOP/s at M = 32768,
// N = 8192, K = 2048 together with the non-temporal stores of the epilogue.)
// The LDS-direct loads are inline assembly (dma_block_asm): the kernel's only ones, counted by hand.
// T = float: the same loop on tiles of 128 bytes of K per row, i.e. 32 elements per k-tile in two k-steps of
// four v_mfma_f32_16x16x4_f32 per fragment pair (true fp32); K-contiguous tiles have the 16-bit layout byte for
// byte, K-major tiles are 32 k-rows of 1 KiB, unswizzled (lds_rd32x4).
// c + the sum of the 8 elements of a fragment register quad (fp32 accumulate).
template <typename T> __device__ __forceinline__ float frag_sum(const u32x4 f, float c) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (Elem<T>::DT == FASTLSTM_FP32) {
        const f32x4 v = __builtin_bit_cast(f32x4, f);
        c += (v[0] + v[1]) + (v[2] + v[3]);
    } else if constexpr (Elem<T>::DT == FASTLSTM_FP16) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        const f16x2 one = {(_Float16)1.f, (_Float16)1.f};
        const f16x8 h = __builtin_bit_cast(f16x8, f);
        c = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 0, 1), one, c, false);
        c = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 2, 3), one, c, false);
        c = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 4, 5), one, c, false);
        c = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 6, 7), one, c, false);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            c += __builtin_bit_cast(float, f[e] << 16) + __builtin_bit_cast(float, f[e] & 0xffff0000u);
    }
#else
    (void)f;
#endif
    return c;
}

// DB: in the k-tiles with (k-tile index of the whole product) % db_mod == db_rem the waves also sum their A
// fragments over k: wave column wn adds the lane's 8 elements of fragments 2 wn and 2 wn + 1 to colsum[0],
// colsum[1] -- this workgroup's share of the column sums of the A operand (the bias gradient of the
// weight-gradient products), as vector instructions of the memory phase.  The column tiles of a row of C tiles
// share the A panel, so each takes every db_mod-th k-tile and none of them is slowed down noticeably (all of
// them in the first column tile: that tile ran 10 % longer and the launch with it).
template <typename T, bool A_KM, bool B_KM, bool DB = false>
__device__ __forceinline__ void gemm16_mainloop_pp(const GemmParams &p, const int m0, const int n0, const int kb,
                                                   const int ke, unsigned char *smem, f32x4 (&acc)[8][4],
                                                   float *colsum = nullptr, const int db_mod = 1, const int db_rem = 0,
                                                   const int tid_salt = 0) {
    constexpr int STAGE = 65536, A_BYTES = 32768;
    // (tid_salt: an opaque zero from a caller inside a loop, see gemm16_mainloop)
    const int tid = threadIdx.x + tid_salt, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = lane >> 4, r = lane & 15;
    const int wm = wave >> 2, wn = wave & 3;
    constexpr int ES = sizeof(T), EPC = 16 / ES;    // element size; elements per 16-byte chunk
    constexpr int BKE = 128 / ES;                     // elements of K per k-tile (rows of 128 bytes)
    constexpr int KROW = 256 * ES, CPR = KROW / 16;   // K-major tile: bytes and 16-byte chunks per k-row
    constexpr int KRB = 8 * 64 / CPR;                 // ... k-rows that the 8 waves fill per load step (16 | 8)
    constexpr bool F32 = ES == 4;
    const int nkt = (ke - kb) / BKE;
    if (nkt <= 0) return;
    const unsigned lds0 = (unsigned)(size_t)((FASTLSTM_LDS_PTR unsigned char *)smem);

    auto rsrc_of = [](const void *base, unsigned bytes) {
        const unsigned long long a = reinterpret_cast<unsigned long long>(base);
        return u32x4{(unsigned)a, (unsigned)(a >> 32) & 0xffffu, bytes, 0x00020000u};
    };
    const u32x4 ra = rsrc_of(p.A, (unsigned)((A_KM ? (size_t)p.K : (size_t)p.M) * p.lda * ES));
    const u32x4 rb = rsrc_of(p.B, (unsigned)((B_KM ? (size_t)p.K : (size_t)p.N) * p.ldb * ES));
    auto swz = [](int k) { return F32 ? 0 : ((k & 3) << 1) ^ (((k >> 3) & 1) << 3); };   // K-major tiles (see gemm16_mainloop)
    auto kswz = [](int r16) { return (r16 >> 1) & 7; };                        // K-contiguous tiles

    // global -> LDS: wave w fills the 1 KiB blocks w, w + 8, w + 16, w + 24 of each operand's 32 KiB tile
    unsigned goff_a, goff_b;
    if constexpr (!A_KM) {
        const int row = wave * 8 + lane / 8, k = ((lane % 8) ^ kswz(row & 15)) * EPC;
        goff_a = (unsigned)(((size_t)(m0 + row) * p.lda + kb + k) * ES);
    } else {
        const int P = wave * 64 + lane, k = P / CPR, mc = (P % CPR) ^ swz(k);
        goff_a = (unsigned)(((size_t)(kb + k) * p.lda + m0 + mc * EPC) * ES);
    }
    if constexpr (!B_KM) {
        const int row = wave * 8 + lane / 8, k = ((lane % 8) ^ kswz(row & 15)) * EPC;
        goff_b = (unsigned)(((size_t)(n0 + row) * p.ldb + kb + k) * ES);
    } else {
        const int P = wave * 64 + lane, k = P / CPR, nc = (P % CPR) ^ swz(k);
        goff_b = (unsigned)(((size_t)(kb + k) * p.ldb + n0 + nc * EPC) * ES);
    }
    const unsigned a_istep = (unsigned)(A_KM ? KRB : 64) * p.lda * ES, b_istep = (unsigned)(B_KM ? KRB : 64) * p.ldb * ES;
    const unsigned a_kstep = A_KM ? (unsigned)BKE * p.lda * ES : 128u, b_kstep = B_KM ? (unsigned)BKE * p.ldb * ES : 128u;
    auto gload = [&](int kt) {
        const unsigned sa = lds0 + (kt & 1) * STAGE + wave * kFragBytes, sb = sa + A_BYTES;
#pragma unroll
        for (int i = 0; i < 4; ++i) dma_block_asm<false>(ra, sa + i * 8 * kFragBytes, goff_a, kt * a_kstep + i * a_istep);
#pragma unroll
        for (int i = 0; i < 4; ++i) dma_block_asm<false>(rb, sb + i * 8 * kFragBytes, goff_b, kt * b_kstep + i * b_istep);
    };

    // LDS -> registers.  K-contiguous operand: fragment i of k-step ks at base[ks] + 2048 i.  K-major operand:
    // the two transposing reads of fragment i at base_i + 16384 ks (+ 2048 for the second one).
    // (fp32 K-major operand: fragment i of k-step ks at base + 64 i + 16384 ks, see lds_rd32x4)
    unsigned a_kc[2], b_kc[2], a_km[8], b_km[4];
    const unsigned a_km32 = lds0 + (unsigned)(q * 4 * KROW + wm * 512 + r * 4);
    const unsigned b_km32 = lds0 + A_BYTES + (unsigned)(q * 4 * KROW + wn * 256 + r * 4);
    {
        const int a = r >> 2, b = r & 3, k = q * 8 + a;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const unsigned c = (unsigned)(r * 128 + (((ks * 4 + q) ^ kswz(r)) * 16));
            a_kc[ks] = lds0 + wm * 16384 + c;
            b_kc[ks] = lds0 + A_BYTES + wn * 8192 + c;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            a_km[i] = lds0 + (unsigned)(k * 512 + ((((wm * 8 + i) * 2 + (b >> 1)) ^ swz(k)) * 16) + (b & 1) * 8);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            b_km[j] = lds0 + A_BYTES + (unsigned)(k * 512 + ((((wn * 4 + j) * 2 + (b >> 1)) ^ swz(k)) * 16) + (b & 1) * 8);
    }
    u32x4 fa[8], fb[4];
    auto read_frags = [&](int kt, auto ks_) {
        constexpr int ks = decltype(ks_)::value;
        const unsigned st = (kt & 1) * STAGE;
        if constexpr (!B_KM) {
            const unsigned ab = b_kc[ks] + st;
            fb[0] = lds_rd128<0>(ab); fb[1] = lds_rd128<2048>(ab); fb[2] = lds_rd128<4096>(ab); fb[3] = lds_rd128<6144>(ab);
        } else if constexpr (F32) {
            const unsigned ab = b_km32 + st;
            fb[0] = lds_rd32x4<ks * 16384>(ab); fb[1] = lds_rd32x4<ks * 16384 + 64>(ab);
            fb[2] = lds_rd32x4<ks * 16384 + 128>(ab); fb[3] = lds_rd32x4<ks * 16384 + 192>(ab);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) fb[j] = lds_rd_tr16x2<ks * 16384>(b_km[j] + st);
        }
        if constexpr (!A_KM) {
            const unsigned aa = a_kc[ks] + st;
            fa[0] = lds_rd128<0>(aa); fa[1] = lds_rd128<2048>(aa); fa[2] = lds_rd128<4096>(aa); fa[3] = lds_rd128<6144>(aa);
            fa[4] = lds_rd128<8192>(aa); fa[5] = lds_rd128<10240>(aa); fa[6] = lds_rd128<12288>(aa); fa[7] = lds_rd128<14336>(aa);
        } else if constexpr (F32) {
            const unsigned aa = a_km32 + st;
            fa[0] = lds_rd32x4<ks * 16384>(aa); fa[1] = lds_rd32x4<ks * 16384 + 64>(aa);
            fa[2] = lds_rd32x4<ks * 16384 + 128>(aa); fa[3] = lds_rd32x4<ks * 16384 + 192>(aa);
            fa[4] = lds_rd32x4<ks * 16384 + 256>(aa); fa[5] = lds_rd32x4<ks * 16384 + 320>(aa);
            fa[6] = lds_rd32x4<ks * 16384 + 384>(aa); fa[7] = lds_rd32x4<ks * 16384 + 448>(aa);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) fa[i] = lds_rd_tr16x2<ks * 16384>(a_km[i] + st);
        }
    };
    auto landed = [&]() {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fa[4]), "+v"(fa[5]), "+v"(fa[6]), "+v"(fa[7]),
                       "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));
#endif
    };
    int db_cnt = DB ? (kb / BKE) % db_mod : 0;   // k-tile index modulo db_mod, counted along
    bool sum_a = false;
    auto compute = [&]() {
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i][j] = mfma_kstep<T>(fb[j], fa[i], acc[i][j]);
        __builtin_amdgcn_s_setprio(0);
    };
    // the column sums of the k-step's A fragments, at the end of the memory phase (the other wave of the
    // SIMD is multiplying meanwhile)
    auto sum_frags = [&]() {
        if constexpr (DB) {
            if (sum_a) {   // the four waves of a row share its 8 A fragments: wave column wn sums fragments 2 wn, 2 wn + 1
                if (wn == 0) { colsum[0] = frag_sum<T>(fa[0], colsum[0]); colsum[1] = frag_sum<T>(fa[1], colsum[1]); }
                else if (wn == 1) { colsum[0] = frag_sum<T>(fa[2], colsum[0]); colsum[1] = frag_sum<T>(fa[3], colsum[1]); }
                else if (wn == 2) { colsum[0] = frag_sum<T>(fa[4], colsum[0]); colsum[1] = frag_sum<T>(fa[5], colsum[1]); }
                else { colsum[0] = frag_sum<T>(fa[6], colsum[0]); colsum[1] = frag_sum<T>(fa[7], colsum[1]); }
            }
        }
    };
    auto phase_end = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    auto loads_landed = [&]() {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
    };

    // k-tiles 0 and 1 are requested up front; tile kt + 1 (kt >= 1) in the first memory phase of k-tile kt, into
    // the stage that k-tile kt - 1 left behind the barrier before (both halves have read its last fragments
    // by then).  A wave waits for its loads of tile kt + 1 at the end of the phase before the one in which the
    // upper half reads that tile's first fragments: the upper half behind the MFMAs of k-tile kt's second
    // k-step, the lower half behind that k-step's fragment reads.
    gload(0);
    if (nkt > 1) {
        gload(1);
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
#endif
    } else {
        loads_landed();
    }
    phase_end();
    if (wm == 1) phase_end();   // the lower half runs one phase behind
    for (int kt = 0; kt < nkt; ++kt) {
        if constexpr (DB) {
            sum_a = db_cnt == db_rem;
            if (++db_cnt == db_mod) db_cnt = 0;
        }
        read_frags(kt, std::integral_constant<int, 0>{});
        if (kt >= 1 && kt + 1 < nkt) gload(kt + 1);
        landed();
        sum_frags();
        phase_end();
        compute();
        phase_end();
        read_frags(kt, std::integral_constant<int, 1>{});
        landed();
        sum_frags();
        if (wm == 1) loads_landed();
        phase_end();
        compute();
        if (wm == 0) loads_landed();
        phase_end();
    }
    if (wm == 0) phase_end();
    __syncthreads();   // every wave has read its last fragments: the LDS is free
}

// Stores the accumulated tile: fp32 partials of `split` when p.splits > 1, else bias + rounding,
// staged through LDS and written with 16-byte row-contiguous stores.
// STREAM: the C tile leaves with non-temporal stores.  A stand-alone product writes 128 KiB per workgroup
// that nothing reads again soon; as ordinary stores those lines displace the operand panels that the
// workgroups of an XCD share through its L2 (M = 32768, N = 8192, K = 2048: 1240 -> 1500 TFLOP/s).
// p.keep_c switches them off for an output that the next kernel reads back while the memory-side cache
// still holds it (the gates of a small-H recurrence: T = 1024, B = 256, H = 64, 128 MiB of gates: the
// time loop that follows runs 0.85 ms after ordinary stores, 1.13 ms after non-temporal ones).
template <typename T, int BM, int BN, int NS, int WVM, int WVN, int KSPT, bool STREAM = false>
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
    if constexpr (sizeof(T) == 4) {
        // fp32: a lane's 4 consecutive n are 16 bytes already, and the tile (256 KiB) would not fit the LDS:
        // stores straight from the accumulators, 64 bytes per row and instruction
        T *Cg = static_cast<T *>(p.C);
        const bool vec = (p.ldc & 3) == 0 && (p.N & 3) == 0 && (reinterpret_cast<size_t>(Cg) & 15) == 0;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int nb = n0 + (wn * TN + j) * 16 + q * 4;
            float b4[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias0)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (nb + e < p.N) b4[e] = bias0[nb + e] + (bias1 ? bias1[nb + e] : 0.f);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = m0 + (wm * TM + i) * 16 + r;
                if (m >= p.M || nb >= p.N) continue;
                f32x4 v = acc[i][j];
                v[0] += b4[0]; v[1] += b4[1]; v[2] += b4[2]; v[3] += b4[3];
                T *dst = Cg + (size_t)m * p.ldc + nb;
                if (vec && nb + 3 < p.N) {
                    if (STREAM && !p.keep_c) __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(dst));
                    else *reinterpret_cast<f32x4 *>(dst) = v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (nb + e < p.N) dst[e] = v[e];
                }
            }
        }
        return;
    }
    // the 4 bias elements of every tile column group: one 8-byte load each where the row of
    // biases allows it (all loads in flight together), element loads at a ragged edge
    float bv[TN][4];
    {
        u32x2 raw0[TN], raw1[TN];
        const bool vec = (p.N & 3) == 0 && ((reinterpret_cast<size_t>(bias0) | reinterpret_cast<size_t>(bias1)) & 7) == 0;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + (wn * TN + j) * 16 + q * 4;
            raw0[j] = raw1[j] = u32x2{0u, 0u};
            if (bias0 && vec && n < p.N) {
                raw0[j] = *reinterpret_cast<const u32x2 *>(bias0 + n);
                if (bias1) raw1[j] = *reinterpret_cast<const u32x2 *>(bias1 + n);
            } else if (bias0) {
                T t0[4], t1[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    t0[e] = n + e < p.N ? bias0[n + e] : Elem<T>::from_f32(0.f);
                    t1[e] = bias1 && n + e < p.N ? bias1[n + e] : Elem<T>::from_f32(0.f);
                }
                raw0[j] = *reinterpret_cast<u32x2 *>(t0);
                raw1[j] = *reinterpret_cast<u32x2 *>(t1);
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const T *t0 = reinterpret_cast<const T *>(&raw0[j]), *t1 = reinterpret_cast<const T *>(&raw1[j]);
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[j][e] = Elem<T>::to_f32(t0[e]) + Elem<T>::to_f32(t1[e]);
        }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int nl = (wn * TN + j) * 16 + q * 4;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int ml = (wm * TM + i) * 16 + r;
            const f32x4 v = acc[i][j];
            T pk[4] = {Elem<T>::from_f32(v[0] + bv[j][0]), Elem<T>::from_f32(v[1] + bv[j][1]),
                       Elem<T>::from_f32(v[2] + bv[j][2]), Elem<T>::from_f32(v[3] + bv[j][3])};
            *reinterpret_cast<u32x2 *>(smem + (size_t)ml * C::C_LD + nl * 2) = *reinterpret_cast<u32x2 *>(pk);
        }
    }
    __syncthreads();
    T *Cg = static_cast<T *>(p.C);
    constexpr int CPR = BN / 8;  // 16-byte chunks per C-tile row
    const bool vec_ok = (p.ldc & 7) == 0;
    if constexpr ((BM * CPR) % THREADS == 0 && THREADS % CPR == 0) {
        // a tile inside the matrix: all reads of a thread in flight, then all its stores (the guarded
        // loop below waits for one LDS read per store)
        if (vec_ok && m0 + BM <= p.M && n0 + BN <= p.N) {
            constexpr int IT = BM * CPR / THREADS, RPI = THREADS / CPR;   // iterations; rows per iteration
            const int ml0 = tid / CPR, nc = tid % CPR;
            const unsigned char *src = smem + (size_t)ml0 * C::C_LD + nc * 16;
            T *dst = Cg + (size_t)(m0 + ml0) * p.ldc + n0 + nc * 8;
            u32x4 v[IT];
#pragma unroll
            for (int it = 0; it < IT; ++it) v[it] = *reinterpret_cast<const u32x4 *>(src + (size_t)it * RPI * C::C_LD);
            if (STREAM && !p.keep_c) {
#pragma unroll
                for (int it = 0; it < IT; ++it)
                    __builtin_nontemporal_store(v[it], reinterpret_cast<u32x4 *>(dst + (size_t)it * RPI * p.ldc));
            } else {
#pragma unroll
                for (int it = 0; it < IT; ++it) *reinterpret_cast<u32x4 *>(dst + (size_t)it * RPI * p.ldc) = v[it];
            }
            return;
        }
    }
    for (int c = tid; c < BM * CPR; c += THREADS) {
        const int ml = c / CPR, nc = c % CPR;
        const int m = m0 + ml, n = n0 + nc * 8;
        if (m >= p.M || n >= p.N) continue;
        const u32x4 v = *reinterpret_cast<const u32x4 *>(smem + (size_t)ml * C::C_LD + nc * 16);
        T *dst = Cg + (size_t)m * p.ldc + n;
        if (vec_ok && n + 8 <= p.N) {
            if (STREAM && !p.keep_c) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(dst));
            else *reinterpret_cast<u32x4 *>(dst) = v;
        } else {
            const T *tv = reinterpret_cast<const T *>(&v);
            for (int e = 0; e < 8; ++e)
                if (n + e < p.N) dst[e] = tv[e];
        }
    }
}

// The C tile of an interior 256 x 256 tile (16-bit types, no split) straight from the accumulators: no LDS
// staging, no barrier, and nothing waits for the stores -- a persistent workgroup goes on to its next tile
// while they drain.  Lane (q, r) holds C[row r][4q .. 4q+3] of each 16 x 16 tile.  Two neighbouring tiles swap
// halves between the lane groups q and q ^ 1 (v_permlane16_swap), which leaves every lane with 8 consecutive
// columns (16 bytes) of one of them; the two 64-byte packets of a row then trade places between rows r and
// r ^ 8 (DPP), so that one store instruction writes 8 rows x 128 bytes: whole cache lines.
// Same values as gemm16_epilogue (bias added in fp32, one rounding).
template <typename T>
__device__ __forceinline__ void gemm16_epilogue_direct(const GemmParams &p, const int m0, const int n0,
                                                       const f32x4 (&acc)[8][4]) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane >> 4, r = lane & 15, wm = wave >> 2, wn = wave & 3;
    const T *bias0 = static_cast<const T *>(p.bias0), *bias1 = static_cast<const T *>(p.bias1);
    float bv[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        u32x2 raw0 = {0u, 0u}, raw1 = {0u, 0u};
        const int n = n0 + (wn * 4 + j) * 16 + q * 4;
        if (bias0) raw0 = *reinterpret_cast<const u32x2 *>(bias0 + n);
        if (bias0 && bias1) raw1 = *reinterpret_cast<const u32x2 *>(bias1 + n);
        const T *t0 = reinterpret_cast<const T *>(&raw0), *t1 = reinterpret_cast<const T *>(&raw1);
#pragma unroll
        for (int e = 0; e < 4; ++e) bv[j][e] = Elem<T>::to_f32(t0[e]) + Elem<T>::to_f32(t1[e]);
    }
    const __amdgpu_buffer_rsrc_t rc =
        __builtin_amdgcn_make_buffer_rsrc(p.C, 0, (unsigned)((size_t)p.M * p.ldc * sizeof(T)), 0x00020000);
    const bool hi = r >= 8;
    const unsigned colb = (unsigned)(n0 + wn * 64 + (hi ? 32 : 0) + (q & 1) * 16 + (q >> 1) * 8);
    const int aux = p.keep_c ? 0 : 2;   // 2: non-temporal
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        u32x4 pkt[2];
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            const f32x4 v0 = acc[i][2 * jp], v1 = acc[i][2 * jp + 1];
            T pk0[4] = {Elem<T>::from_f32(v0[0] + bv[2 * jp][0]), Elem<T>::from_f32(v0[1] + bv[2 * jp][1]),
                        Elem<T>::from_f32(v0[2] + bv[2 * jp][2]), Elem<T>::from_f32(v0[3] + bv[2 * jp][3])};
            T pk1[4] = {Elem<T>::from_f32(v1[0] + bv[2 * jp + 1][0]), Elem<T>::from_f32(v1[1] + bv[2 * jp + 1][1]),
                        Elem<T>::from_f32(v1[2] + bv[2 * jp + 1][2]), Elem<T>::from_f32(v1[3] + bv[2 * jp + 1][3])};
            const u32x2 a = *reinterpret_cast<u32x2 *>(pk0), b = *reinterpret_cast<u32x2 *>(pk1);
            // lane group q: tile 2 jp + (q & 1), columns 8 (q >> 1) .. + 7
            const u32x2 s0 = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);
            const u32x2 s1 = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
            pkt[jp] = u32x4{s0[0], s1[0], s0[1], s1[1]};
        }
        // rows r < 8 keep their columns 0 .. 31 and take those of row r + 8; rows r >= 8 keep their columns 32 .. 63
        // and take those of row r - 8
        const u32x4 snd = hi ? pkt[0] : pkt[1];
        u32x4 rcv;
#pragma unroll
        for (int e = 0; e < 4; ++e) rcv[e] = (unsigned)__builtin_amdgcn_update_dpp(0, (int)snd[e], 0x128 /* row_ror:8 */, 0xf, 0xf, false);
        const u32x4 first = hi ? rcv : pkt[0], second = hi ? pkt[1] : rcv;   // rows (r & 7) and (r & 7) + 8 of the 16
        const unsigned row0 = (unsigned)(m0 + (wm * 8 + i) * 16 + (r & 7));
        const unsigned off = (row0 * (unsigned)p.ldc + colb) * (unsigned)sizeof(T);
        if (aux) {
            __builtin_amdgcn_raw_buffer_store_b128(first, rc, off, 0, 2);
            __builtin_amdgcn_raw_buffer_store_b128(second, rc, off + 8u * (unsigned)p.ldc * (unsigned)sizeof(T), 0, 2);
        } else {
            __builtin_amdgcn_raw_buffer_store_b128(first, rc, off, 0, 0);
            __builtin_amdgcn_raw_buffer_store_b128(second, rc, off + 8u * (unsigned)p.ldc * (unsigned)sizeof(T), 0, 0);
        }
    }
#else
    (void)p; (void)m0; (void)n0; (void)acc;
#endif
}

// One BM x BN tile of C (rows m0.., columns n0.., K range of `split`): main loop + epilogue.
// ALONE: the tile of a stand-alone GEMM launch (streaming stores); PP: the ping-pong main loop where the
// configuration has one.
template <typename T, bool A_KM, bool B_KM, int BM, int BN, int NS, int WVM, int WVN, int KSPT, bool ALONE = false,
          bool PP = ALONE>
__device__ __forceinline__ bool gemm16_tile(const GemmParams &p, const int m0, const int n0, const int split,
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
    const int k_end = (A_KM && B_KM) ? (p.K + 63) / 64 * 64 : p.K;   // (rows past K read as zeros)
    if constexpr (PP && BM == 256 && BN == 256 && NS == 2 && WVM == 2 && WVN == 4 && KSPT == 2)
        gemm16_mainloop_pp<T, A_KM, B_KM>(p, m0, n0, kb, min(k_end, kb + p.k_per_split), smem, acc);
    else
        gemm16_mainloop<T, A_KM, B_KM, BM, BN, NS, WVM, WVN, KSPT>(p, m0, n0, kb, min(k_end, kb + p.k_per_split), smem, acc);
    if (p.trace) t_epi = (long long)wall_clock64();
    bool lds_used = true;   // (by the epilogue: a caller that goes on to another tile has to wait for its readers)
    if constexpr (ALONE && sizeof(T) == 2 && BM == 256 && BN == 256 && WVM == 2 && WVN == 4) {
        // the whole tile inside C, rows that take 16-byte stores, biases that take 8-byte loads (or none)
        const bool direct = p.splits == 1 && m0 + BM <= p.M && n0 + BN <= p.N && (p.ldc & 7) == 0 &&
                            (reinterpret_cast<size_t>(p.C) & 15) == 0 && (size_t)p.M * p.ldc * sizeof(T) < ((size_t)1 << 32) &&
                            ((reinterpret_cast<size_t>(p.bias0) | reinterpret_cast<size_t>(p.bias1)) & 7) == 0;
        if (direct) {
            gemm16_epilogue_direct<T>(p, m0, n0, acc);
            lds_used = false;
        } else {
            gemm16_epilogue<T, BM, BN, NS, WVM, WVN, KSPT, ALONE>(p, m0, n0, split, smem, acc);
        }
    } else {
        gemm16_epilogue<T, BM, BN, NS, WVM, WVN, KSPT, ALONE>(p, m0, n0, split, smem, acc);
        lds_used = !(sizeof(T) == 4 || p.splits > 1);   // (those store from the accumulators)
    }
    if (p.trace && threadIdx.x == 0) {   // stamps: start, main loop entered (= start), main loop left, done
        long long *t = p.trace + (size_t)trace_slot * 4;
        t[0] = t_start; t[1] = t_start; t[2] = t_epi; t[3] = (long long)wall_clock64();
    }
    return lds_used;
}

template <typename T, bool A_KM, bool B_KM, int BM, int BN, int NS, int WVM, int WVN, int KSPT>
__global__ __launch_bounds__(64 * WVM * WVN) void gemm16_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tiles_n = cdiv(p.N, BN), tiles_m = cdiv(p.M, BM);
    const int total = tiles_m * tiles_n * p.splits;
    // A launch with more tiles than the device has CUs is a grid of one workgroup per CU that walks through the
    // tile list (tile b, b + gridDim.x, ...: the tiles that a one-tile-per-workgroup launch would run together
    // still do, on the same XCDs): a workgroup starts its next tile while the stores of the last one drain.
    for (int b = blockIdx.x; b < total; b += gridDim.x) {
        int bid = b;
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
        const bool lds_used = gemm16_tile<T, A_KM, B_KM, BM, BN, NS, WVM, WVN, KSPT, true>(p, m0, n0, split, smem, b);
        if (lds_used && b + (int)gridDim.x < total) __syncthreads();   // the staged C tile was read: the stages are free
    }
}

// One tile per workgroup, symmetric main loop, C staged through LDS and written with ordinary stores: the tile
// kernel as it was before the ping-pong loop, the register epilogue and the persistent tile loop (the same tile
// function, other template arguments).  Two uses: measurements that time both forms in one process
// (set_gemm_baseline), and one round of tiles of a product of two K-major operands, where the symmetric loop is
// the faster one (M = 8192, N = 2048, K = 32768, bf16: 817 us against 845 us for the ping-pong loop).
template <typename T, bool A_KM, bool B_KM>
__global__ __launch_bounds__(512) void gemm16_onetile_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tiles_n = cdiv(p.N, 256), tiles_m = cdiv(p.M, 256);
    int bid = blockIdx.x;
    const int split = bid / (tiles_m * tiles_n);
    bid -= split * tiles_m * tiles_n;
    constexpr int GM = 8;
    const int lin = xcd_major_id(bid, tiles_m * tiles_n);
    const int per_group = GM * tiles_n, first_m = (lin / per_group) * GM;
    const int gsz = min(tiles_m - first_m, GM);
    const int m0 = (first_m + (lin % per_group) % gsz) * 256, n0 = ((lin % per_group) / gsz) * 256;
    gemm16_tile<T, A_KM, B_KM, 256, 256, 2, 2, 4, 2, false, false>(p, m0, n0, split, smem, (int)blockIdx.x);
}

// Both weight-gradient products and the bias gradient of a layer in one launch:
//     dWx[M][I] = A^T . x,   dWh[M][H] = A^T . h,   db[M] = column sums of A        (A = d_ifgo[K][M], K = T*B rows)
// as one tile grid over [M] x [I | H]: the column tiles of the h product follow those of the x product, so the
// A panels are shared by both products in the L2 and one split factor fills the device for both.  (h.N == 0:
// the x product alone.)  Column tile nt of the grid sums the A fragments of the k-tiles congruent to nt modulo
// the number of column tiles into db_part[split][nt][M] (gemm16_mainloop_pp, DB).  With splits > 1 the
// products are fp32 partials per split as well; wgrad_reduce_kernel adds everything up in a fixed order.
struct WgradParams {
    GemmParams x, h;    // A, M, K, lda, splits, k_per_split agree; C / Cpart / B / N / ldb / ldc per product
    int tiles_nx;       // column tiles of the x product
    float *db_part;     // [splits][column tiles][M], or nullptr: no bias gradient
};

template <typename T> __global__ __launch_bounds__(512) void gemm16_wgrad_kernel(const WgradParams w) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tiles_m = cdiv(w.x.M, 256), tiles_n = w.tiles_nx + cdiv(w.h.N, 256);
    int bid = blockIdx.x;
    const int split = bid / (tiles_m * tiles_n);
    bid -= split * tiles_m * tiles_n;
    constexpr int GM = 8;
    const int lin = xcd_major_id(bid, tiles_m * tiles_n);
    const int per_group = GM * tiles_n, first_m = (lin / per_group) * GM;
    const int gsz = min(tiles_m - first_m, GM);
    const int m0 = (first_m + (lin % per_group) % gsz) * 256, nt = (lin % per_group) / gsz;
    const bool second = nt >= w.tiles_nx;
    GemmParams p = w.x;
    if (second) {
        p.B = w.h.B; p.C = w.h.C; p.Cpart = w.h.Cpart;
        p.N = w.h.N; p.ldb = w.h.ldb; p.ldc = w.h.ldc;
    }
    const int n0 = (second ? nt - w.tiles_nx : nt) * 256;
    f32x4 acc[8][4];
    float colsum[2] = {0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int kb = split * p.k_per_split, k_end = (p.K + 63) / 64 * 64;   // (rows past K read as zeros)
    // (no bias gradient wanted: remainder -1 never comes up)
    gemm16_mainloop_pp<T, true, true, true>(p, m0, n0, kb, min(k_end, kb + p.k_per_split), smem, acc, colsum, tiles_n,
                                            w.db_part ? nt : -1);
    bool direct = false;
    if constexpr (sizeof(T) == 2)
        direct = p.splits == 1 && m0 + 256 <= p.M && n0 + 256 <= p.N && (p.ldc & 7) == 0 &&
                 (reinterpret_cast<size_t>(p.C) & 15) == 0 && (size_t)p.M * p.ldc * sizeof(T) < ((size_t)1 << 32);
    if (direct) {
        if constexpr (sizeof(T) == 2) gemm16_epilogue_direct<T>(p, m0, n0, acc);   // (no biases in these products)
    } else {
        gemm16_epilogue<T, 256, 256, 2, 2, 4, 2, true>(p, m0, n0, split, smem, acc);
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (w.db_part) {
        // lane (q, r) holds the sum over its k-groups for row r of its two fragments: add the four lane groups
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            float v = colsum[i];
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            const int m = m0 + ((wave >> 2) * 8 + (wave & 3) * 2 + i) * 16 + (lane & 15);
            if (lane < 16 && m < p.M) w.db_part[((size_t)split * tiles_n + nt) * p.M + m] = v;
        }
    }
}

// Finishes a weight-gradient launch: out = the sum over splits of the fp32 partials, in split order, for dWx
// (M x I) and dWh (M x H) -- not called for with splits == 1, then I = H = 0 here -- and db (M) = the sum of its
// db_parts partial sums.  A thread owns four consecutive elements of a matrix (I and H are multiples of 8) or
// one element of db.
template <typename T>
__global__ void wgrad_reduce_kernel(const float *part_x, T *dWx, const float *part_h, T *dWh, const float *part_db, T *db,
                                    int M, int I, int H, int splits, int db_parts) {
    const size_t qx = (size_t)M * I / 4, qh = (size_t)M * H / 4;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const float *part;
    T *out;
    size_t total;
    if (i < qx) { part = part_x; out = dWx; total = (size_t)M * I; }
    else if (i < qx + qh) { i -= qx; part = part_h; out = dWh; total = (size_t)M * H; }
    else {
        i -= qx + qh;
        if (i >= (size_t)M || !db) return;
        float s = 0.f;
        for (int k = 0; k < db_parts; ++k) s += part_db[(size_t)k * M + i];
        db[i] = Elem<T>::from_f32(s);
        return;
    }
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < splits; ++k) s += *reinterpret_cast<const f32x4 *>(part + (size_t)k * total + i * 4);
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<f32x4 *>(out + i * 4) = s;
    } else {
        T o[4] = {Elem<T>::from_f32(s[0]), Elem<T>::from_f32(s[1]), Elem<T>::from_f32(s[2]), Elem<T>::from_f32(s[3])};
        *reinterpret_cast<u32x2 *>(out + i * 4) = *reinterpret_cast<u32x2 *>(o);
    }
}

}  // namespace fastlstm

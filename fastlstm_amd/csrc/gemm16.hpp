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
    const int k_end = (A_KM && B_KM) ? (p.K + 63) / 64 * 64 : p.K;   // (rows past K read as zeros)
    gemm16_mainloop<T, A_KM, B_KM, BM, BN, NS, WVM, WVN, KSPT>(p, m0, n0, kb, min(k_end, kb + p.k_per_split), smem, acc);
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

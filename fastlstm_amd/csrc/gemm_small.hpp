// The reverse pass's three products and the bias gradient for a narrow layer, in ONE pass over d_ifgo:
//     dx[R][I]  = d_ifgo . Wx                    (K5)
//     dWx[G][I] = d_ifgo^T . x,  dWh[G][H] = d_ifgo^T . h,  db[G] = column sums of d_ifgo      (K8, K9, db)
// for G = 4H <= 256, I <= 64, H <= 64 (multiples of 16), 16-bit elements, R = T*B rows.  With rows this short
// every product is bound by the memory traffic of d_ifgo (a row of d_ifgo is 4 to 8 times as wide as the rows
// of x, h and dx together), and as four launches d_ifgo is read four times.  Here a workgroup takes blocks of
// 64 rows: it brings the block of d_ifgo (<= 32 KiB) and the matching blocks of x and h into LDS ONCE and uses
// it for all of them:
//     K-major (transposing reads, k = row)  -> dW tiles: wave w owns G tiles 2w, 2w + 1 x all column tiles, the
//                                              accumulators stay in registers over all blocks of the workgroup;
//                                              the bias gradient is one more column tile against a fragment of ones
//     row-major (k = gate column)           -> the block's 64 x I tile of dx against W_x fragments held in registers
// The partial weight gradients of the workgroups (fp32) are added up in a fixed order by small_bwd_reduce_kernel.
// Loads are LDS-direct, two stages: the next block is in flight while this one is multiplied.
#pragma once
#include "gemm16.hpp"

namespace fastlstm {

struct SmallBwdParams {
    const void *d_ifgo, *Wx, *x, *h;   // [R][G], [G][I], [R][I], [R][H]
    void *dx;                          // [R][I], or nullptr: not wanted
    float *part;                       // [workers][G * (I + H + 1)] fp32: dWx | dWh | db of each worker; nullptr: not wanted
    int R, G, I, H;
};

constexpr int kSmallRows = 64;                                   // rows of a block
constexpr int kSmallDBytes = kSmallRows * 512, kSmallXBytes = kSmallRows * 128;
constexpr int kSmallStage = kSmallDBytes + 2 * kSmallXBytes;     // d_ifgo | x | h blocks
constexpr int kSmallLdsBytes = 2 * kSmallStage;

// two transposing reads OFF2 bytes apart (4 k-rows), see lds_rd_tr16x2
template <int OFF2> __device__ __forceinline__ u32x4 lds_rd_tr16_pair(unsigned addr) {
    u32x2 lo = {0u, 0u}, hi = {0u, 0u};
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(addr));
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(OFF2));
#else
    (void)addr;
#endif
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
}

template <int N> __device__ __forceinline__ void small_frags_landed(u32x4 (&f)[N]) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < N; ++i) asm volatile("" : "+v"(f[i]));
#else
    (void)f;
#endif
}

// Worker `worker` of `n_workers` takes blocks worker, worker + n_workers, ... (counted from the last rows down when
// `from_end`: the order in which a reverse recurrence produces them).  gate(first_row, rows) is called before a
// block's loads are requested; a caller that runs next to the producer of d_ifgo waits there.  512 threads,
// kSmallLdsBytes of LDS at smem; ends behind a workgroup barrier.
template <typename T, typename Gate>
__device__ __forceinline__ void small_bwd_pass(const SmallBwdParams &p, unsigned char *smem, const int worker,
                                               const int n_workers, const bool from_end, Gate gate) {
    static_assert(sizeof(T) == 2, "16-bit element types");
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = lane >> 4, r = lane & 15, a = r >> 2, b = r & 3;
    const unsigned lds0 = (unsigned)(size_t)((FASTLSTM_LDS_PTR unsigned char *)smem);
    const bool want_w = p.part != nullptr, want_dx = p.dx != nullptr;
    const int G = p.G, I = p.I, H = p.H, R = p.R;
    const int nblk = (R + kSmallRows - 1) / kSmallRows;

    auto rsrc_of = [](const void *base, unsigned bytes) {
        const unsigned long long ad = reinterpret_cast<unsigned long long>(base);
        return u32x4{(unsigned)ad, (unsigned)(ad >> 32) & 0xffffu, bytes, 0x00020000u};
    };
    const u32x4 rd = rsrc_of(p.d_ifgo, (unsigned)((size_t)R * G * 2)), rx = rsrc_of(p.x, (unsigned)((size_t)R * I * 2));
    const u32x4 rh = rsrc_of(p.h, (unsigned)((size_t)R * H * 2)), rw = rsrc_of(p.Wx, (unsigned)((size_t)G * I * 2));
    // XOR swizzles of the 16-byte chunk index of a row, as functions of the row: the rows that the lanes of one
    // transposing read touch (k, k + 1, k + 2, k + 3 and the same eight rows on) land in different banks.
    // Rows of 512 bytes (d_ifgo) and rows of 128 bytes (x, h, W_x).
    auto swzd = [](int k) { return ((k & 3) << 1) ^ (((k >> 3) & 1) << 3); };
    auto swzx = [](int k) { return (((k >> 1) & 1) | (((k >> 3) & 1) << 1)) << 1; };
    constexpr unsigned kOut = 0xfffffff0u;   // an offset outside every operand: the load returns zeros

    // ---- global -> LDS.  One wave instruction fills 1 KiB: lane l the 16 bytes at 16 l.  d_ifgo: 32 blocks of two
    // rows each, wave w fills blocks w, w + 8, w + 16, w + 24 (rows 2w + 16j + l / 32); x, h: 8 blocks of 8 rows, one per wave.
    const int d_row = 2 * wave + (lane >> 5), d_c = (lane & 31) ^ swzd(d_row);
    const int x_row = 8 * wave + (lane >> 3), x_c = (lane & 7) ^ swzx(x_row);
    const bool d_ok = d_c * 8 < G, x_ok = x_c * 8 < I, h_ok = x_c * 8 < H;
    auto issue = [&](int row0, int stage) {
        const unsigned sd = lds0 + stage * kSmallStage + wave * kFragBytes;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned off = (unsigned)(((size_t)(row0 + d_row + 16 * j) * G + d_c * 8) * 2);
            dma_block_asm<false>(rd, sd + j * 8 * kFragBytes, d_ok ? off : kOut, 0u);
        }
        const unsigned sx = lds0 + stage * kSmallStage + kSmallDBytes + wave * kFragBytes;
        if (want_w) {
            const unsigned offx = (unsigned)(((size_t)(row0 + x_row) * I + x_c * 8) * 2);
            const unsigned offh = (unsigned)(((size_t)(row0 + x_row) * H + x_c * 8) * 2);
            dma_block_asm<false>(rx, sx, x_ok ? offx : kOut, 0u);
            dma_block_asm<false>(rh, sx + kSmallXBytes, h_ok ? offh : kOut, 0u);
        }
    };
    auto loads_landed = [&]() {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
        __syncthreads();
    };

    // ---- fragment addresses.  Transposing reads: lane (a, b) of a 16-lane group addresses 4 consecutive columns
    // (8 bytes) of row k = 8q + a; the second read takes rows k + 4 (same swizzle).
    const int k0 = q * 8 + a;   // + 32 ks
    auto tr_d = [&](unsigned stage_base, int gt, int ks) {
        const int k = ks * 32 + k0;
        return lds_rd_tr16_pair<4 * 512>(stage_base + (unsigned)(k * 512 + (((gt * 2 + (b >> 1)) ^ swzd(k)) * 16) + (b & 1) * 8));
    };
    auto tr_x = [&](unsigned base, int ct, int ks) {
        const int k = ks * 32 + k0;
        return lds_rd_tr16_pair<4 * 128>(base + (unsigned)(k * 128 + (((ct * 2 + (b >> 1)) ^ swzx(k)) * 16) + (b & 1) * 8));
    };

    // ---- W_x as MFMA fragments in registers (dx): through LDS once, in the layout of an x block of 256 rows
    const int rt = wave & 3, ct0 = 2 * (wave >> 2);   // dx: row tile and first of two column tiles of this wave
    u32x4 wx[2][8];
    if (want_dx) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int g = 8 * (wave + 8 * j) + (lane >> 3);
            const unsigned off = (unsigned)(((size_t)g * I + x_c * 8) * 2);   // (g >= G: outside the operand)
            dma_block_asm<false>(rw, lds0 + (wave + 8 * j) * kFragBytes, x_ok ? off : kOut, 0u);
        }
        loads_landed();
#pragma unroll
        for (int c = 0; c < 2; ++c) {
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) wx[c][ks] = tr_x(lds0, ct0 + c, ks);
            small_frags_landed(wx[c]);
        }
        __syncthreads();
    }

    f32x4 accx[2][4], acch[2][4], accb[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        accb[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c) accx[t][c] = acch[t][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    u32x4 ones;
    if constexpr (Elem<T>::DT == FASTLSTM_FP16) ones = u32x4{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
    else ones = u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    const int gt0 = 2 * wave;
    const bool g_on[2] = {gt0 * 16 < G, (gt0 + 1) * 16 < G};
    const int nxt = I / 16, nht = H / 16;

    auto row0_of = [&](int blk) { return (from_end ? nblk - 1 - blk : blk) * kSmallRows; };
    int blk = worker;
    if (blk < nblk) {
        gate(row0_of(blk), kSmallRows);
        issue(row0_of(blk), 0);
    }
    for (int n = 0; blk < nblk; blk += n_workers, ++n) {
        const int stage = n & 1, row0 = row0_of(blk);
        loads_landed();   // this block is in LDS; every wave is done with the other stage
        if (blk + n_workers < nblk) {
            gate(row0_of(blk + n_workers), kSmallRows);
            issue(row0_of(blk + n_workers), stage ^ 1);
        }
        const unsigned sd = lds0 + stage * kSmallStage, sx = sd + kSmallDBytes, sh = sx + kSmallXBytes;
        if (want_w && g_on[0]) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                u32x4 f[10];   // d^T fragments of the two G tiles, x and h fragments of the column tiles
                f[0] = tr_d(sd, gt0, ks);
                f[1] = tr_d(sd, gt0 + 1, ks);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    f[2 + c] = tr_x(sx, c, ks);
                    f[6 + c] = tr_x(sh, c, ks);
                }
                small_frags_landed(f);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    if (!g_on[t]) continue;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        if (c < nxt) accx[t][c] = mfma_kstep<T>(f[2 + c], f[t], accx[t][c]);
                        if (c < nht) acch[t][c] = mfma_kstep<T>(f[6 + c], f[t], acch[t][c]);
                    }
                    accb[t] = mfma_kstep<T>(ones, f[t], accb[t]);
                }
            }
        }
        if (want_dx && ct0 < nxt) {
            u32x4 f[8];   // rows rt*16 + r of the block, all of G
            const int row = rt * 16 + r;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) f[ks] = lds_rd128<0>(sd + (unsigned)(row * 512 + (((ks * 4 + q) ^ swzd(row)) * 16)));
            small_frags_landed(f);
            f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                if (ks * 32 >= G) continue;
                acc[0] = mfma_kstep<T>(wx[0][ks], f[ks], acc[0]);
                acc[1] = mfma_kstep<T>(wx[1][ks], f[ks], acc[1]);
            }
            // lane (q, r): dx[row0 + 16 rt + r][16 (ct0 + c) + 4q .. + 3]
            if (row0 + row < R) {
                T *dst = static_cast<T *>(p.dx) + (size_t)(row0 + row) * I + ct0 * 16 + 4 * q;
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    if (ct0 + c >= nxt) continue;
                    typedef T tx4 __attribute__((ext_vector_type(4)));
                    const tx4 v = {Elem<T>::from_f32(acc[c][0]), Elem<T>::from_f32(acc[c][1]), Elem<T>::from_f32(acc[c][2]),
                                   Elem<T>::from_f32(acc[c][3])};
                    *reinterpret_cast<tx4 *>(dst + c * 16) = v;
                }
            }
        }
    }
    __syncthreads();
    if (want_w) {
        // lane (q, r): dW[16 (gt0 + t) + r][16 c + 4q .. + 3]
        float *part = p.part + (size_t)worker * G * (I + H + 1);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (!g_on[t]) continue;
            const int g = (gt0 + t) * 16 + r;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (c < nxt) *reinterpret_cast<f32x4 *>(part + (size_t)g * I + c * 16 + 4 * q) = accx[t][c];
                if (c < nht) *reinterpret_cast<f32x4 *>(part + (size_t)G * I + (size_t)g * H + c * 16 + 4 * q) = acch[t][c];
            }
            if (q == 0) part[(size_t)G * (I + H) + g] = accb[t][0];
        }
    }
}

template <typename T> __global__ __launch_bounds__(512) void small_bwd_kernel(const SmallBwdParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    small_bwd_pass<T>(p, smem, (int)blockIdx.x, (int)gridDim.x, false, [](int, int) {});
}

// dWx | dWh | db = the sum over the workers' partial sums, in worker order.  A thread block takes 32 groups of four
// consecutive sums; its 8 x 32 threads add every eighth worker each and then the eight slices in order.
template <typename T>
__global__ __launch_bounds__(256) void small_bwd_reduce_kernel(const float *part, T *dWx, T *dWh, T *db, int G, int I, int H,
                                                               int workers) {
    __shared__ f32x4 sm[8][32];
    const int S = G * (I + H + 1), quad = blockIdx.x * 32 + (threadIdx.x & 31), sl = threadIdx.x >> 5;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    if (quad * 4 < S) {
        const float *src = part + (size_t)sl * S + quad * 4;
        int w = sl;
        for (; w + 24 < workers; w += 32, src += (size_t)32 * S) {   // four loads in flight per thread
            const f32x4 a = *reinterpret_cast<const f32x4 *>(src), b = *reinterpret_cast<const f32x4 *>(src + (size_t)8 * S);
            const f32x4 c = *reinterpret_cast<const f32x4 *>(src + (size_t)16 * S), d = *reinterpret_cast<const f32x4 *>(src + (size_t)24 * S);
            s += a; s += b; s += c; s += d;
        }
        for (; w < workers; w += 8, src += (size_t)8 * S) s += *reinterpret_cast<const f32x4 *>(src);
    }
    sm[sl][threadIdx.x & 31] = s;
    __syncthreads();
    if (sl != 0 || quad * 4 >= S) return;
#pragma unroll
    for (int i = 1; i < 8; ++i) s += sm[i][threadIdx.x & 31];
    const int e = quad * 4;
    T *out = e < G * I ? dWx + e : e < G * (I + H) ? dWh + (e - G * I) : db + (e - G * (I + H));
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = Elem<T>::from_f32(s[i]);
}

// K1 of a narrow layer: ifgo[R][G] = x[R][I] . Wx[G][I]^T + bx + bh for G = 4H <= 256, I <= 64 (multiples of 16),
// 16-bit elements -- a product that writes four to sixteen times what it reads and is bound by that write stream
// (~3 TB/s on this device).  The host takes it where I is no multiple of 64, which the tile kernel needs; where both
// apply the tile kernel is 10-30 % faster.
// Both operands are K-contiguous, so the MFMA fragments are 16-byte global loads (no LDS on the way in): a wave keeps
// the W_x fragments of its two G tiles and the bias sums in registers for the whole launch and streams blocks of 64
// rows of x, the next block's fragments in flight while this one is multiplied.  The results are the bits of the
// tile kernel (gemm16_kernel: the same two k-steps in the same order, bias added in fp32 before rounding); they
// leave through one of two LDS tiles as whole rows, 16 bytes per lane, with ordinary stores -- the time loop reads
// them next and finds them in the memory-side cache.
struct SmallK1Params {
    const void *x, *Wx, *bx, *bh;   // [R][I], [G][I], [G], [G]
    void *ifgo;                     // [R][G]
    int R, G, I;
};
constexpr int kSmallK1Row = 512 + 32;                      // bytes of a staged row (bank spread)
constexpr int kSmallK1LdsBytes = 2 * kSmallRows * kSmallK1Row;

template <typename T> __global__ __launch_bounds__(512) void small_k1_kernel(const SmallK1Params p) {
    static_assert(sizeof(T) == 2, "16-bit element types");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane >> 4, r = lane & 15;
    const int G = p.G, I = p.I, R = p.R;
    const int nblk = (R + kSmallRows - 1) / kSmallRows;
    const T *Wx = static_cast<const T *>(p.Wx), *bx = static_cast<const T *>(p.bx), *bh = static_cast<const T *>(p.bh);
    const u32x4 zero = {0u, 0u, 0u, 0u};
    // x and ifgo through buffer descriptors: a row past R reads as zeros and its stores are dropped, so every
    // load and store below is unconditional and the compiler's counted waits leave the stores of a block in flight
    // while the next block's fragments are awaited
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.x), 0, (unsigned)((size_t)R * I * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(p.ifgo, 0, (unsigned)((size_t)R * G * 2), 0x00020000);
    constexpr unsigned kOut = 0xfffffff0u;

    // this wave's two G tiles: fragments of W_x (lane (q, r): row 16 gt + r, k = 32 ks + 8q ..) and the bias sums of
    // the lane's four output columns 16 gt + 4q ..
    u32x4 wf[2][2];
    float bv[2][4];
    bool g_on[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int gt = 2 * wave + t, g = gt * 16 + r;
        g_on[t] = gt * 16 < G;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int k = ks * 32 + 8 * q;
            wf[t][ks] = (g < G && k < I) ? *reinterpret_cast<const u32x4 *>(Wx + (size_t)g * I + k) : zero;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int gc = gt * 16 + 4 * q + e;
            bv[t][e] = gc < G ? Elem<T>::to_f32(bx[gc]) + Elem<T>::to_f32(bh[gc]) : 0.f;
        }
    }
    // fragments of a block of x: lane (q, r): row 16 rt + r of the block, k = 32 ks + 8q .. (k past I: zeros)
    unsigned xoff[4][2];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int k = ks * 32 + 8 * q;
            xoff[rt][ks] = k < I ? (unsigned)(((rt * 16 + r) * I + k) * 2) : kOut;
        }
    u32x4 xf[4][2];
    auto load_x = [&](int blk) {
        const unsigned base = (unsigned)((size_t)blk * kSmallRows * I * 2);
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
                xf[rt][ks] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, xoff[rt][ks] == kOut ? kOut : xoff[rt][ks] + base, 0, 0));
    };
    // stores: 16-byte chunk c = tid + 512 j of the staged block -> row c / (G / 8), columns 8 (c % (G / 8)) ..
    const int cpr = G / 8;
    unsigned so_lds[4], so_glb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = tid + 512 * j, row = c / cpr, cc = c - row * cpr;
        const bool ok = c < kSmallRows * cpr;
        so_lds[j] = ok ? (unsigned)(row * kSmallK1Row + cc * 16) : 0u;
        so_glb[j] = ok ? (unsigned)((row * G + cc * 8) * 2) : kOut;
    }
    int blk = blockIdx.x;
    if (blk < nblk) load_x(blk);
    // (four stores outside the operand, which the hardware drops: the loop is then entered with the same sequence of
    // vector-memory operations in flight as it is re-entered with -- 8 loads, 4 stores -- and the compiler's counted
    // wait for the fragments leaves the 4 stores of the last block in flight instead of draining everything)
#pragma unroll
    for (int j = 0; j < 4; ++j) __builtin_amdgcn_raw_buffer_store_b128(zero, ro, kOut, 0, 0);
    for (int n = 0; blk < nblk; blk += gridDim.x, ++n) {
        unsigned char *st = smem + (n & 1) * kSmallRows * kSmallK1Row;
        f32x4 acc[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                acc[t][rt] = mfma_kstep<T>(wf[t][0], xf[rt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                acc[t][rt] = mfma_kstep<T>(wf[t][1], xf[rt][1], acc[t][rt]);
            }
        load_x(blk + gridDim.x);   // in flight behind the staging and the stores (past the last block: zeros, unused)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (!g_on[t]) continue;
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                // lane (q, r): ifgo[row 16 rt + r][16 gt + 4q .. + 3]
                typedef T tx4 __attribute__((ext_vector_type(4)));
                const tx4 v = {Elem<T>::from_f32(acc[t][rt][0] + bv[t][0]), Elem<T>::from_f32(acc[t][rt][1] + bv[t][1]),
                               Elem<T>::from_f32(acc[t][rt][2] + bv[t][2]), Elem<T>::from_f32(acc[t][rt][3] + bv[t][3])};
                *reinterpret_cast<tx4 *>(st + (rt * 16 + r) * kSmallK1Row + ((2 * wave + t) * 16 + 4 * q) * 2) = v;
            }
        }
        __syncthreads();   // the block is staged (and every wave is done reading the other tile: two barriers ago)
        const unsigned base = (unsigned)((size_t)blk * kSmallRows * G * 2);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(st + so_lds[j]), ro,
                                                   so_glb[j] == kOut ? kOut : so_glb[j] + base, 0, 0);
    }
}

}  // namespace fastlstm

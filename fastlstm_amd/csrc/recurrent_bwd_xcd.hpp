// Persistent reverse-time kernel, XCD-local form: the hidden tiles of one batch tile run on one XCD
// and exchange d_ifgo[t] through that XCD's L2.  Same mathematics and results as
// lstm_bwd_persistent_kernel (which replaces fastlstm/kernels.py:1201-1409); placement, exchange
// ring, L2 counter barrier and the register-resident weight slice follow lstm_fwd_xcd_kernel.
//
// Per reverse step s (timestep t = T-1-s) a workgroup of NWV waves, owning 16*MT hidden units and
// 16*NTW batch rows:
//   gate backward for its (unit, row) items -> d_ifgo[t] tile (LDS) and exchange slot s (L2)
//   counter barrier over the group
//   dh_rec(units, rows) = Wh[:, units]^T . d_ifgo[t](rows, :)^T over K = 4H:
//       the waves split K NWV ways; wave w holds A fragments (MT unit tiles x NKW k-steps
//       w, w + NWV, ...) of Wh^T in registers and requests its NKW*NTW operand blocks at once
//   cross-wave sum of the NWV partials through LDS
// K index = 4 * source unit + gate, as in the general kernel.
#pragma once
#include <type_traits>

#include "recurrent_fwd_xcd.hpp"

namespace fastlstm {

struct BwdXcdParams {
    const void *dout;   // [T,B,H]
    void *dh, *dc;      // [B,H] in: grads of h_T, c_T; out: grads of h_0, c_0
    const void *ifgo;   // [T,B,4H]
    const void *cell;   // [T+1,B,H]
    void *d_ifgo;       // [T,B,4H]
    const void *Wh;     // [4H,H]
    WsHeader *hdr;
    int *counters;         // [groups][kXcdReplicas][kXcdCounterStride], zero at launch
    unsigned char *xbuf;   // [2 slots][groups][NT][KSB] operand blocks; reverse step s uses slot s % 2
    int T, B, H;
    int n_ht, gpx, n_groups;
    int b_base;         // first batch row of this launch (a large batch runs as several launches over row ranges)
    int KSB;            // k-steps covering 4H
    // In-kernel dx = d_ifgo . Wx (HELP instantiations, k5_tiles_n > 0): the workgroups without a role
    // in the recurrence compute it in 256 x 256 tiles, latest timesteps first, as soon as the
    // recurrence has finished a chunk of k5_chunk_steps timesteps (k5_chunk_tiles row tiles);
    // chunk_done[c] counts the recurrence workgroups (n_active) whose part of chunk c is in memory.
    GemmParams k5;      // M = T*B, N = I, K = 4H, A = d_ifgo, B = Wx (K-major), C = dx
    // Bias gradient inside the launch (HELP instantiations, db_part != nullptr): every recurrence workgroup sums the
    // d_ifgo values it produces over all timesteps -- thread-private fp32 slots in LDS, updated behind the publish of
    // each step, while the workgroup waits for its peers anyway -- and writes the sums of its 16-row batch tiles to
    // db_part[batch tile][4H] at the end; a small kernel adds the batch tiles up.  The separate column-sum pass
    // over d_ifgo (one more read of T*B*4H elements) is not needed then.
    float *db_part, *db_part_lo;   // [ceil(B / 16)][4H] each; _lo: the lower layer of a stacked launch
    int db_lds_off;                // byte offset of the slots in the workgroup's LDS (behind the recurrence's own use)
    int k5_tail_by_rec; // 1: the dx tiles of the chunk that completes last (timesteps 0 ..) are computed by the recurrence
                        // workgroups once their time loop has ended, not by the helpers, which still owe that chunk's
                        // share of their weight-gradient tiles (single-layer launches)
    int k5_tiles_m, k5_tiles_n;
    int k5_chunk_tiles, k5_chunk_steps, k5_chunks;
    // In-kernel weight gradients (wg_tiles > 0): dWx = d_ifgo^T . x and dWh = d_ifgo^T . h, 256 x 256
    // output tiles, the first n_helpers of them one per helper: a helper adds the K range (rows of
    // T*B) of every finished chunk to its accumulators and stores the tile after the last chunk.
    GemmParams k8, k9;  // M = 4H, N = I | H, K = T*B, A = d_ifgo (K-major), B = x | h (K-major), C = dWx | dWh
    int k8_tiles_n, k9_tiles_n, wg_tiles_m, wg_tiles;
    int n_active;       // workgroups of one layer's recurrence
    int *chunk_done;    // [<= kMaxChunks] device-scope counters, zero at launch
    // Two stacked layers in one launch (n_layers == 2, HELP instantiations).  The fields above describe
    // the UPPER layer, whose groups come first in the group numbering.  The lower layer's recurrence
    // reads the upper layer's dx (k5.C) as its dout: the helpers write it chunk by chunk, latest
    // timesteps first (dx_done[c] counts the finished tiles of chunk c), and the lower recurrence
    // requests the dout of a timestep only when its chunk is complete.  The helpers also compute the
    // lower layer's dx (k5_lo, when its C is not null) behind that recurrence and, with wg_lo_tiles > 0,
    // the lower layer's weight gradients (k8_lo, k9_lo: the same scheme as k8, k9, one tile per helper
    // accumulated chunk by chunk as the lower recurrence finishes them); otherwise those are left to
    // the caller.
    int n_layers;       // (also 2, without helpers: two independent recurrences side by side, the second one described
                        // by the *_lo fields and k5.C = its dout)
    void *dh_lo, *dc_lo;
    const void *ifgo_lo, *cell_lo;
    void *d_ifgo_lo;
    const void *Wh_lo;
    GemmParams k5_lo;   // M = T*B, N = I of the lower layer, K = 4H, A = d_ifgo_lo, B = Wx_lo (K-major), C = dx_lo
    int k5_lo_tiles_n;
    int *chunk_done_lo; // [<= kMaxChunks]
    int *dx_done;       // [<= kMaxChunks]
    float *wg_scratch;  // stacked launches: 256 KiB per helper that owns a weight-gradient tile
    GemmParams k8_lo, k9_lo;   // the lower layer's dWx, dWh (A = d_ifgo_lo, B = its x | h)
    int k8_lo_tiles_n, wg_lo_tiles;
    float *wg_scratch_lo;
    long long spin_limit;
    // Without helpers, n_layers = 3 or 4 independent recurrences: recurrence r >= 2 is described by entry r - 2.
    const void *dout_more[2], *ifgo_more[2], *cell_more[2], *Wh_more[2];
    void *dh_more[2], *dc_more[2], *d_ifgo_more[2];
    unsigned char *partials;   // lstm_bwd_wide_split_kernel: the teams' partial sums (see there)
};

#ifndef FASTLSTM_HELPER_PP
#define FASTLSTM_HELPER_PP true   // the GEMM tiles inside the recurrent launches use the ping-pong main loop
#endif

// One 256 x 256 tile of dx = d_ifgo . Wx as a real function call.  The caller keeps the 128
// accumulator registers of its weight-gradient tile across the call: the calling convention saves
// and restores them around it (once per dx tile), where inlining would spill inside the GEMM
// loops of both products.  Arguments of a function arrive in vector registers; every one of them
// is the same in all lanes and goes back to scalar registers first.
template <typename T>
__device__ __attribute__((noinline)) void helper_dx_tile(const void *A, const void *B, void *C, int M, int N, int K,
                                                         int m0, int n0, FASTLSTM_LDS_PTR unsigned char *lds) {
    GemmParams g{};
    g.A = uniform_ptr(A); g.B = uniform_ptr(B); g.C = uniform_ptr(C);
    g.M = uniform_int(M); g.N = uniform_int(N); g.K = uniform_int(K);
    g.lda = g.K; g.ldb = g.N; g.ldc = g.N;
    g.splits = 1; g.k_per_split = g.K;
    unsigned char *smem = (unsigned char *)(FASTLSTM_LDS_PTR unsigned char *)(size_t)(unsigned)uniform_int((int)(size_t)lds);
    gemm16_tile<T, false, true, 256, 256, 2, 2, 4, 2, false, FASTLSTM_HELPER_PP>(g, uniform_int(m0), uniform_int(n0), 0, smem, 0);
    __syncthreads();   // the LDS is reused by the caller
}

// Stacked launch: one chunk's K range added to the helper's weight-gradient tile, whose fp32
// accumulators live in `park` (256 KiB, lane-major, 16-byte accesses) between the chunks; with
// `last` the tile is stored instead of parked.  A function call for the same reason as
// helper_dx_tile: inlined next to the stacked helper's other work, the GEMM loop spills.
template <typename T>
__device__ __attribute__((noinline)) void helper_wgrad_chunk(const void *A, const void *B, void *C, int M, int N, int K,
                                                             int ldb, int m0, int n0, int kb, int ke, f32x4 *park, int first,
                                                             int last, FASTLSTM_LDS_PTR unsigned char *lds) {
    constexpr int WVM = 2, WVN = 4, TM = 256 / WVM / 16, TN = 256 / WVN / 16;
    GemmParams g{};
    g.A = uniform_ptr(A); g.B = uniform_ptr(B); g.C = uniform_ptr(C);
    g.M = uniform_int(M); g.N = uniform_int(N); g.K = uniform_int(K);
    g.lda = g.M; g.ldb = uniform_int(ldb); g.ldc = g.N;
    g.splits = 1; g.k_per_split = g.K;
    unsigned char *smem = (unsigned char *)(FASTLSTM_LDS_PTR unsigned char *)(size_t)(unsigned)uniform_int((int)(size_t)lds);
    park = uniform_ptr(park) + threadIdx.x;
    m0 = uniform_int(m0); n0 = uniform_int(n0);
    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
            acc[i][j] = uniform_int(first) ? f32x4{0.f, 0.f, 0.f, 0.f} : park[(i * TN + j) * (kWave * 8)];
    if constexpr (FASTLSTM_HELPER_PP) gemm16_mainloop_pp<T, true, true>(g, m0, n0, uniform_int(kb), uniform_int(ke), smem, acc);
    else gemm16_mainloop<T, true, true, 256, 256, 2, WVM, WVN, 2>(g, m0, n0, uniform_int(kb), uniform_int(ke), smem, acc);
    if (uniform_int(last)) {
        gemm16_epilogue<T, 256, 256, 2, WVM, WVN, 2>(g, m0, n0, 0, smem, acc);
        __syncthreads();
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) park[(i * TN + j) * (kWave * 8)] = acc[i][j];
    }
}

// Stacked launch: waits until the lower layer has finished chunk c (the k-th in reverse time) and
// computes this helper's share of the chunk's dx tiles of the lower layer.  A function call for the
// same reason as helper_dx_tile.
template <typename T>
__device__ __attribute__((noinline)) void helper_lower_dx(int *chunk_done, int n_active, WsHeader *hdr, long long spin_limit,
                                                          const void *A, const void *B, void *C, int M, int N, int K,
                                                          int chunk_tiles, int tiles_n, int tiles_m, int c, int k, int h,
                                                          int n_helpers, FASTLSTM_LDS_PTR unsigned char *lds) {
    chunk_done = uniform_ptr(chunk_done); hdr = uniform_ptr(hdr);
    n_active = uniform_int(n_active); chunk_tiles = uniform_int(chunk_tiles); tiles_n = uniform_int(tiles_n);
    tiles_m = uniform_int(tiles_m); c = uniform_int(c); k = uniform_int(k); h = uniform_int(h); n_helpers = uniform_int(n_helpers);
    if ((threadIdx.x >> 6) == 0) wait_versions<100>(chunk_done, 1, n_active, hdr, spin_limit, -3, c);
    __syncthreads();
    if (!uniform_ptr(C)) return;
    const int per = chunk_tiles * tiles_n;
    for (int i = k * per + ((h - k * per) % n_helpers + n_helpers) % n_helpers; i < (k + 1) * per; i += n_helpers) {
        const int r = i - k * per;
        const int rt = c * chunk_tiles + r / tiles_n, ct = r % tiles_n;
        if (rt >= tiles_m) continue;
        helper_dx_tile<T>(A, B, C, M, N, K, rt * 256, ct * 256, lds);
    }
}

// The workgroups (8 waves) without a role in the recurrence.  Chunks of timesteps become available
// in reverse time order.  Helper h of n owns weight-gradient tile h (if there is one), which it
// accumulates chunk by chunk in registers, and takes the dx tiles h, h + n, ... of the list ordered
// by chunk.
// STACKED: two layers share the launch (a separate instantiation: the single-layer code keeps the
// register allocation of its GEMM loops).
template <typename T, bool STACKED>
__device__ __forceinline__ void bwd_helper(const BwdXcdParams &p, unsigned char *smem) {
    constexpr int WVM = 2, WVN = 4, TM = 256 / WVM / 16, TN = 256 / WVN / 16;   // 8 waves, 128 x 64 each
    int n_helpers;
    const int h = helper_rank(p.n_ht, p.gpx, p.n_groups * (STACKED ? 2 : 1), &n_helpers);
    const int per_chunk = p.k5_chunk_tiles * p.k5_tiles_n;
    // the weight-gradient tile of this helper: tiles of dWx first, then those of dWh
    const int n8 = p.wg_tiles_m * p.k8_tiles_n;
    const bool own = h < p.wg_tiles;
    const bool is8 = h < n8;
    const GemmParams &wp = is8 ? p.k8 : p.k9;
    const int wi = is8 ? h : h - n8, wtn = is8 ? p.k8_tiles_n : p.k9_tiles_n;
    const int wm0 = (wi / wtn) * 256, wn0 = (wi % wtn) * 256;
    constexpr bool stacked = STACKED;
    const int lag = 2;   // the lower layer's chunks are taken this many chunks behind the upper layer's
    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
#ifdef FASTLSTM_BWD_STAMPS
    long long *stamps = reinterpret_cast<long long *>(p.counters + 8192) + blockIdx.x * 4;
    long long waited = 0;
    if (threadIdx.x == 0) stamps[0] = (long long)wall_clock64();
#endif
    // the lower layer's dx tiles of the k-th chunk in reverse time, this helper's share
    auto lower_dx = [&](int k) {
        helper_lower_dx<T>(p.chunk_done_lo + (p.k5_chunks - 1 - k), p.n_active, p.hdr, p.spin_limit, p.k5_lo.A, p.k5_lo.B,
                           p.k5_lo.C, p.k5_lo.M, p.k5_lo.N, p.k5_lo.K, p.k5_chunk_tiles, p.k5_lo_tiles_n, p.k5_tiles_m,
                           p.k5_chunks - 1 - k, k, h, n_helpers, (FASTLSTM_LDS_PTR unsigned char *)smem);
    };
    // ... and the chunk's K range of this helper's weight-gradient tile of the lower layer
    const int n8_lo = p.wg_tiles_m * p.k8_lo_tiles_n;
    auto lower_wgrad = [&](int k) {
        if (!stacked || h >= p.wg_lo_tiles) return;
        const bool lo8 = h < n8_lo;
        const GemmParams &q = lo8 ? p.k8_lo : p.k9_lo;
        const int qi = lo8 ? h : h - n8_lo, qtn = lo8 ? p.k8_lo_tiles_n : p.k9_tiles_n;
        const int c = p.k5_chunks - 1 - k;
        const int kb = c * p.k5_chunk_tiles * 256, ke = min((q.K + 63) / 64 * 64, kb + p.k5_chunk_tiles * 256);   // (rows past K read as zeros)
        helper_wgrad_chunk<T>(q.A, q.B, q.C, q.M, q.N, q.K, q.ldb, (qi / qtn) * 256, (qi % qtn) * 256, kb, ke,
                              reinterpret_cast<f32x4 *>(p.wg_scratch_lo) + (size_t)h * (256 * 256 / 4), k == 0,
                              k + 1 == p.k5_chunks, (FASTLSTM_LDS_PTR unsigned char *)smem);
    };
    for (int k = 0; k < p.k5_chunks; ++k) {
        const int c = p.k5_chunks - 1 - k;   // chunk in forward time
        // d_ifgo of the chunk's timesteps is in memory once every recurrence workgroup said so
#ifdef FASTLSTM_BWD_STAMPS
        const long long w0 = (long long)wall_clock64();
#endif
        if ((threadIdx.x >> 6) == 0) wait_versions<100>(p.chunk_done + c, 1, p.n_active, p.hdr, p.spin_limit, -1, c);
        __syncthreads();
#ifdef FASTLSTM_BWD_STAMPS
        waited += (long long)wall_clock64() - w0;
        if (threadIdx.x == 0 && k == p.k5_chunks - 1) stamps[3] = (long long)wall_clock64();
#endif
        if (own) {
            const int kb = c * p.k5_chunk_tiles * 256, ke = min((wp.K + 63) / 64 * 64, kb + p.k5_chunk_tiles * 256);   // (rows past K read as zeros)
            if constexpr (STACKED) {
                helper_wgrad_chunk<T>(wp.A, wp.B, wp.C, wp.M, wp.N, wp.K, wp.ldb, wm0, wn0, kb, ke,
                                      reinterpret_cast<f32x4 *>(p.wg_scratch) + (size_t)h * (256 * 256 / 4), k == 0,
                                      k + 1 == p.k5_chunks, (FASTLSTM_LDS_PTR unsigned char *)smem);
            } else {
                int salt = 0;
                asm volatile("" : "+v"(salt));   // opaque zero: see gemm16_mainloop
                // (the symmetric loop: the ping-pong loop, inlined here with the accumulators live across the
                // calls around it, spills them inside its k loop)
                gemm16_mainloop<T, true, true, 256, 256, 2, WVM, WVN, 2>(wp, wm0, wn0, kb, ke, smem, acc, salt);
            }
        }
        for (int i = k * per_chunk + ((h - k * per_chunk) % n_helpers + n_helpers) % n_helpers; i < (k + 1) * per_chunk;
             i += n_helpers) {
            const int r = i - k * per_chunk;
            const int rt = c * p.k5_chunk_tiles + r / p.k5_tiles_n, ct = r % p.k5_tiles_n;
            if (rt >= p.k5_tiles_m || !p.k5.C) continue;   // (no dx wanted: the helpers only accumulate weight gradients)
            if (!stacked && c == 0 && p.k5_tail_by_rec) continue;   // the recurrence workgroups take these
            helper_dx_tile<T>(p.k5.A, p.k5.B, p.k5.C, p.k5.M, p.k5.N, p.k5.K, rt * 256, ct * 256,
                              (FASTLSTM_LDS_PTR unsigned char *)smem);
            if (stacked) {   // the tile's stores acknowledged, this XCD's L2 written back, then counted
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (threadIdx.x == 0) __hip_atomic_fetch_add(p.dx_done + c, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (stacked && k >= lag) {
            lower_dx(k - lag);       // waits for the lower layer's chunk
            lower_wgrad(k - lag);
        }
    }
    if (own && !STACKED) {
        gemm16_epilogue<T, 256, 256, 2, WVM, WVN, 2>(wp, wm0, wn0, 0, smem, acc);
        __syncthreads();
    }
    if (stacked)
        for (int k = max(p.k5_chunks - lag, 0); k < p.k5_chunks; ++k) {
            lower_dx(k);
            lower_wgrad(k);
        }
#ifdef FASTLSTM_BWD_STAMPS
    if (threadIdx.x == 0) { stamps[1] = (long long)wall_clock64(); stamps[2] = waited; }
#endif
    // weight-gradient tiles beyond one per helper: everything they need is in memory now
    for (int w = h + n_helpers; w < p.wg_tiles; w += n_helpers) {
        const bool w8 = w < n8;
        const GemmParams &q = w8 ? p.k8 : p.k9;
        const int qi = w8 ? w : w - n8, qtn = w8 ? p.k8_tiles_n : p.k9_tiles_n;
        gemm16_tile<T, true, true, 256, 256, 2, WVM, WVN, 2, false, FASTLSTM_HELPER_PP>(q, (qi / qtn) * 256, (qi % qtn) * 256, 0, smem, 0);
        __syncthreads();
    }
    if (stacked)
        for (int w = h + n_helpers; w < p.wg_lo_tiles; w += n_helpers) {
            const bool w8 = w < n8_lo;
            const GemmParams &q = w8 ? p.k8_lo : p.k9_lo;
            const int qi = w8 ? w : w - n8_lo, qtn = w8 ? p.k8_lo_tiles_n : p.k9_tiles_n;
            gemm16_tile<T, true, true, 256, 256, 2, WVM, WVN, 2, false, FASTLSTM_HELPER_PP>(q, (qi / qtn) * 256, (qi % qtn) * 256, 0, smem, 0);
            __syncthreads();
        }
}

// HELP: 0 = recurrence only; 1 = the workgroups without a role compute dx and the weight gradients;
// 2 = the same for two stacked layers that share the launch.
template <typename T, int MT, int NKW, int NTW, int NWV, int HELP = 0>
__global__ __launch_bounds__(kWave * NWV) void lstm_bwd_xcd_kernel(const BwdXcdParams p) {
    static_assert(!HELP || (NWV == 8 && sizeof(T) == 2), "the in-kernel GEMM tile is the 8-wave 16-bit one");
    using E = Elem<T>;
    constexpr bool ACC = (E::DT == FASTLSTM_FP32);
    constexpr int NTHR = kWave * NWV;
    constexpr int NT = NTW, HT = 16 * MT, BT = 16 * NT;
    constexpr int IPT = (HT * BT + NTHR - 1) / NTHR;   // (unit, batch row) items per thread
    constexpr int GSEG = HT * E::BYTES;
    constexpr int GROW = 4 * GSEG + 16, SROW = GSEG + 16;
    constexpr int PPSEG = GSEG / 16;
    constexpr int GPIECES = BT * 4 * PPSEG, SPIECES = BT * PPSEG;
    constexpr int IOT = NTHR - kWave;                  // wave 0 polls, the others move the tiles
    constexpr int GPT = (GPIECES + IOT - 1) / IOT, SPT = (SPIECES + IOT - 1) / IOT;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // (uniform: in a scalar register)
    const int q = lane >> 4, r = lane & 15;
    const int KSB = p.KSB, H = p.H, B = p.B, T_ = p.T;

    // ---- placement: group g lives on XCD g % 8 ------------------------------------------
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int gl = slot / p.n_ht, j = slot % p.n_ht;
    const int vg = gl * kNumXcd + xcd;          // group index over the layers of the launch
    // two recurrences in the launch: a stack (HELP == 2), or two independent ones of the same shape side by side
    // (HELP == 0 with n_layers == 2: the two directions of a bidirectional layer; `lower` is then simply the second)
    const int n_layers = HELP == 2 ? 2 : (HELP == 0 ? max(1, min(p.n_layers, kMaxSideBySide)) : 1);
    if (gl >= p.gpx || vg >= p.n_groups * n_layers) {
        if constexpr (HELP != 0) {
            if (p.k5_tiles_n > 0) bwd_helper<T, HELP == 2>(p, smem);
        }
        return;
    }
    check_xcd_placement(p.hdr);
    const int rec = vg / p.n_groups;                        // which recurrence of the launch
    const bool lower = rec == 1;                            // the lower layer of a stack (see BwdXcdParams::n_layers)
    const bool follows = HELP == 2 && lower;                // ... whose dout the helpers produce during the launch
    const int g = vg - rec * p.n_groups;
    // (constant indices only: a run-time index into the kernel's arguments would move them all to scratch memory;
    // the helper instantiations never see more than two recurrences)
    auto pick = [&](auto a0, auto a1, auto a2, auto a3) {
        if constexpr (HELP != 0) return lower ? a1 : a0;
        else return rec == 0 ? a0 : rec == 1 ? a1 : rec == 2 ? a2 : a3;
    };
    const int u0 = j * HT, b0 = p.b_base + g * BT;   // b_base: first batch row of this launch
    const bool k5_live = HELP && p.k5_tiles_n > 0;
    int *chunk_done = lower ? p.chunk_done_lo : p.chunk_done;
    // chunk c of the upper layer's dx (this layer's dout) is complete when all its tiles were counted
    auto wait_dout = [&](int tt) {
        const int c = tt / p.k5_chunk_steps;
        const int rows = min(p.k5_chunk_tiles, p.k5_tiles_m - c * p.k5_chunk_tiles);
        wait_versions(p.dx_done + c, 1, rows * p.k5_tiles_n, p.hdr, p.spin_limit, vg, tt);
    };
#ifdef FASTLSTM_BWD_STAMPS
    long long *stamps = reinterpret_cast<long long *>(p.counters + 8192) + blockIdx.x * 4;
    if (tid == 0) stamps[0] = (long long)wall_clock64();
#endif

    f32x4 *red = reinterpret_cast<f32x4 *>(smem);                                    // [NWV][MT][NT][64]
    unsigned char *tiles = reinterpret_cast<unsigned char *>(red + NWV * MT * NT * kWave);   // gates, c, dout tiles
    const int io_tid = tid - kWave;

    const T *dout = static_cast<const T *>(pick(p.dout, static_cast<const void *>(p.k5.C), p.dout_more[0], p.dout_more[1]));
    const T *ifgo = static_cast<const T *>(pick(p.ifgo, p.ifgo_lo, p.ifgo_more[0], p.ifgo_more[1]));
    const T *cell = static_cast<const T *>(pick(p.cell, p.cell_lo, p.cell_more[0], p.cell_more[1]));
    T *d_ifgo = static_cast<T *>(pick(p.d_ifgo, p.d_ifgo_lo, p.d_ifgo_more[0], p.d_ifgo_more[1]));
    const T *Wh = static_cast<const T *>(pick(p.Wh, p.Wh_lo, p.Wh_more[0], p.Wh_more[1]));
    T *dh_state = static_cast<T *>(pick(p.dh, p.dh_lo, p.dh_more[0], p.dh_more[1]));
    T *dc_state_buf = static_cast<T *>(pick(p.dc, p.dc_lo, p.dc_more[0], p.dc_more[1]));
    float *db_part = nullptr;
    if constexpr (HELP != 0) db_part = lower ? p.db_part_lo : p.db_part;
    f32x4 *db_slots = reinterpret_cast<f32x4 *>(smem + p.db_lds_off) + tid;   // slot of item m: db_slots[m * NTHR]
    if (db_part)
#pragma unroll
        for (int m = 0; m < IPT; ++m) db_slots[m * NTHR] = f32x4{0.f, 0.f, 0.f, 0.f};

    // ---- prologue: this wave's fragments of Wh[:, units]^T, gathered from global memory ----
    // fragment (unit tile a, k-step ks): lane (q, r) holds row r = unit u0 + 16a + r and
    // k = ks*KSTEP + q*EPL + e, e < EPL, with k = 4 * source unit + gate
    u32x4 wreg[MT][NKW];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int ki = 0; ki < NKW; ++ki) {
            const int ks = wave + NWV * ki;
            T tmp[E::EPL];
#pragma unroll
            for (int e = 0; e < E::EPL; ++e) {
                const int k = ks * E::KSTEP + q * E::EPL + e;
                const int uk = k >> 2, gate = k & 3;
                const bool ok = ks < KSB && uk < H;
                const T v = Wh[ok ? ((size_t)gate * H + uk) * H + u0 + a * 16 + r : 0];
                tmp[e] = ok ? v : E::from_f32(0.f);
            }
            wreg[a][ki] = *reinterpret_cast<u32x4 *>(tmp);
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
        valid[m] = nt < NT && b < B;
        off_h[m] = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        xoff[m] = (nt < NT ? nt : 0) * KSB * kFragBytes + frag_offset<T>(n, unit * 4);
        pair_lead[m] = valid[m] && ((ul & 1) == 0);
        const int a = ul >> 4, ur = ul & 15;
        roff[m] = ((a * NT + (nt < NT ? nt : 0)) * kWave + (ur >> 2) * 16 + n) * 4 + (ur & 3);
        goff[m] = ((nt < NT ? nt : 0) * 16 + n) * GROW + ul * E::BYTES;
        soff[m] = ((nt < NT ? nt : 0) * 16 + n) * SROW + ul * E::BYTES;
        dh_rec[m] = valid[m] ? E::to_f32(dh_state[off_h[m]]) : 0.f;
        dc_state[m] = valid[m] ? E::to_f32(dc_state_buf[off_h[m]]) : 0.f;
        c1v[m] = valid[m] ? E::to_f32(cell[(size_t)T_ * BH + off_h[m]]) : 0.f;
    }

    const unsigned xgrp = (unsigned)vg * NT * KSB * kFragBytes;
    const size_t xslot = (size_t)p.n_groups * n_layers * NT * KSB * kFragBytes;
    int *grp_counters = p.counters + (size_t)vg * kXcdGroupStride;
    int *my_counter = grp_counters + (j % kXcdReplicas) * kXcdCounterStride;

    // ---- coalesced tile I/O: ifgo[t], cell[t], dout[t] in, d_ifgo[t] out --------------------
    // Buffer loads / stores: the step's base addresses in scalar registers, per-lane byte offsets that never change.
    // Groups of 16 rows keep two sets of tile pieces in flight in registers: the tiles of step s + 2 are requested
    // right after step s's tile went out and go to the LDS behind step s + 1's K loop -- almost two steps later,
    // which also covers the memory latency while the workgroups without a role in the recurrence stream their
    // GEMM operands.  Groups of 32 rows have no registers for that (the pieces were spilled right behind their
    // loads, and a spill waits for its load): there the three tiles go global -> LDS tiles with LDS-direct loads,
    // one step ahead, slot by slot (a padded tile row is a whole number of 16-byte slots; lane l of wave
    // instruction w fills slot 64 w + l of its tile; pad slots and rows past B stay untouched), and the d_ifgo tile
    // leaves by the slots the same wave filled.
    constexpr bool DMA = NTW == 2;
    constexpr int DIST = DMA ? 1 : 2;                    // steps between the request of a tile and its use
    constexpr int SPRG = GROW / 16, SPRS = SROW / 16;    // slots per padded row
    constexpr int NG = (BT * SPRG + kWave - 1) / kWave, NS = (BT * SPRS + kWave - 1) / kWave;   // wave instructions per tile
    constexpr int DT = (NG + 2 * NS + NWV - 2) / (NWV - 1);                                     // per moving wave
    constexpr int GD = DMA ? DT : GPT, SD = DMA ? 1 : SPT;
    u32x4 gpre[DMA ? 1 : 2][DMA ? 1 : GPT], cpre[DMA ? 1 : 2][DMA ? 1 : SPT], dpre[DMA ? 1 : 2][DMA ? 1 : SPT];
    unsigned g_off[GD], s_off[SD];
    int g_lds[GD], s_lds[SD], g_kind[GD];   // DMA: tile of item d (0 gates, 1 c, 2 dout; uniform), g_lds = byte inside that tile
    bool g_ok[GD], s_ok[SD];
    const size_t tile_org = (size_t)b0 * 4 * H + u0, state_org = (size_t)b0 * H + u0;
    const unsigned g_bytes = (unsigned)((size_t)BT * 4 * H * E::BYTES), s_bytes = (unsigned)((size_t)BT * H * E::BYTES);
#pragma unroll
    for (int i = 0; i < GD; ++i) {
        if constexpr (DMA) {
            const int w = (wave - 1) + (NWV - 1) * i;
            g_kind[i] = w < NG ? 0 : (w < NG + NS ? 1 : 2);
            const int wi = w < NG ? w : (w < NG + NS ? w - NG : w - NG - NS), sl = wi * kWave + lane;
            if (g_kind[i] == 0) {
                const int row = sl / SPRG, idx = sl % SPRG;
                g_ok[i] = wave >= 1 && sl < BT * SPRG && idx < 4 * PPSEG && b0 + row < B;
                g_off[i] = g_ok[i] ? (unsigned)(((size_t)row * 4 * H + (size_t)(idx / PPSEG) * H + (idx % PPSEG) * (16 / E::BYTES)) * E::BYTES) : 0u;
            } else {
                const int row = sl / SPRS, idx = sl % SPRS;
                g_ok[i] = wave >= 1 && w < NG + 2 * NS && sl < BT * SPRS && idx < PPSEG && b0 + row < B;
                g_off[i] = g_ok[i] ? (unsigned)(((size_t)row * H + idx * (16 / E::BYTES)) * E::BYTES) : 0u;
            }
            g_lds[i] = sl * 16;
        } else {
            const int pc = io_tid + IOT * i;
            const int row = pc / (4 * PPSEG), rem = pc % (4 * PPSEG);
            const int seg = rem / PPSEG, k = rem % PPSEG;
            g_kind[i] = 0;
            g_ok[i] = io_tid >= 0 && pc < GPIECES && b0 + row < B;
            g_lds[i] = g_ok[i] ? row * GROW + seg * GSEG + k * 16 : 0;
            g_off[i] = g_ok[i] ? (unsigned)(((size_t)row * 4 * H + (size_t)seg * H + k * (16 / E::BYTES)) * E::BYTES) : 0u;
        }
    }
#pragma unroll
    for (int i = 0; i < SD; ++i) {
        const int pc = io_tid + IOT * i;
        const int row = pc / PPSEG, k = pc % PPSEG;
        s_ok[i] = !DMA && io_tid >= 0 && pc < SPIECES && b0 + row < B;
        s_lds[i] = s_ok[i] ? row * SROW + k * 16 : 0;
        s_off[i] = s_ok[i] ? (unsigned)(((size_t)row * H + k * (16 / E::BYTES)) * E::BYTES) : 0u;
    }
    auto fetch_tiles = [&](int t, u32x4(&gp)[DMA ? 1 : GPT], u32x4(&cp)[DMA ? 1 : SPT], u32x4(&dp)[DMA ? 1 : SPT]) {
        if (io_tid < 0) return;
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(ifgo) + (size_t)t * B4H + tile_org, 0, g_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(cell) + (size_t)t * BH + state_org, 0, s_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(dout) + (size_t)t * BH + state_org, 0, s_bytes, 0x00020000);
        if constexpr (DMA) {
#pragma unroll
            for (int i = 0; i < GD; ++i) {
                const int w = (wave - 1) + (NWV - 1) * i;
                if (g_kind[i] == 0) {
                    if (g_ok[i]) load_block_to_lds(rg, tiles + (size_t)w * kFragBytes, g_off[i], 0);
                } else if (g_kind[i] == 1) {
                    if (g_ok[i]) load_block_to_lds(rc, tiles + BT * GROW + (size_t)(w - NG) * kFragBytes, g_off[i], 0);
                } else {
                    if (g_ok[i]) load_block_to_lds(rd, tiles + BT * GROW + BT * SROW + (size_t)(w - NG - NS) * kFragBytes, g_off[i], 0);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < GPT; ++i) gp[i] = __builtin_amdgcn_raw_buffer_load_b128(rg, g_off[i], 0, 0);   // (pieces that do not exist read the tile's first bytes)
#pragma unroll
            for (int i = 0; i < SPT; ++i) {
                cp[i] = __builtin_amdgcn_raw_buffer_load_b128(rc, s_off[i], 0, 0);
                dp[i] = __builtin_amdgcn_raw_buffer_load_b128(rd, s_off[i], 0, 0);
            }
        }
    };
    auto tiles_to_lds = [&](const u32x4(&gp)[DMA ? 1 : GPT], const u32x4(&cp)[DMA ? 1 : SPT], const u32x4(&dp)[DMA ? 1 : SPT]) {
        if constexpr (!DMA) {
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
        }
    };
    // With helpers in the launch the d_ifgo tiles are written THROUGH to memory (sc1): the chunk
    // hand-over below then needs no write-back of this XCD's L2, which stalled the releasing wave --
    // and with it the whole group -- for several microseconds per chunk.
    auto tile_to_global = [&](int t) {
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(d_ifgo + (size_t)t * B4H + tile_org, 0, g_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < GD; ++i)
            if (g_kind[i] == 0 && g_ok[i]) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(tiles + g_lds[i]);
                if (k5_live) __builtin_amdgcn_raw_buffer_store_b128(v, rg, g_off[i], 0, 16);
                else __builtin_amdgcn_raw_buffer_store_b128(v, rg, g_off[i], 0, 0);
            }
    };
    if (follows) {   // the latest chunk(s) of this layer's dout have to be there
        if (wave == 0) {
            wait_dout(T_ - 1);
            if (DIST > 1 && T_ > 1) wait_dout(T_ - 2);
        }
        __syncthreads();
    }
    fetch_tiles(T_ - 1, gpre[0], cpre[0], dpre[0]);
    if constexpr (DMA) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // every wave's share of the tiles has landed before anyone reads them
    } else {
        if (T_ > 1) fetch_tiles(T_ - 2, gpre[1], cpre[1], dpre[1]);
        tiles_to_lds(gpre[0], cpre[0], dpre[0]);   // step 0 works on the LDS tiles right away
    }
    __syncthreads();

    // one reverse step; PAR = s % 2 picks the register sets at compile time
    auto step = [&](const int s, auto par) __attribute__((always_inline)) {
        constexpr int PAR = DMA ? 0 : decltype(par)::value, PARN = DMA ? 0 : (PAR ^ 1);
        const int t = T_ - 1 - s;
        const XchgL2 xch(p.xbuf + (size_t)(s & 1) * xslot, (unsigned)xslot);
        // the dout of timestep t - DIST is requested behind this step's publish barrier: when it is the
        // latest timestep of a chunk, that chunk of the upper layer's dx must be complete
        if (follows && wave == 0 && t >= DIST && (t - DIST) % p.k5_chunk_steps == p.k5_chunk_steps - 1) wait_dout(t - DIST);

        // ---- point-wise gate backward for this thread's items --------------------------
        u32x2 d_kept[IPT];   // the items' four stored gate gradients, for the bias sums behind the publish
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
            if constexpr (HELP != 0 && E::BYTES == 2) d_kept[m] = *reinterpret_cast<u32x2 *>(st_d);
            // exchange copy: 4 consecutive k = (unit, gate 0..3).  16-bit types: lanes l and l+16
            // own units u and u+1 of the same batch row; the even-unit lane writes both (16 bytes)
            if constexpr (E::BYTES == 2) {
                const u32x2 mine = *reinterpret_cast<u32x2 *>(st_d);
                u32x2 other;
                other[0] = (unsigned)__shfl_down((int)mine[0], 16);
                other[1] = (unsigned)__shfl_down((int)mine[1], 16);
                if (pair_lead[m])
                    __builtin_amdgcn_raw_buffer_store_b128(u32x4{mine[0], mine[1], other[0], other[1]}, xch.rsrc,
                                                           xgrp + xoff[m], 0, 0);
            } else {
                if (valid[m])
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<u32x4 *>(st_d), xch.rsrc, xgrp + xoff[m], 0, 0);
            }
        }
        // ---- publish: stores acknowledged by the L2, then the group's counters ----------------
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid < kXcdReplicas)
            __hip_atomic_fetch_add(grp_counters + tid * kXcdCounterStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        tile_to_global(t);
        if (s + DIST < T_) fetch_tiles(t - DIST, gpre[PAR], cpre[PAR], dpre[PAR]);
        if constexpr (HELP != 0 && E::BYTES == 2) {
            if (db_part) {   // (the rounded values, as they were stored: db is the column sum of d_ifgo)
#pragma unroll
                for (int m = 0; m < IPT; ++m) {
                    const T *dv = reinterpret_cast<const T *>(&d_kept[m]);
                    f32x4 a = db_slots[m * NTHR];
                    a[0] += E::to_f32(dv[0]); a[1] += E::to_f32(dv[1]); a[2] += E::to_f32(dv[2]); a[3] += E::to_f32(dv[3]);
                    db_slots[m * NTHR] = a;
                }
            }
        }

        if (wave == 0) wait_counter(my_counter, p.n_ht * (s + 1), p.hdr, p.spin_limit, vg, s);
        __syncthreads();
        // Every workgroup of the group has passed this step's publish point, where its stores of the
        // previous steps (the written-through d_ifgo tiles included) were acknowledged: they are in
        // memory.  When the previous step closed a chunk, ONE workgroup hands the group's share of it to
        // the helpers on the other XCDs and counts for all n_ht workgroups.
        if (k5_live && j == 0 && tid == kWave && s > 0 && (t + 1) % p.k5_chunk_steps == 0)
            __hip_atomic_fetch_add(chunk_done + (t + 1) / p.k5_chunk_steps, p.n_ht, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);

        // ---- dh_rec(units, rows) = Wh[:, units]^T . d_ifgo[t](rows, :)^T over this wave's k-steps
        f32x4 acc[MT][NTW];
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int i = 0; i < NTW; ++i) acc[a][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        // the operand blocks of the wave are requested in batches of at most 8 k-steps (registers):
        // all loads of a batch are issued before its first MFMA -- one round trip per batch
        constexpr int KB = NKW > 8 ? 8 : NKW;   // (all 16 at once: slower, the L2 is the bound, not the round trips)
#pragma unroll
        for (int k0 = 0; k0 < NKW; k0 += KB) {
            u32x4 bq[KB][NTW];
#pragma unroll
            for (int kk = 0; kk < KB; ++kk) {
                const int ks = min(wave + NWV * (k0 + kk), KSB - 1);   // past the end: any valid block (its weights are zero)
#pragma unroll
                for (int i = 0; i < NTW; ++i)
                    bq[kk][i] = xch.load16_l2(xgrp + (unsigned)((i * KSB + ks) * kWave + lane) * 16u);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < KB; ++kk)
#pragma unroll
                for (int a = 0; a < MT; ++a)
#pragma unroll
                    for (int i = 0; i < NTW; ++i) acc[a][i] = mfma_kstep<T>(wreg[a][k0 + kk], bq[kk][i], acc[a][i]);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int i = 0; i < NTW; ++i) red[((wave * MT + a) * NT + i) * kWave + lane] = acc[a][i];
        // the tile was drained before the barrier above: the next step's inputs take its place
        if (s + 1 < T_) tiles_to_lds(gpre[PARN], cpre[PARN], dpre[PARN]);
        __syncthreads();
        const float *redf = reinterpret_cast<const float *>(red);
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            float v = redf[roff[m]];
#pragma unroll
            for (int pp = 1; pp < NWV; ++pp) v += redf[roff[m] + pp * MT * NT * kWave * 4];
            dh_rec[m] = v;
        }
        // the next step's publish barrier orders these reads before the next writes to `red`
    };
    for (int s = 0; s < T_; s += 2) {
        step(s, std::integral_constant<int, 0>{});
        if (s + 1 < T_) step(s + 1, std::integral_constant<int, 1>{});
    }

    if (k5_live) {   // the last chunk (timesteps 0 ..)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == kWave) __hip_atomic_fetch_add(chunk_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#ifdef FASTLSTM_BWD_STAMPS
    if (tid == 0) { stamps[1] = (long long)wall_clock64(); stamps[2] = -1; }
#endif
#pragma unroll
    for (int m = 0; m < IPT; ++m)
        if (valid[m]) {
            dh_state[off_h[m]] = E::from_f32(dh_rec[m]);
            dc_state_buf[off_h[m]] = E::from_f32(dc_state[m]);
        }
    if constexpr (HELP != 0) {
        if (db_part) {   // sums over the 16 rows of a batch tile (16 neighbouring lanes), one lane writes the four gates
#pragma unroll
            for (int m = 0; m < IPT; ++m) {
                f32x4 a = db_slots[m * NTHR];
#pragma unroll
                for (int d = 1; d < 16; d <<= 1) {
                    a[0] += __shfl_xor(a[0], d); a[1] += __shfl_xor(a[1], d);
                    a[2] += __shfl_xor(a[2], d); a[3] += __shfl_xor(a[3], d);
                }
                const int it = tid + NTHR * m, rest = it >> 4, ul = rest % HT, nt = rest / HT;
                if ((it & 15) == 0 && nt < NT && b0 + nt * 16 < B) {
                    float *dst = db_part + (size_t)((b0 + nt * 16) >> 4) * 4 * H + u0 + ul;
                    dst[0] = a[0]; dst[H] = a[1]; dst[2 * (size_t)H] = a[2]; dst[3 * (size_t)H] = a[3];
                }
            }
        }
    }
    if constexpr (HELP == 1) {
        // The time loop is over and this CU would idle while the helpers finish: the dx tiles of the last chunk
        // (complete once every recurrence workgroup has counted it, just above) are dealt to the recurrence
        // workgroups, one 256 x 256 tile each as far as they go.
        if (k5_live && p.k5.C && p.k5_tail_by_rec) {
            if (wave == 0) wait_versions<100>(p.chunk_done, 1, p.n_active, p.hdr, p.spin_limit, -1, 0);
            __syncthreads();
            const int per = min(p.k5_chunk_tiles, p.k5_tiles_m) * p.k5_tiles_n;
            for (int i = g * p.n_ht + j; i < per; i += p.n_active)
                helper_dx_tile<T>(p.k5.A, p.k5.B, p.k5.C, p.k5.M, p.k5.N, p.k5.K, (i / p.k5_tiles_n) * 256, (i % p.k5_tiles_n) * 256,
                                  (FASTLSTM_LDS_PTR unsigned char *)smem);
        }
    }
#ifdef FASTLSTM_BWD_STAMPS
    if (tid == 0) stamps[3] = (long long)wall_clock64();
#endif
}

}  // namespace fastlstm

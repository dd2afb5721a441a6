// LDS-tiled MFMA GEMM for the time-parallel stages of the LSTM:
//   K1  ifgo = x . Wx^T + (bx + bh)         (fastlstm/lstm.py:66-68)
//   K5  dx   = d_ifgo . Wx                  (fastlstm/lstm.py:294)
//   K8  dWx  = d_ifgo^T . x                 (fastlstm/lstm.py:498)
//   K9  dWh  = d_ifgo^T . h[0..T-1]         (fastlstm/lstm.py:499)
// One kernel template computes  C[m][n] = sum_k A(m,k) * B(n,k)  with each operand
// stored either with K contiguous ("KC", A[m*ld + k]) or with K as the slow axis
// ("KM", A[k*ld + m]); the weight-gradient products read d_ifgo, x and h as they lie
// in memory -- the transposed copy the reference makes (lstm.py:495) does not exist.
//
// Tiling: 128 x 128 x (2 k-steps) per workgroup, 4 waves in 2 x 2, each wave 4 x 4
// MFMA 16x16 tiles (64 fp32 accumulators per lane), register-prefetched double-buffered
// LDS stages.  The MFMA is issued with the roles of the operands swapped so that a lane
// ends up holding 4 consecutive n of one output row: the epilogue stores 8/16 bytes.
#pragma once
#include "common.hpp"

namespace fastlstm {

struct GemmParams {
    const void *A, *B;
    void *C;              // [M][ldc] in T (splits == 1)
    float *Cpart;         // [splits][M][N] fp32 (splits > 1)
    const void *bias0, *bias1;  // optional [N] in T, added in fp32
    int M, N, K;
    int lda, ldb, ldc;
    int splits, k_per_split;
    int keep_c;           // 1: C leaves with ordinary stores even from a stand-alone launch (a kernel that reads it next
                          // finds it in the memory-side cache); 0: non-temporal stores there
    long long *trace;     // optional: 4 clock stamps per workgroup (diagnostics), else nullptr
};

constexpr int kBM = 128, kBN = 128;

template <typename T> struct GemmTile {
    using E = Elem<T>;
    static constexpr int BK = 2 * E::KSTEP;                  // elements of K per LDS stage
    static constexpr int KC_LD = BK + E::EPL;                // padded row length, K-contiguous tile
    static constexpr int KM_LD = kBM + E::EPL;               // padded row length, K-major tile
    static constexpr int KC_BYTES = kBM * KC_LD * E::BYTES;
    static constexpr int KM_BYTES = BK * KM_LD * E::BYTES;
    static constexpr int OP_BYTES = KC_BYTES > KM_BYTES ? KC_BYTES : KM_BYTES;
    static constexpr int LDS_BYTES = 4 * OP_BYTES;           // 2 operands x 2 stages
    static constexpr int CHUNKS = kBM * BK / E::EPL / kThreads;  // 16-byte chunks per thread per operand
};

// EPL elements base[row*ld + col ...], zero-filled outside [0,rows) x [0,cols).
template <typename T>
__device__ __forceinline__ u32x4 load_chunk(const T *base, int row, int col, int ld, int rows, int cols,
                                            bool vec_ok) {
    using E = Elem<T>;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < rows && col < cols) {
        const T *src = base + (size_t)row * ld + col;
        if (vec_ok && col + E::EPL <= cols) {
            v = *reinterpret_cast<const u32x4 *>(src);
        } else {
            T tmp[E::EPL];
#pragma unroll
            for (int e = 0; e < E::EPL; ++e) tmp[e] = (col + e < cols) ? src[e] : E::from_f32(0.f);
            v = *reinterpret_cast<u32x4 *>(tmp);
        }
    }
    return v;
}

template <typename T, bool A_KM, bool B_KM>
__global__ __launch_bounds__(kThreads) void gemm_kernel(const GemmParams p) {
    using E = Elem<T>;
    using G = GemmTile<T>;
    constexpr int BK = G::BK;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane >> 4, r = lane & 15;
    const int wm = wave >> 1, wn = wave & 1;

    const int tiles_n = cdiv(p.N, kBN), tiles_m = cdiv(p.M, kBM);
    int bid = blockIdx.x;
    const int split = bid / (tiles_m * tiles_n);
    bid -= split * tiles_m * tiles_n;
    const int m0 = (bid / tiles_n) * kBM, n0 = (bid % tiles_n) * kBN;
    const int kb = split * p.k_per_split;
    const int ke = min(p.K, kb + p.k_per_split);
    const int nkt = cdiv(ke - kb, BK);

    const T *A = static_cast<const T *>(p.A);
    const T *B = static_cast<const T *>(p.B);
    const bool a_vec = (p.lda % E::EPL) == 0, b_vec = (p.ldb % E::EPL) == 0;

    auto lds_op = [&](int operand, int stage) { return smem + (size_t)(operand * 2 + stage) * G::OP_BYTES; };

    u32x4 ra[G::CHUNKS], rb[G::CHUNKS];
    auto gload = [&](int kt) {
        const int k0 = kb + kt * BK;
#pragma unroll
        for (int i = 0; i < G::CHUNKS; ++i) {
            const int c = tid + kThreads * i;
            if constexpr (!A_KM) {
                const int row = c / (BK / E::EPL), kc = c % (BK / E::EPL);
                ra[i] = load_chunk<T>(A, m0 + row, k0 + kc * E::EPL, p.lda, p.M, ke, a_vec);
            } else {
                const int k = c / (kBM / E::EPL), mc = c % (kBM / E::EPL);
                ra[i] = load_chunk<T>(A, k0 + k, m0 + mc * E::EPL, p.lda, ke, p.M, a_vec);
            }
            if constexpr (!B_KM) {
                const int row = c / (BK / E::EPL), kc = c % (BK / E::EPL);
                rb[i] = load_chunk<T>(B, n0 + row, k0 + kc * E::EPL, p.ldb, p.N, ke, b_vec);
            } else {
                const int k = c / (kBN / E::EPL), nc = c % (kBN / E::EPL);
                rb[i] = load_chunk<T>(B, k0 + k, n0 + nc * E::EPL, p.ldb, ke, p.N, b_vec);
            }
        }
    };
    auto lstore = [&](int stage) {
        unsigned char *la = lds_op(0, stage), *lb = lds_op(1, stage);
#pragma unroll
        for (int i = 0; i < G::CHUNKS; ++i) {
            const int c = tid + kThreads * i;
            if constexpr (!A_KM) {
                const int row = c / (BK / E::EPL), kc = c % (BK / E::EPL);
                *reinterpret_cast<u32x4 *>(la + ((size_t)row * G::KC_LD + kc * E::EPL) * E::BYTES) = ra[i];
            } else {
                const int k = c / (kBM / E::EPL), mc = c % (kBM / E::EPL);
                *reinterpret_cast<u32x4 *>(la + ((size_t)k * G::KM_LD + mc * E::EPL) * E::BYTES) = ra[i];
            }
            if constexpr (!B_KM) {
                const int row = c / (BK / E::EPL), kc = c % (BK / E::EPL);
                *reinterpret_cast<u32x4 *>(lb + ((size_t)row * G::KC_LD + kc * E::EPL) * E::BYTES) = rb[i];
            } else {
                const int k = c / (kBN / E::EPL), nc = c % (kBN / E::EPL);
                *reinterpret_cast<u32x4 *>(lb + ((size_t)k * G::KM_LD + nc * E::EPL) * E::BYTES) = rb[i];
            }
        }
    };
    // 16-byte MFMA fragment of matrix row `row` (0..127), k-step `ks` of the stage
    auto frag = [&](const unsigned char *tile, bool km, int row, int ks) -> u32x4 {
        if (!km) {
            return *reinterpret_cast<const u32x4 *>(
                tile + ((size_t)row * G::KC_LD + ks * E::KSTEP + q * E::EPL) * E::BYTES);
        } else {
            T tmp[E::EPL];
            const T *t = reinterpret_cast<const T *>(tile);
#pragma unroll
            for (int e = 0; e < E::EPL; ++e) tmp[e] = t[(size_t)(ks * E::KSTEP + q * E::EPL + e) * G::KM_LD + row];
            return *reinterpret_cast<u32x4 *>(tmp);
        }
    };

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) acc[i][jn] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (nkt > 0) {
        gload(0);
        lstore(0);
    }
    __syncthreads();
    for (int kt = 0; kt < nkt; ++kt) {
        const int st = kt & 1;
        if (kt + 1 < nkt) gload(kt + 1);
        const unsigned char *la = lds_op(0, st), *lb = lds_op(1, st);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            u32x4 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = frag(la, A_KM, wm * 64 + i * 16 + r, ks);
#pragma unroll
            for (int i = 0; i < 4; ++i) fb[i] = frag(lb, B_KM, wn * 64 + i * 16 + r, ks);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int jn = 0; jn < 4; ++jn) acc[i][jn] = mfma_kstep<T>(fb[jn], fa[i], acc[i][jn]);
        }
        if (kt + 1 < nkt) lstore(st ^ 1);
        __syncthreads();
    }

    // epilogue: lane holds C[m][nb .. nb+3], m = tile row r, nb = 4q
    const T *bias0 = static_cast<const T *>(p.bias0), *bias1 = static_cast<const T *>(p.bias1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + wm * 64 + i * 16 + r;
        if (m >= p.M) continue;
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) {
            const int nb = n0 + wn * 64 + jn * 16 + q * 4;
            if (nb >= p.N) continue;
            f32x4 v = acc[i][jn];
            if (p.splits > 1) {
                float *dst = p.Cpart + ((size_t)split * p.M + m) * p.N + nb;
                if ((p.N & 3) == 0) {
                    *reinterpret_cast<f32x4 *>(dst) = v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (nb + e < p.N) dst[e] = v[e];
                }
                continue;
            }
            if (bias0) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (nb + e < p.N) v[e] += E::to_f32(bias0[nb + e]) + (bias1 ? E::to_f32(bias1[nb + e]) : 0.f);
            }
            T *dst = static_cast<T *>(p.C) + (size_t)m * p.ldc + nb;
            if ((p.ldc & 3) == 0 && nb + 3 < p.N) {
                T pk[4] = {E::from_f32(v[0]), E::from_f32(v[1]), E::from_f32(v[2]), E::from_f32(v[3])};
                if constexpr (E::BYTES == 2) *reinterpret_cast<u32x2 *>(dst) = *reinterpret_cast<u32x2 *>(pk);
                else *reinterpret_cast<u32x4 *>(dst) = *reinterpret_cast<u32x4 *>(pk);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (nb + e < p.N) dst[e] = E::from_f32(v[e]);
            }
        }
    }
}

// C[m][n] = sum_s part[s][m][n]  (deterministic split-K finish), cast to T.
template <typename T>
__global__ void splitk_reduce_kernel(const float *part, T *C, int M, int N, int ldc, int splits, int slices) {
    // 256 threads = 256 / slices outputs x slices (1 or 4) of the splits (k = slice, slice + slices, ...),
    // eight loads in flight per thread; four slices (many splits, few outputs) are combined through LDS in a
    // fixed order
    __shared__ float red[4][64];
    const size_t total = (size_t)M * N;
    const int per_block = 256 / slices;
    const int ol = threadIdx.x % per_block, slice = threadIdx.x / per_block;
    const size_t i = (size_t)blockIdx.x * per_block + ol;
    float s = 0.f;
    if (i < total) {
        int k = slice;
        for (; k + 7 * slices < splits; k += 8 * slices) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(size_t)(k + slices * u) * total + i];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; k < splits; k += slices) s += part[(size_t)k * total + i];
    }
    if (slices == 4) {
        red[slice][ol] = s;
        __syncthreads();
        s = (red[0][ol] + red[1][ol]) + (red[2][ol] + red[3][ol]);
        if (slice != 0) return;
    }
    if (i < total) C[(i / N) * ldc + (i % N)] = Elem<T>::from_f32(s);
}

// Column sums of in[R][C] (db = sum over time and batch of d_ifgo, lstm.py:497), two
// deterministic stages: part[chunk][C] in fp32, then the sum over chunks.
template <typename T, int VEC>
__global__ void colsum_partial_kernel(const T *in, float *part, int R, int C, int rows_per_chunk, int col_threads) {
    // 128 threads = col_threads column groups (VEC columns each) x 128 / col_threads row lanes: a narrow
    // matrix still fills the block; row lane y takes rows r0 + y, r0 + y + lanes, ... of the chunk and the
    // lanes are summed through LDS in a fixed order
    __shared__ float red[128][VEC];
    const int tx = threadIdx.x % col_threads, ty = threadIdx.x / col_threads, lanes = 128 / col_threads;
    const int c0 = (blockIdx.x * col_threads + tx) * VEC;
    const bool live = c0 < C;
    const int r0 = blockIdx.y * rows_per_chunk, r1 = min(R, r0 + rows_per_chunk);
    float s[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) s[e] = 0.f;
    constexpr int U = 8;   // rows in flight per thread: the kernel is a pure HBM stream
    int rr = r0 + ty;
    if constexpr (VEC > 1) {
        for (; live && rr + (U - 1) * lanes < r1; rr += U * lanes) {
            u32x4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = *reinterpret_cast<const u32x4 *>(in + (size_t)(rr + u * lanes) * C + c0);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const T *tv = reinterpret_cast<const T *>(&v[u]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) s[e] += Elem<T>::to_f32(tv[e]);
            }
        }
    }
    for (; live && rr < r1; rr += lanes) {
        const T *src = in + (size_t)rr * C + c0;
        if constexpr (VEC == 1) {
            s[0] += Elem<T>::to_f32(src[0]);
        } else {
            u32x4 v = *reinterpret_cast<const u32x4 *>(src);
            const T *tv = reinterpret_cast<const T *>(&v);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s[e] += Elem<T>::to_f32(tv[e]);
        }
    }
    if (lanes > 1) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[threadIdx.x][e] = s[e];
        __syncthreads();
        if (ty == 0)
            for (int y = 1; y < lanes; ++y)
#pragma unroll
                for (int e = 0; e < VEC; ++e) s[e] += red[y * col_threads + tx][e];
    }
    if (live && ty == 0)
#pragma unroll
        for (int e = 0; e < VEC; ++e) part[(size_t)blockIdx.y * C + c0 + e] = s[e];
}

// out[c] = sum over chunks of part[chunk][c].  A block of 256 threads covers 64 columns with 4
// threads each (chunks k = slice, slice + 4, ...), summed through LDS in a fixed order.
// 256 threads = 16 columns x 16 slices of the chunks; a thread sums chunks slice, slice + 16, ... with 8 loads in
// flight (a chain of dependent loads over all chunks is pure latency), the slices meet in LDS in a fixed order.
constexpr int kColsumFinalCols = 16;
template <typename T> __global__ void colsum_final_kernel(const float *part, T *out, int C, int chunks) {
    __shared__ float red[16][kColsumFinalCols];
    const int cl = threadIdx.x & 15, slice = threadIdx.x >> 4;
    const int c = blockIdx.x * kColsumFinalCols + cl;
    float s = 0.f;
    if (c < C) {
        int k = slice;
        for (; k + 7 * 16 < chunks; k += 8 * 16) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(size_t)(k + 16 * u) * C + c];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; k < chunks; k += 16) s += part[(size_t)k * C + c];
    }
    red[slice][cl] = s;
    __syncthreads();
    if (slice == 0 && c < C) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) t += red[i][cl];
        out[c] = Elem<T>::from_f32(t);
    }
}

}  // namespace fastlstm

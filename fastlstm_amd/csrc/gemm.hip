// Host launchers for the MFMA GEMM stages (K1, K5, K8, K9) and the db column sum.
#include "gemm.hpp"
#include "gemm16.hpp"
#include <atomic>
#include "internal.hpp"

namespace fastlstm {

namespace {

template <typename T, bool A_KM, bool B_KM>
hipError_t launch_gemm_t(const GemmParams &p, hipStream_t stream) {
    using G = GemmTile<T>;
    static bool attr_set = false;
    auto kern = gemm_kernel<T, A_KM, B_KM>;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int grid = cdiv(p.M, kBM) * cdiv(p.N, kBN) * p.splits;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), G::LDS_BYTES, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (p.splits > 1) {
        const size_t total = (size_t)p.M * p.N;
        const int slices = p.splits >= 16 ? 4 : 1;     // many splits: four threads per output
        const int blocks = (int)((total * slices + 255) / 256);
        hipLaunchKernelGGL(splitk_reduce_kernel<T>, dim3(blocks), dim3(256), 0, stream, p.Cpart,
                           static_cast<T *>(p.C), p.M, p.N, p.ldc, p.splits, slices);
        e = hipGetLastError();
    }
    return e;
}

std::atomic<int> g_gemm_baseline{0};   // diagnostics: 1 = stand-alone 16-bit 256 x 256 launches run gemm16_onetile_kernel

// one 256 x 256 tile per workgroup (gemm16_onetile_kernel); with splits > 1 the caller reduces the partials
template <typename T, bool A_KM, bool B_KM> static hipError_t launch_onetile_t(const GemmParams &p, hipStream_t stream) {
    using C = Gemm16Cfg<256, 256, 2, 2, 4, 2>;
    static bool attr_set = false;
    auto kern = gemm16_onetile_kernel<T, A_KM, B_KM>;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           C::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(cdiv(p.M, 256) * cdiv(p.N, 256) * p.splits), dim3(C::THREADS), C::LDS_BYTES, stream, p);
    return hipGetLastError();
}

template <typename T, bool A_KM, bool B_KM, int BM, int BN, int NS, int WVM, int WVN, int KSPT>
hipError_t launch_gemm16_t(const GemmParams &p, hipStream_t stream) {
    using C = Gemm16Cfg<BM, BN, NS, WVM, WVN, KSPT>;
    static bool attr_set = false;
    const bool baseline = BM == 256 && BN == 256 && sizeof(T) == 2 && g_gemm_baseline.load() != 0;
    auto kern = gemm16_kernel<T, A_KM, B_KM, BM, BN, NS, WVM, WVN, KSPT>;
    if constexpr (BM == 256 && BN == 256 && sizeof(T) == 2) {
        if (baseline)
            if (hipError_t e = launch_onetile_t<T, A_KM, B_KM>(p, stream)) return e;
    }
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    // the 256 x 256 configuration (one workgroup per CU) walks through a longer tile list with one workgroup per CU
    const int tiles = cdiv(p.M, BM) * cdiv(p.N, BN) * p.splits;
    const int grid = (BM == 256 && BN == 256) ? std::min(tiles, kNumXcd * 32) : tiles;
    if (!baseline) hipLaunchKernelGGL(kern, dim3(grid), dim3(C::THREADS), C::LDS_BYTES, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (p.splits > 1) {
        const size_t total = (size_t)p.M * p.N;
        const int slices = p.splits >= 16 ? 4 : 1;     // many splits: four threads per output
        const int blocks = (int)((total * slices + 255) / 256);
        hipLaunchKernelGGL(splitk_reduce_kernel<T>, dim3(blocks), dim3(256), 0, stream, p.Cpart,
                           static_cast<T *>(p.C), p.M, p.N, p.ldc, p.splits, slices);
        e = hipGetLastError();
    }
    return e;
}

template <typename T, int BM, int BN, int NS, int WVM, int WVN, int KSPT>
hipError_t launch_gemm16_dt(const GemmParams &p, bool a_km, bool b_km, hipStream_t s) {
    if (!a_km && !b_km) return launch_gemm16_t<T, false, false, BM, BN, NS, WVM, WVN, KSPT>(p, s);
    if (!a_km && b_km) return launch_gemm16_t<T, false, true, BM, BN, NS, WVM, WVN, KSPT>(p, s);
    if (a_km && b_km) return launch_gemm16_t<T, true, true, BM, BN, NS, WVM, WVN, KSPT>(p, s);
    return hipErrorInvalidValue;
}

template <typename T> hipError_t launch_gemm_dt(const GemmParams &p, bool a_km, bool b_km, hipStream_t s) {
    if (!a_km && !b_km) return launch_gemm_t<T, false, false>(p, s);
    if (!a_km && b_km) return launch_gemm_t<T, false, true>(p, s);
    if (a_km && b_km) return launch_gemm_t<T, true, true>(p, s);
    return hipErrorInvalidValue;
}

template <typename T>
hipError_t launch_colsum_t(const void *in, void *out, float *part, int R, int C, int chunks, hipStream_t s) {
    using E = Elem<T>;
    const int rpc = cdiv(R, chunks);
    // column groups per block: the power of two that covers the columns, at most the whole block
    auto col_threads = [](int groups) {
        int ct = 1;
        while (ct < 128 && ct < groups) ct *= 2;
        return ct;
    };
    if (C % E::EPL == 0) {
        const int ct = col_threads(C / E::EPL);
        dim3 grid(cdiv(C, ct * E::EPL), chunks);
        hipLaunchKernelGGL((colsum_partial_kernel<T, E::EPL>), grid, dim3(128), 0, s,
                           static_cast<const T *>(in), part, R, C, rpc, ct);
    } else {
        const int ct = col_threads(C);
        dim3 grid(cdiv(C, ct), chunks);
        hipLaunchKernelGGL((colsum_partial_kernel<T, 1>), grid, dim3(128), 0, s, static_cast<const T *>(in),
                           part, R, C, rpc, ct);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(colsum_final_kernel<T>, dim3(cdiv(C, kColsumFinalCols)), dim3(256), 0, s, part, static_cast<T *>(out),
                       C, chunks);
    return hipGetLastError();
}

}  // namespace

// The 16-bit fast kernel needs: K range of every split a multiple of 64, 16-byte aligned
// rows, operands addressable with 32-bit byte offsets.
bool gemm16_eligible(int dtype, int M, int N, int K, int lda, int ldb, bool a_km, bool b_km) {
    // (fp32 runs on the 256 x 256 tile only: see gemm_plan)
    const int es = dtype == FASTLSTM_FP32 ? 4 : 2, epc = 16 / es;
    // K-major x K-major (the weight gradients, K = T*B rows): any K -- the loop runs to the next multiple of 64 and the
    // rows past K lie outside both operands' buffer ranges, where loads return zero
    if ((K % 64 != 0 && !(a_km && b_km)) || lda % epc != 0 || ldb % epc != 0) return false;
    // 32-bit byte offsets, with room for the rows a partial tile reaches past the operand
    const size_t a_bytes = (size_t)((a_km ? K : M) + 256) * lda * es, b_bytes = (size_t)((b_km ? K : N) + 256) * ldb * es;
    return a_bytes < (1ull << 32) && b_bytes < (1ull << 32);
}

// Tile edge (256 or 128; 0 = generic kernel) and split-K factor for a product.
void gemm_plan(int dtype, int M, int N, int K, int lda, int ldb, bool a_km, bool b_km, bool allow_split,
               int *tile, int *splits) {
    *splits = 1;
    if (!gemm16_eligible(dtype, M, N, K, lda, ldb, a_km, b_km)) {
        *tile = 0;
        const int tiles = cdiv(M, kBM) * cdiv(N, kBN);
        if (allow_split && tiles < 128) {
            const int bk = gemm_bk(dtype);
            *splits = std::max(1, std::min(std::min(cdiv(512, tiles), std::max(1, K / (4 * bk))), 1024));
        }
        return;
    }
    const int t256 = cdiv(M, 256) * cdiv(N, 256), t128 = cdiv(M, 128) * cdiv(N, 128);
    const int max_split = allow_split ? std::max(1, K / 512) : 1;  // >= 8 k-tiles per split
    if (t256 >= 192) {
        *tile = 256;
    } else if (std::min(256 / t256, max_split) * t256 >= 192) {   // (one round of workgroups: the factor rounded down)
        *tile = 256;
        *splits = std::min(256 / t256, max_split);
    } else if (dtype == FASTLSTM_FP32) {
        // true-fp32 MFMA runs at 1/16 of the 16-bit rate: a product too small to fill the device with 256 x 256 tiles is
        // left to the generic 128 x 128 kernel (two workgroups per CU), planned as above
        *tile = 0;
        const int tiles = cdiv(M, kBM) * cdiv(N, kBN);
        if (allow_split && tiles < 128) {
            const int bk = gemm_bk(dtype);
            *splits = std::max(1, std::min(std::min(cdiv(512, tiles), std::max(1, K / (4 * bk))), 1024));
        }
    } else {
        *tile = 128;
        if (t128 < 192) *splits = std::max(1, std::min(cdiv(512, t128), max_split));
    }
}

// ---- both weight gradients + the bias gradient on the tile kernel (gemm16_wgrad_kernel) ------------------------
// Taken for 16-bit products that the 256 x 256 tile kernel holds.  *merged: both products as one tile grid with
// one split factor (K = T*B is split so that the tiles of both together fill the device); otherwise each product
// fills the device on its own and they run as two launches of one round of tiles each, the bias gradient with
// the first (a second round of tiles starts out of step with its neighbours and shares less in the L2:
// M = 8192, I = H = 2048, K = 32768: 1.85 ms merged against 2 x 0.86).
bool wgrad_merged_plan(int dtype, int M, int I, int H, int K, int *splits, int *k_per_split, bool *merged) {
    if (!gemm16_eligible(dtype, M, I, K, M, I, true, true) || !gemm16_eligible(dtype, M, H, K, M, H, true, true)) return false;
    if (M < 256 || I < 128 || H < 128) return false;   // thin outputs: the 128 x 128 tiles waste less
    const int tx = cdiv(M, 256) * cdiv(I, 256), th = cdiv(M, 256) * cdiv(H, 256);
    *merged = !(tx >= 192 && th >= 192 && tx <= 256 && th <= 256);
    int sp = 1;
    // (rounded down: one round of at most 256 workgroups; 60 tiles x 5 splits would be a full round and a sixth of one)
    if (*merged && tx + th < 192) sp = std::max(1, std::min(256 / (tx + th), K / 512));   // >= 8 k-tiles per split
    // true-fp32 MFMA runs at 1/16 of the 16-bit rate: products that do not fill the device with 256 x 256 tiles stay
    // with the generic 128 x 128 kernel and its finer split (T*B = 2048, 4H = 1024, I = H = 256: 0.06 against 0.15 ms)
    if (dtype == FASTLSTM_FP32 && (tx + th) * sp < 192) return false;
    const int kps = cdiv(cdiv(K, sp), 64) * 64;
    *k_per_split = kps;
    *splits = cdiv(K, kps);
    return true;
}

// workspace: [splits][column tiles][M] for the bias gradient + [splits][M][I] + [splits][M][H] floats with a split
size_t wgrad_merged_workspace(int dtype, int M, int I, int H, int K) {
    int sp, kps;
    bool merged;
    if (!wgrad_merged_plan(dtype, M, I, H, K, &sp, &kps, &merged)) return 0;
    const size_t dbp = align_up((size_t)sp * (cdiv(I, 256) + cdiv(H, 256)) * M * sizeof(float), 256);
    return dbp + (sp > 1 ? (size_t)sp * M * ((size_t)I + H) * sizeof(float) : 0);
}

template <typename T>
static hipError_t launch_wgrad_kernel_t(const WgradParams &w, hipStream_t s) {
    using C = Gemm16Cfg<256, 256, 2, 2, 4, 2>;
    static bool attr_set = false;
    auto kern = gemm16_wgrad_kernel<T>;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           C::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int grid = cdiv(w.x.M, 256) * (w.tiles_nx + cdiv(w.h.N, 256)) * w.x.splits;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(C::THREADS), C::LDS_BYTES, s, w);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_wgrad_merged_t(const WgradParams &w, bool merged, void *db, hipStream_t s) {
    const int M = w.x.M, I = w.x.N, H = w.h.N, splits = w.x.splits;
    int db_parts;
    if (merged) {
        if (hipError_t e = launch_wgrad_kernel_t<T>(w, s)) return e;
        db_parts = splits * (w.tiles_nx + cdiv(H, 256));
    } else {   // the x product with the bias gradient, then the h product alone
        WgradParams a = w, b = w;
        a.h.N = 0;
        b.x = w.h; b.h.N = 0; b.tiles_nx = cdiv(H, 256); b.db_part = nullptr;
        if (hipError_t e = launch_wgrad_kernel_t<T>(a, s)) return e;
        if constexpr (sizeof(T) == 2) {   // one round of tiles, both operands K-major: the symmetric loop (gemm16_onetile_kernel)
            if (hipError_t e = launch_onetile_t<T, true, true>(w.h, s)) return e;
        } else {
            if (hipError_t e = launch_wgrad_kernel_t<T>(b, s)) return e;
        }
        db_parts = splits * w.tiles_nx;
    }
    const int ri = splits > 1 ? I : 0, rh = splits > 1 ? H : 0;   // the products need no pass without a split
    const size_t threads = (size_t)M * ri / 4 + (size_t)M * rh / 4 + M;
    hipLaunchKernelGGL(wgrad_reduce_kernel<T>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, w.x.Cpart,
                       static_cast<T *>(w.x.C), w.h.Cpart, static_cast<T *>(w.h.C), w.db_part, static_cast<T *>(db), M, ri, rh,
                       splits, db_parts);
    return hipGetLastError();
}

hipError_t launch_wgrad_merged(int dtype, const void *d_ifgo, const void *x, const void *h, void *dWx, void *dWh, void *db,
                               void *ws, int M, int I, int H, int K, hipStream_t s) {
    WgradParams w{};
    int sp, kps;
    bool merged;
    if (!wgrad_merged_plan(dtype, M, I, H, K, &sp, &kps, &merged)) return hipErrorInvalidValue;
    float *db_part = static_cast<float *>(ws);
    float *part_x = reinterpret_cast<float *>(static_cast<unsigned char *>(ws) +
                                              align_up((size_t)sp * (cdiv(I, 256) + cdiv(H, 256)) * M * sizeof(float), 256));
    GemmParams g{};
    g.A = d_ifgo; g.M = M; g.K = K; g.lda = M; g.splits = sp; g.k_per_split = kps;
    w.x = g; w.x.B = x; w.x.C = dWx; w.x.N = I; w.x.ldb = I; w.x.ldc = I; w.x.Cpart = part_x;
    w.h = g; w.h.B = h; w.h.C = dWh; w.h.N = H; w.h.ldb = H; w.h.ldc = H; w.h.Cpart = part_x + (size_t)sp * M * I;
    w.tiles_nx = cdiv(I, 256);
    w.db_part = db_part;
    return dtype == FASTLSTM_FP32 ? launch_wgrad_merged_t<float>(w, merged, db, s)
           : dtype == FASTLSTM_FP16 ? launch_wgrad_merged_t<_Float16>(w, merged, db, s)
                                    : launch_wgrad_merged_t<__bf16>(w, merged, db, s);
}

void set_gemm_baseline(int on) { g_gemm_baseline.store(on ? 1 : 0); }
int gemm_baseline() { return g_gemm_baseline.load(); }

static long long *g_trace = nullptr;
void set_gemm_trace(long long *buf) { g_trace = buf; }

hipError_t launch_gemm_tiled(int dtype, const GemmParams &p_in, bool a_km, bool b_km, int tile, hipStream_t s) {
    GemmParams p = p_in;
    p.trace = g_trace;
#define FASTLSTM_TILE_CASE(ID, BM, BN, NS, WVM, WVN, KSPT)                                                  \
    if (tile == ID)                                                                                         \
        return dtype == FASTLSTM_FP16 ? launch_gemm16_dt<_Float16, BM, BN, NS, WVM, WVN, KSPT>(p, a_km, b_km, s) \
                                      : launch_gemm16_dt<__bf16, BM, BN, NS, WVM, WVN, KSPT>(p, a_km, b_km, s);
    if (tile == 256 && dtype == FASTLSTM_FP32) return launch_gemm16_dt<float, 256, 256, 2, 2, 4, 2>(p, a_km, b_km, s);
    if (dtype == FASTLSTM_FP32) return launch_gemm(dtype, p, a_km, b_km, s);
    FASTLSTM_TILE_CASE(128, 128, 128, 2, 2, 2, 2)   // 2 workgroups per CU
    FASTLSTM_TILE_CASE(256, 256, 256, 2, 2, 4, 2)   // 8 waves, 128 x 64 per wave, 2 x 64 KiB stages
#undef FASTLSTM_TILE_CASE
    return launch_gemm(dtype, p, a_km, b_km, s);
}

hipError_t launch_gemm(int dtype, const GemmParams &p, bool a_km, bool b_km, hipStream_t s) {
    switch (dtype) {
        case FASTLSTM_FP32: return launch_gemm_dt<float>(p, a_km, b_km, s);
        case FASTLSTM_FP16: return launch_gemm_dt<_Float16>(p, a_km, b_km, s);
        default: return launch_gemm_dt<__bf16>(p, a_km, b_km, s);
    }
}

hipError_t launch_colsum(int dtype, const void *in, void *out, float *part, int R, int C, int chunks,
                         hipStream_t s) {
    switch (dtype) {
        case FASTLSTM_FP32: return launch_colsum_t<float>(in, out, part, R, C, chunks, s);
        case FASTLSTM_FP16: return launch_colsum_t<_Float16>(in, out, part, R, C, chunks, s);
        default: return launch_colsum_t<__bf16>(in, out, part, R, C, chunks, s);
    }
}

// the second stage alone: out[C] = the sum over `chunks` rows of part[chunks][C]
hipError_t launch_colsum_final(int dtype, const float *part, void *out, int C, int chunks, hipStream_t s) {
    const dim3 grid(cdiv(C, kColsumFinalCols)), block(256);
    if (dtype == FASTLSTM_FP32) hipLaunchKernelGGL(colsum_final_kernel<float>, grid, block, 0, s, part, static_cast<float *>(out), C, chunks);
    else if (dtype == FASTLSTM_FP16) hipLaunchKernelGGL(colsum_final_kernel<_Float16>, grid, block, 0, s, part, static_cast<_Float16 *>(out), C, chunks);
    else hipLaunchKernelGGL(colsum_final_kernel<__bf16>, grid, block, 0, s, part, static_cast<__bf16 *>(out), C, chunks);
    return hipGetLastError();
}

int gemm_bk(int dtype) { return dtype == FASTLSTM_FP32 ? GemmTile<float>::BK : GemmTile<_Float16>::BK; }

}  // namespace fastlstm

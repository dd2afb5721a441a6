// Host launcher of the one-pass reverse products of a narrow layer (gemm_small.hpp).
#include "gemm_small.hpp"
#include "internal.hpp"

namespace fastlstm {

// Shapes the pass is built for, and from where on it pays: 16-bit elements, 4H <= 256 and I <= 64 in whole MFMA
// tiles, operands that a 32-bit byte offset addresses.
bool small_bwd_eligible(int dtype, int R, int I, int H) {
    return dtype != FASTLSTM_FP32 && H % 16 == 0 && H <= 64 && I % 16 == 0 && I <= 64 && R >= 256 &&
           (size_t)R * 4 * H * 2 < ((size_t)1 << 31);
}

static int small_bwd_workers(int R) { return std::min(cdiv(R, kSmallRows), kNumXcd * 32); }

size_t small_bwd_workspace(int R, int I, int H) {
    return (size_t)small_bwd_workers(R) * 4 * H * (I + H + 1) * sizeof(float);
}

template <typename T>
static hipError_t launch_small_bwd_t(const SmallBwdParams &p, void *dWx, void *dWh, void *db, hipStream_t s) {
    static bool attr_set = false;
    auto kern = small_bwd_kernel<T>;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kSmallLdsBytes);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int workers = small_bwd_workers(p.R);
    hipLaunchKernelGGL(kern, dim3(workers), dim3(512), kSmallLdsBytes, s, p);
    if (hipError_t e = hipGetLastError()) return e;
    if (!p.part) return hipSuccess;
    const int quads = p.G * (p.I + p.H + 1) / 4;
    hipLaunchKernelGGL(small_bwd_reduce_kernel<T>, dim3(cdiv(quads, 32)), dim3(256), 0, s, p.part, static_cast<T *>(dWx),
                       static_cast<T *>(dWh), static_cast<T *>(db), p.G, p.I, p.H, workers);
    return hipGetLastError();
}

// dx (or nullptr) and dWx, dWh, db (all three, or all nullptr) from d_ifgo[R][4H], Wx[4H][I], x[R][I], h[R][H];
// ws: small_bwd_workspace bytes (weight gradients only)
hipError_t launch_small_bwd(int dtype, const void *d_ifgo, const void *Wx, const void *x, const void *h, void *dx, void *dWx,
                            void *dWh, void *db, void *ws, int R, int I, int H, hipStream_t s) {
    SmallBwdParams p{};
    p.d_ifgo = d_ifgo; p.Wx = Wx; p.x = x; p.h = h;
    p.dx = dx;
    p.part = dWx ? static_cast<float *>(ws) : nullptr;
    p.R = R; p.G = 4 * H; p.I = I; p.H = H;
    return dtype == FASTLSTM_FP16 ? launch_small_bwd_t<_Float16>(p, dWx, dWh, db, s) : launch_small_bwd_t<__bf16>(p, dWx, dWh, db, s);
}

// K1 of a narrow layer (small_k1_kernel): rows [0, R) of x[R][I] -> ifgo[R][4H]; the shapes of small_bwd_eligible
hipError_t launch_small_k1(int dtype, const void *x, const void *Wx, const void *bx, const void *bh, void *ifgo, int R, int I,
                           int H, hipStream_t s) {
    SmallK1Params p{};
    p.x = x; p.Wx = Wx; p.bx = bx; p.bh = bh; p.ifgo = ifgo;
    p.R = R; p.G = 4 * H; p.I = I;
    const int grid = std::min(cdiv(R, kSmallRows), 2 * kNumXcd * 32);   // two workgroups per CU (68 KiB of LDS each)
    auto launch = [&](auto kern) {
        static bool attr_set = false;
        if (!attr_set) {
            if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                   kSmallK1LdsBytes))
                return e;
            attr_set = true;
        }
        hipLaunchKernelGGL(kern, dim3(grid), dim3(512), kSmallK1LdsBytes, s, p);
        return hipGetLastError();
    };
    return dtype == FASTLSTM_FP16 ? launch(small_k1_kernel<_Float16>) : launch(small_k1_kernel<__bf16>);
}

}  // namespace fastlstm

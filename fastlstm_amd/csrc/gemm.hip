// Host launchers for the MFMA GEMM stages (K1, K5, K8, K9) and the db column sum.
#include "gemm.hpp"
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
        const int blocks = (int)std::min<size_t>((total + 255) / 256, 4096);
        hipLaunchKernelGGL(splitk_reduce_kernel<T>, dim3(blocks), dim3(256), 0, stream, p.Cpart,
                           static_cast<T *>(p.C), p.M, p.N, p.ldc, p.splits);
        e = hipGetLastError();
    }
    return e;
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
    if (C % E::EPL == 0) {
        dim3 grid(cdiv(C, 128 * E::EPL), chunks);
        hipLaunchKernelGGL((colsum_partial_kernel<T, E::EPL>), grid, dim3(128), 0, s,
                           static_cast<const T *>(in), part, R, C, rpc);
    } else {
        dim3 grid(cdiv(C, 128), chunks);
        hipLaunchKernelGGL((colsum_partial_kernel<T, 1>), grid, dim3(128), 0, s, static_cast<const T *>(in),
                           part, R, C, rpc);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(colsum_final_kernel<T>, dim3(cdiv(C, 256)), dim3(256), 0, s, part, static_cast<T *>(out),
                       C, chunks);
    return hipGetLastError();
}

}  // namespace

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

int gemm_bk(int dtype) { return dtype == FASTLSTM_FP32 ? GemmTile<float>::BK : GemmTile<_Float16>::BK; }

}  // namespace fastlstm

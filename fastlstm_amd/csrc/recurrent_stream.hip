// Instantiates the streamed-weights kernels (recurrent_stream.hpp) for the three element types.
#include "recurrent_stream.hpp"
#include "recurrent_launch.hpp"

namespace fastlstm {

template <typename T>
static hipError_t fwd_stream_t(const FwdStreamParams &p, int mt, int nt, int grid, int lds, hipStream_t s, int *occ) {
#define CASE(MT, NT) \
    if (mt == MT && nt == NT) return launch_one(lstm_fwd_stream_kernel<T, MT, NT>, p, grid, lds, s, occ)
    CASE(4, 1); CASE(4, 2); CASE(4, 4); CASE(8, 1); CASE(8, 2); CASE(16, 1);
#undef CASE
    return hipErrorInvalidConfiguration;
}
template <typename T>
static hipError_t bwd_stream_t(const BwdStreamParams &p, int mtb, int nt, int grid, int lds, hipStream_t s, int *occ) {
#define CASE(MTB, NT) \
    if (mtb == MTB && nt == NT) return launch_one(lstm_bwd_stream_kernel<T, MTB, NT>, p, grid, lds, s, occ)
    CASE(1, 1); CASE(1, 2); CASE(1, 4); CASE(2, 1); CASE(2, 2); CASE(4, 1);
#undef CASE
    return hipErrorInvalidConfiguration;
}

hipError_t launch_fwd_stream(int dtype, const FwdStreamParams &p, int mt, int nt, int grid, int lds, hipStream_t s, int *occ) {
    if (dtype == FASTLSTM_FP32) return fwd_stream_t<float>(p, mt, nt, grid, lds, s, occ);
    if (dtype == FASTLSTM_FP16) return fwd_stream_t<_Float16>(p, mt, nt, grid, lds, s, occ);
    return fwd_stream_t<__bf16>(p, mt, nt, grid, lds, s, occ);
}
hipError_t launch_bwd_stream(int dtype, const BwdStreamParams &p, int mtb, int nt, int grid, int lds, hipStream_t s, int *occ) {
    if (dtype == FASTLSTM_FP32) return bwd_stream_t<float>(p, mtb, nt, grid, lds, s, occ);
    if (dtype == FASTLSTM_FP16) return bwd_stream_t<_Float16>(p, mtb, nt, grid, lds, s, occ);
    return bwd_stream_t<__bf16>(p, mtb, nt, grid, lds, s, occ);
}

template <typename T>
static hipError_t pack_t(bool backward, const void *Wh, unsigned char *wpack, int H, int KS, int KSP, int mt, int n_ht,
                         hipStream_t s) {
    const size_t total = (size_t)n_ht * mt * KSP * kWave;
    const int grid = (int)std::min<size_t>((total + 255) / 256, 16384);
    if (backward) pack_wh_bwd_kernel<T><<<grid, 256, 0, s>>>(static_cast<const T *>(Wh), wpack, H, KS, KSP, mt, n_ht);
    else pack_wh_fwd_kernel<T><<<grid, 256, 0, s>>>(static_cast<const T *>(Wh), wpack, H, KS, KSP, mt, n_ht);
    return hipGetLastError();
}
hipError_t launch_pack_wh(int dtype, bool backward, const void *Wh, unsigned char *wpack, int H, int KS, int KSP, int mt,
                          int n_ht, hipStream_t s) {
    if (dtype == FASTLSTM_FP32) return pack_t<float>(backward, Wh, wpack, H, KS, KSP, mt, n_ht, s);
    if (dtype == FASTLSTM_FP16) return pack_t<_Float16>(backward, Wh, wpack, H, KS, KSP, mt, n_ht, s);
    return pack_t<__bf16>(backward, Wh, wpack, H, KS, KSP, mt, n_ht, s);
}

}  // namespace fastlstm

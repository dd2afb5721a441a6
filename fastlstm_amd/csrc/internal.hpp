// Declarations shared between the translation units of libfastlstm_hip.so.
#pragma once
#include <algorithm>

#include "common.hpp"

namespace fastlstm {

struct GemmParams;
struct FwdParams;
struct BwdParams;
struct FwdXcdParams;
struct BwdXcdParams;

hipError_t launch_gemm(int dtype, const GemmParams &p, bool a_km, bool b_km, hipStream_t s);
// diagnostics: the stand-alone 16-bit tile launches in their earlier form (gemm16_onetile_kernel)
void set_gemm_baseline(int on);
int gemm_baseline();
hipError_t launch_colsum_final(int dtype, const float *part, void *out, int C, int chunks, hipStream_t s);
hipError_t launch_colsum(int dtype, const void *in, void *out, float *part, int R, int C, int chunks,
                         hipStream_t s);
int gemm_bk(int dtype);
bool gemm16_eligible(int dtype, int M, int N, int K, int lda, int ldb, bool a_km, bool b_km);
void set_gemm_trace(long long *buf);
void gemm_plan(int dtype, int M, int N, int K, int lda, int ldb, bool a_km, bool b_km, bool allow_split,
               int *tile, int *splits);
hipError_t launch_gemm_tiled(int dtype, const GemmParams &p, bool a_km, bool b_km, int tile, hipStream_t s);
// dWx[M][I], dWh[M][H], db[M] from d_ifgo[K][M], x[K][I], h[K][H] in one launch (16-bit shapes that
// wgrad_merged_plan accepts; ws holds wgrad_merged_workspace bytes)
bool wgrad_merged_plan(int dtype, int M, int I, int H, int K, int *splits, int *k_per_split, bool *merged);
size_t wgrad_merged_workspace(int dtype, int M, int I, int H, int K);
hipError_t launch_wgrad_merged(int dtype, const void *d_ifgo, const void *x, const void *h, void *dWx, void *dWh, void *db,
                               void *ws, int M, int I, int H, int K, hipStream_t s);
// K5, K8, K9 and the bias gradient of a narrow 16-bit layer in one pass over d_ifgo (gemm_small.hpp); dx may be null,
// and so may dWx, dWh, db (all three); ws: small_bwd_workspace bytes
bool small_bwd_eligible(int dtype, int R, int I, int H);
size_t small_bwd_workspace(int R, int I, int H);
hipError_t launch_small_bwd(int dtype, const void *d_ifgo, const void *Wx, const void *x, const void *h, void *dx, void *dWx,
                            void *dWh, void *db, void *ws, int R, int I, int H, hipStream_t s);

hipError_t launch_small_k1(int dtype, const void *x, const void *Wx, const void *bx, const void *bh, void *ifgo, int R, int I,
                           int H, hipStream_t s);

// one function per element type (separate translation units, compiled in parallel)
#define FASTLSTM_DECL_REC(SUF)                                                                       \
    hipError_t launch_fwd_##SUF(const FwdParams &p, int ht, int bt, int split, int grid, int lds,   \
                                hipStream_t s, int *max_blocks_per_cu);                              \
    hipError_t launch_bwd_##SUF(const BwdParams &p, int ht, int bt, int split, int grid, int lds,   \
                                hipStream_t s, int *max_blocks_per_cu);                              \
    hipError_t launch_fwd_wreg_##SUF(const FwdParams &p, int mt, int ntw, int grid, int lds,        \
                                     hipStream_t s, int *max_blocks_per_cu);                         \
    hipError_t launch_fwd_xcd_##SUF(const FwdXcdParams &p, int mt, int nkw, int ntw, int nwv, int grid, int lds, \
                                    hipStream_t s, int *max_blocks_per_cu);                          \
    hipError_t launch_bwd_xcd_##SUF(const BwdXcdParams &p, int mt, int nkw, int ntw, int grid, int lds, \
                                    hipStream_t s, int *max_blocks_per_cu);                          \
    hipError_t launch_fwd_xcd_help_##SUF(const FwdXcdParams &p, int ntw, int grid, int lds, hipStream_t s, \
                                         int *max_blocks_per_cu);                                 \
    hipError_t launch_bwd_xcd_help_##SUF(const BwdXcdParams &p, int mt, int nkw, int ntw, int grid, int lds, \
                                         hipStream_t s, int *max_blocks_per_cu);                  \
    hipError_t launch_fwd_wide_##SUF(const FwdXcdParams &p, int nkw, int nt, int grid, int lds, hipStream_t s, \
                                     int *max_blocks_per_cu);                                    \
    hipError_t launch_bwd_wide_##SUF(const BwdXcdParams &p, int nkw, int nt, int grid, int lds, hipStream_t s, \
                                     int *max_blocks_per_cu);                                    \
    hipError_t launch_bwd_wide_split_##SUF(const BwdXcdParams &p, int nkw, int v, int grid, int lds, hipStream_t s, \
                                           int *max_blocks_per_cu);
FASTLSTM_DECL_REC(f32)
FASTLSTM_DECL_REC(f16)
FASTLSTM_DECL_REC(bf16)
#undef FASTLSTM_DECL_REC

// streamed-weights kernels (recurrent_stream.hpp): plans with wave_split == 3
struct FwdStreamParams;
struct BwdStreamParams;
hipError_t launch_fwd_stream(int dtype, const FwdStreamParams &p, int mt, int nt, int grid, int lds, hipStream_t s,
                             int *max_blocks_per_cu);
hipError_t launch_bwd_stream(int dtype, const BwdStreamParams &p, int mtb, int nt, int grid, int lds, hipStream_t s,
                             int *max_blocks_per_cu);
hipError_t launch_pack_wh(int dtype, bool backward, const void *Wh, unsigned char *wpack, int H, int KS, int KSP, int mt,
                          int n_ht, hipStream_t s);
// Workspace layout of a streamed-weights plan: header | counters | per batch chunk: flags, 2 exchange slots | packed W_h
struct StreamLayout {
    int KS, KSP;            // k-steps of the contraction, padded to the K loop's granule
    int mt;                 // operand row tiles of a workgroup's weight slice (forward: ht / 4, reverse: ht / 16)
    size_t flags_bytes, slot_bytes, chunk_bytes, wpack_off, wpack_bytes;
};
StreamLayout stream_layout(const fastlstm_plan &plan, int H, int dtype, bool backward);

int fwd_lds_bytes(int H, int dtype, int ht, int bt, int split, bool sync);
int bwd_lds_bytes(int H, int dtype, int ht, int bt, int split, bool sync);
size_t recurrent_flags_bytes(int n_bt, int n_ht);
size_t recurrent_slot_bytes(int H, int dtype, int bt, int n_bt, bool backward);
size_t recurrent_ws_bytes(int H, int dtype, int bt, int n_bt, int n_ht, int chunks, bool backward, bool sync,
                          int slots);

}  // namespace fastlstm

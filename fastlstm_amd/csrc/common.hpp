// Shared device/host helpers for the gfx950 LSTM kernels: element-type traits,
// MFMA wrappers with one fragment convention for all three dtypes, fast gate
// non-linearities and the host-side launch plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fastlstm_hip.h"
#include "../../include/fastlstm_hip_diag.h"

namespace fastlstm {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kThreads = 256;  // 4 waves, one per SIMD
constexpr int kFragBytes = 1024;  // one MFMA operand block: 64 lanes x 16 bytes

// ---------------------------------------------------------------------------
// Element traits.  A "fragment" is 16 bytes per lane: EPL elements of K for the
// matrix row (lane % 16), K-group (lane / 16).  One "k-step" contracts
// KSTEP = 4 * EPL elements of K:
//   16-bit: one v_mfma_f32_16x16x32 (lane holds 8 consecutive k),
//   fp32  : four v_mfma_f32_16x16x4 (MFMA e contracts element e of all 4 lane
//           groups; the K order inside a k-step is permuted identically for
//           both operands, which leaves the product unchanged).
// Logical k of (kstep, lanegroup q, element e) = kstep*KSTEP + q*EPL + e.
// ---------------------------------------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int EPL = 4, KSTEP = 16, BYTES = 4;
    static constexpr int DT = FASTLSTM_FP32;
    static __device__ __forceinline__ float to_f32(float v) { return v; }
    static __device__ __forceinline__ float from_f32(float v) { return v; }
};
template <> struct Elem<_Float16> {
    static constexpr int EPL = 8, KSTEP = 32, BYTES = 2;
    static constexpr int DT = FASTLSTM_FP16;
    static __device__ __forceinline__ float to_f32(_Float16 v) { return (float)v; }
    static __device__ __forceinline__ _Float16 from_f32(float v) { return (_Float16)v; }
};
template <> struct Elem<__bf16> {
    static constexpr int EPL = 8, KSTEP = 32, BYTES = 2;
    static constexpr int DT = FASTLSTM_BF16;
    static __device__ __forceinline__ float to_f32(__bf16 v) { return (float)v; }
    static __device__ __forceinline__ __bf16 from_f32(float v) { return (__bf16)v; }
};

// D(16x16) += A(16 x KSTEP) . B(KSTEP x 16); a/b are the 16-byte fragments.
// Result layout: lane holds D[4*(lane/16) + e][lane % 16], e = 0..3.
template <typename T>
__device__ __forceinline__ f32x4 mfma_kstep(const u32x4 a, const u32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma_kstep<_Float16>(const u32x4 a, const u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma_kstep<__bf16>(const u32x4 a, const u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma_kstep<float>(const u32x4 a, const u32x4 b, f32x4 c) {
    const f32x4 af = __builtin_bit_cast(f32x4, a), bf = __builtin_bit_cast(f32x4, b);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[0], bf[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[1], bf[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[2], bf[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[3], bf[3], c, 0, 0, 0);
    return c;
}

// Gate non-linearities in fp32.  The 16-bit types use the hardware exp2 / rcp approximations as they come (error
// ~1e-7 absolute, far below the 16-bit rounding of every stored value).  The fp32 element type (parity bar 1e-4,
// element-wise, against nn.LSTM over 100+ steps) uses the same two instructions with the reciprocal refined by one
// Newton step: absolute error ~2e-7 per activation -- the library exp, tanh and the IEEE division it replaces are
// ~250 vector instructions per cell against ~60, and the gate arithmetic is a fifth of an fp32 step (T = 128,
// B = 16, I = H = 256: forward 2.2-2.3 -> 2.0-2.1 us per step, reverse 2.5-2.7 -> 2.3-2.4; worst element of that
// shape's outputs and gradients against nn.LSTM at 0.29 of the bar, 0.39 over the reference's test grid -- 0.43 with
// the library forms: the fp32 summation order sets it, not the activations).
// -DFASTLSTM_FP32_LIBM brings the library forms back.
// 1 / d for d >= 1: the hardware reciprocal and one Newton step (what an IEEE division spends 10 instructions on)
__device__ __forceinline__ float rcp_refined(float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(r, __builtin_fmaf(-d, r, 1.0f), r);
}
template <bool ACCURATE> __device__ __forceinline__ float sigmoidf_(float x) {
    if constexpr (ACCURATE) {
#ifdef FASTLSTM_FP32_LIBM
        return 1.0f / (1.0f + expf(-x));
#else
        return rcp_refined(1.0f + __expf(fminf(-x, 80.0f)));   // (e^80 is finite: the Newton step has no inf x 0)
#endif
    } else {
        return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
    }
}
template <bool ACCURATE> __device__ __forceinline__ float tanhf_(float x) {
    if constexpr (ACCURATE) {
#ifdef FASTLSTM_FP32_LIBM
        return tanhf(x);
#else
        return 1.0f - 2.0f * rcp_refined(1.0f + __expf(fminf(2.0f * x, 80.0f)));
#endif
    } else {
        // 1 - 2/(1+e^{2x}); saturates correctly at +-inf of the exponential
        return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * x));
    }
}

constexpr int kNumXcd = 8;

// Workgroups are handed to the 8 XCDs (each with its own L2) round-robin by id.  Numbering
// them XCD-major gives every XCD a contiguous range of logical ids, so that neighbours in
// the logical order -- the hidden tiles of one batch tile, adjacent C tiles of a GEMM --
// share an L2.
__device__ __forceinline__ int xcd_major_id(int bid, int nwg) {
    const int xcd = bid % kNumXcd, slot = bid / kNumXcd;
    const int base = nwg / kNumXcd, rem = nwg % kNumXcd;
    return xcd * base + (xcd < rem ? xcd : rem) + slot;
}

__host__ __device__ inline int cdiv(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline int elem_bytes(int dtype) { return dtype == FASTLSTM_FP32 ? 4 : 2; }
inline bool dtype_ok(int dtype) { return dtype >= FASTLSTM_FP32 && dtype <= FASTLSTM_BF16; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Workspace header shared by the two recurrent kernels (first 256 bytes).
struct WsHeader {
    int abort_flag;  // set to 1 by the first barrier wait that times out
    int timeout_group, timeout_step, timeout_seen;
    int xcd_rotation;  // 1 + (XCD of a workgroup - its id) mod 8, agreed on by the workgroups of an XCD-placed launch
    int reserved[59];
};
static_assert(sizeof(WsHeader) == 256, "workspace header is 256 bytes");

// Chunk counters of the launches that run GEMM tiles next to a recurrence: three arrays of
// kMaxChunks device-scope counters behind the WsHeader, inside the 1 KiB header block (zero at launch).
constexpr int kMaxChunks = 64;
inline int *ws_chunk_counters(WsHeader *hdr, int which) { return reinterpret_cast<int *>(hdr + 1) + which * kMaxChunks; }

// Recurrence workspace: header block (1 KiB, WsHeader in front) | 64 KiB of L2 barrier counters of
// the XCD-local kernels (plans with a cross-CU barrier only) | flags | exchange slots.
constexpr size_t kWsHeaderBytes = 1024;
static_assert(sizeof(WsHeader) + 3 * kMaxChunks * sizeof(int) <= kWsHeaderBytes, "chunk counters fit the header block");
constexpr size_t kWsCounterBytes = 65536;

long long spin_limit_ticks();

}  // namespace fastlstm

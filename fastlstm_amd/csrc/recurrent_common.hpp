// Pieces shared by the forward and the reverse persistent kernels: the
// XCD-aware workgroup -> (batch tile, hidden tile) map and the per-timestep
// flag barrier between the hidden tiles of one batch tile.
//
// Barrier protocol (replaces the atomic counter of fastlstm/kernels.py:546-548,
// 659-661 and 1355-1359): every workgroup owns ONE int flag that it overwrites
// with the number of data versions it has published so far (no read-modify-write,
// no contention on a shared counter); a consumer polls the n_htiles flags of its
// group with one coalesced load per poll until all of them reached the version it
// needs.  The 8 XCDs of an MI355X have separate L2s, so the exchange data and the
// flags are WRITTEN with device-scope stores (sc1: write through to memory) and the
// flags are polled with device-scope loads.  That keeps the per-step critical path free
// of whole-L2 write-backs and invalidates: a producer drains its own exchange stores
// (s_waitcnt vmcnt(0)), the workgroup meets at a barrier, one thread raises the flag.
// The exchange DATA is read in one of two ways:
//  * history ring (default): every timestep writes a fresh slot of the exchange buffer, so
//    no cache can hold a stale copy of an address before its only write; consumers use
//    ordinary cached loads and the 32 CUs of an XCD share one fetch through their L2
//    (the data crosses the fabric once per XCD instead of once per CU);
//  * coherent loads (sc1, miss the non-coherent cache levels): used when the workspace is
//    too small for T+1 slots, or when two workgroups write parts of the same 128-byte line.
// Every wait is bounded: after `spin_limit` ticks of the 100 MHz clock it raises an
// abort flag in the workspace header that ends every other wait as well, so the grid
// always drains.
#pragma once
#include <type_traits>

#include "common.hpp"

namespace fastlstm {

constexpr int kAuxDevice = 16;  // buffer-instruction cache policy: sc1 = device scope
constexpr int kMaxSideBySide = 4;   // independent recurrences of one shape in one launch of the XCD-local kernels

// Exchange buffer in global memory, addressed through a buffer resource so that the
// 16-byte operand loads can carry the device-scope cache policy.
struct XchgGlobal {
    __amdgpu_buffer_rsrc_t rsrc;
    unsigned char *base;
    __device__ __forceinline__ XchgGlobal(unsigned char *b, unsigned bytes)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(b, 0, bytes, 0x00020000)), base(b) {}
    // COHERENT: device-scope load (sc1); otherwise an ordinary cached load
    template <bool COHERENT> __device__ __forceinline__ u32x4 load16(unsigned off) const {
        if constexpr (COHERENT) return __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, kAuxDevice);
        else return __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
    }
    template <typename T> __device__ __forceinline__ void store_elem(unsigned off, T v) const {
        if constexpr (sizeof(T) == 2) {
            __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), rsrc, off, 0, kAuxDevice);
        } else {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rsrc, off, 0, kAuxDevice);
        }
    }
    __device__ __forceinline__ void store8(unsigned off, u32x2 v) const {
        __builtin_amdgcn_raw_buffer_store_b64(v, rsrc, off, 0, kAuxDevice);
    }
    __device__ __forceinline__ void store16(unsigned off, u32x4 v) const {
        __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, off, 0, kAuxDevice);
    }
};

// Same interface over LDS (barrier-free small-H kernels: the exchange never leaves the CU).
struct XchgLds {
    unsigned char *base;
    __device__ __forceinline__ XchgLds(unsigned char *b, unsigned) : base(b) {}
    template <bool COHERENT> __device__ __forceinline__ u32x4 load16(unsigned off) const {
        return *reinterpret_cast<const u32x4 *>(base + off);
    }
    template <typename T> __device__ __forceinline__ void store_elem(unsigned off, T v) const {
        *reinterpret_cast<T *>(base + off) = v;
    }
    __device__ __forceinline__ void store8(unsigned off, u32x2 v) const { *reinterpret_cast<u32x2 *>(base + off) = v; }
    __device__ __forceinline__ void store16(unsigned off, u32x4 v) const { *reinterpret_cast<u32x4 *>(base + off) = v; }
};


// f(integral_constant<int, I>) for I = 0 .. N-1, each with its own compile-time index
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// lanes 0..7 of every row of 16 lanes keep lo, lanes 8..15 take hi of the lane 8 below (row_ror:8 into banks 2 and 3)
__device__ __forceinline__ float fold_upper_half(float lo, float hi) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, lo), __builtin_bit_cast(int, hi), 0x128, 0xf, 0xc, false));
}
// lanes 4j .. 4j + 3 of every row of 16 lanes take v_j of the lane 4j below (row_ror:4j into bank j)
__device__ __forceinline__ float fold_quarters(float v0, float v1, float v2, float v3) {
    int r = __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v0), __builtin_bit_cast(int, v1), 0x124, 0xf, 0x2, false);
    r = __builtin_amdgcn_update_dpp(r, __builtin_bit_cast(int, v2), 0x128, 0xf, 0x4, false);
    r = __builtin_amdgcn_update_dpp(r, __builtin_bit_cast(int, v3), 0x12c, 0xf, 0x8, false);
    return __builtin_bit_cast(float, r);
}

// A value that is the same in all lanes, moved to scalar registers (the compiler cannot always tell).
__device__ __forceinline__ int uniform_int(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename P> __device__ __forceinline__ P *uniform_ptr(P *ptr) {
    const unsigned long long v = reinterpret_cast<unsigned long long>(ptr);
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return reinterpret_cast<P *>(((unsigned long long)hi << 32) | lo);
}

// Called by wave 0 of a workgroup.  flags: the n flags of this barrier group.  NAP: s_sleep units
// (64 clocks each) between polls; waits that are expected to last many microseconds nap longer so
// that their polling stays out of the way of the traffic they wait for.
template <int NAP = 1>
__device__ __forceinline__ void wait_versions(const int *flags, int n, int target, WsHeader *hdr,
                                              long long spin_limit, int group, int step) {
    const int lane = threadIdx.x & (kWave - 1);
    long long t0 = 0;
    int polls = 0;
    for (;;) {
        int ok = 1;
        for (int j = lane; j < n; j += kWave)
            ok &= (__hip_atomic_load(flags + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= target);
        if (__all(ok)) break;
        __builtin_amdgcn_s_sleep(NAP);
        // a spin limit <= 1 means "give up at the first failed poll" (host-forced failure path)
        if (++polls >= 32 || spin_limit <= 1) {
            polls = 0;
            if (__hip_atomic_load(&hdr->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
            const long long now = (long long)wall_clock64();
            if (t0 == 0 && spin_limit > 1) {
                t0 = now;
            } else if (now - t0 > spin_limit) {
                if (lane == 0) {
                    hdr->timeout_group = group;
                    hdr->timeout_step = step;
                    __hip_atomic_store(&hdr->abort_flag, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                }
                break;
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // compiler ordering only: the data is read at device scope
}

// Called by all threads of the workgroup after they stored the data of `version`.
__device__ __forceinline__ void publish_version(int *flag, int version) {
    // every wave drains its own (write-through) exchange stores before the workgroup
    // barrier, then one thread raises the flag
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(flag, version, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Members of a barrier group that is placed by XCD.  The hardware deals the workgroups of a dispatch to
// the 8 XCDs in turn, but not always starting with XCD 0 (seen: a dispatch replayed from a HIP graph, and
// eager dispatches after it, start at another XCD): workgroup i runs on XCD (i + r) % 8 with one r per
// dispatch.  The grouping i % 8 == group % 8 puts a group on ONE XCD for every r, which is all the kernels
// need.  What they cannot survive is a dispatch without a common r: a member on another XCD than its
// peers would exchange through the wrong L2 and read stale lines without ever timing out.  So every
// member checks: the first one to arrive records its r in the workspace header, every other one
// compares, and a mismatch raises the abort flag (ends every wait of the launch; timeout_group = -3,
// timeout_step = the workgroup id, timeout_seen = its XCD).  One register read and one atomic per workgroup
// and launch.
__device__ __forceinline__ void check_xcd_placement(WsHeader *hdr) {
    if (threadIdx.x == 0) {
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        const int mine = 1 + (int)(((xcc & 15u) + kNumXcd - blockIdx.x % kNumXcd) % kNumXcd);
        int expected = 0;
        if (!__hip_atomic_compare_exchange_strong(&hdr->xcd_rotation, &expected, mine, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT) &&
            expected != mine) {
            hdr->timeout_group = -3;
            hdr->timeout_step = (int)blockIdx.x;
            hdr->timeout_seen = (int)(xcc & 15u);
            __hip_atomic_store(&hdr->abort_flag, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Unsigned vector type of N bytes, for moving N / sizeof(T) neighbouring elements with one access.
template <int N> struct VecBytes;
template <> struct VecBytes<2> { using type = unsigned short; };
template <> struct VecBytes<4> { using type = unsigned; };
template <> struct VecBytes<8> { using type = u32x2; };
template <> struct VecBytes<16> { using type = u32x4; };

// Byte offset of element k of matrix row r inside a run of fragment blocks
// (block = 64 lanes x 16 B; lane = 16*(lane group) + row).
template <typename T> __device__ __forceinline__ int frag_offset(int r, int k) {
    using E = Elem<T>;
    const int ks = k / E::KSTEP, kk = k % E::KSTEP;
    return (ks * kWave + (kk / E::EPL) * 16 + r) * 16 + (kk % E::EPL) * E::BYTES;
}

}  // namespace fastlstm

// Pieces shared by the forward and the reverse persistent kernels: the
// XCD-aware workgroup -> (batch tile, hidden tile) map and the per-timestep
// flag barrier between the hidden tiles of one batch tile.
//
// Barrier protocol (replaces the atomic counter of fastlstm/kernels.py:546-548,
// 659-661 and 1355-1359): every workgroup owns ONE int flag that it overwrites
// with the number of data versions it has published so far (no read-modify-write,
// no contention on a shared counter); a consumer polls the n_htiles flags of its
// group with one coalesced load per poll until all of them reached the version it
// needs.  Publishing is a device-scope release (L2 write-back), waiting ends in a
// device-scope acquire (L1/L2 invalidate), because the 8 XCDs of an MI355X have
// separate L2s.  Every wait is bounded: after `spin_limit` ticks of the 100 MHz
// clock it raises an abort flag in the workspace header that ends every other
// wait as well, so the grid always drains.
#pragma once
#include "common.hpp"

namespace fastlstm {

constexpr int kNumXcd = 8;

// Workgroups are handed to the XCDs round-robin by id.  Number the workgroups
// XCD-major so that consecutive logical ids -- the hidden tiles of one batch
// tile -- sit on as few XCDs (L2s) as possible.
__device__ __forceinline__ int xcd_major_id(int bid, int nwg) {
    const int xcd = bid % kNumXcd, slot = bid / kNumXcd;
    const int base = nwg / kNumXcd, rem = nwg % kNumXcd;
    return xcd * base + (xcd < rem ? xcd : rem) + slot;
}

// Called by wave 0 of a workgroup.  flags: the n flags of this barrier group.
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
        __builtin_amdgcn_s_sleep(1);
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
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

// Called by all threads of the workgroup after they stored the data of `version`.
__device__ __forceinline__ void publish_version(int *flag, int version) {
    // every wave drains its own stores to L2 before the workgroup barrier, then
    // one thread writes L2 back to memory and raises the flag
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0)
        __hip_atomic_store(flag, version, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// Byte offset of element k of matrix row r inside a run of fragment blocks
// (block = 64 lanes x 16 B; lane = 16*(lane group) + row).
template <typename T> __device__ __forceinline__ int frag_offset(int r, int k) {
    using E = Elem<T>;
    const int ks = k / E::KSTEP, kk = k % E::KSTEP;
    return (ks * kWave + (kk / E::EPL) * 16 + r) * 16 + (kk % E::EPL) * E::BYTES;
}

}  // namespace fastlstm

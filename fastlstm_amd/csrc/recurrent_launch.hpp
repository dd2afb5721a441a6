// Launch helper shared by the translation units that instantiate the persistent kernels.
#pragma once
#include <map>
#include <mutex>

#include "internal.hpp"

namespace fastlstm {
namespace {

struct OccKey {
    const void *fn;
    int lds;
    bool operator<(const OccKey &o) const { return fn < o.fn || (fn == o.fn && lds < o.lds); }
};

template <typename K, typename P>
hipError_t launch_one(K kern, const P &p, int grid, int lds, hipStream_t s, int *max_blocks_per_cu,
                      int threads = kThreads) {
    // the LDS attribute and the occupancy of (kernel, LDS size) are looked up once
    static std::map<OccKey, int> cache;
    static std::mutex mu;
    int occ;
    {
        std::lock_guard<std::mutex> lock(mu);
        const OccKey key{reinterpret_cast<const void *>(kern), lds};
        auto it = cache.find(key);
        if (it == cache.end()) {
            hipError_t e = hipFuncSetAttribute(key.fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
            if (e != hipSuccess) return e;
            int nb = 0;
            e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kern, threads, (size_t)lds);
            if (e != hipSuccess) return e;
            it = cache.emplace(key, nb).first;
        }
        occ = it->second;
    }
    if (max_blocks_per_cu) *max_blocks_per_cu = occ;
    if (grid <= 0) return hipSuccess;  // query only
    hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), (size_t)lds, s, p);
    return hipGetLastError();
}

}  // namespace
}  // namespace fastlstm

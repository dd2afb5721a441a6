// Diagnostics: the latency bound of one recurrence step, measured with the recurrence's own
// barrier and exchange code and nothing else.
//
// A timestep of the persistent kernels (which replace fastlstm/kernels.py:414-663, 1201-1409) is a
// chain: publish my part of h_t -> wait until every member of the barrier group has published ->
// fetch the group's whole h_t -> MFMA -> gates.  The first three links are pure latency that no
// amount of arithmetic throughput removes; this kernel runs exactly those links (the functions the
// real kernels call) for `steps` rounds so that the host can time them:
//   mode 0  empty barrier: publish + wait only
//   mode 1  + every member stores its share of a `rows`-row h tile into the step's exchange slot (slot t % 2)
//   mode 2  + every wave fetches its operand blocks of the step with the loads the real kernels use (they go
//           past the L1 to the L2: a slot is rewritten every second step)
//   mode 3, 4  (kind 0) the same exchange WITHOUT a barrier: a ring of 4 slots whose unwritten values hold
//           a sentinel bit pattern (all ones: a NaN no gate output produces); a member stores its share
//           of h_{t+1}, resets its share of the slot two versions back, and every wave polls its operand
//           blocks with loads that bypass the L1 (mode 3: sc1, mode 4: sc0 sc1) until no sentinel is left
// group kinds:
//   0  XCD-local group: `members` (<= 32) workgroups of ONE XCD, counters in its L2, polled with
//      scalar loads (recurrent_fwd_xcd.hpp)
//   1  flag group over all XCDs: `members` (<= 256) workgroups, one flag each, device-scope stores
//      and loads (recurrent_common.hpp; the general and the register-resident kernels)
// No counterpart in the reference.
#include "recurrent_fwd_xcd.hpp"
#include "recurrent_launch.hpp"

namespace fastlstm {

struct ProbeParams {
    WsHeader *hdr;
    int *counters;         // kind 0: [kXcdReplicas][kXcdCounterStride]; kind 1: one flag per member
    unsigned char *xbuf;   // modes 0-2: 2 slots, modes 3-4: 4 slots of [NT][KS] operand blocks of NT 16-row batch tiles
    int members, steps, KS, H, mode, kind, NT;
    long long spin_limit;
    unsigned *sink;        // one word per workgroup: keeps the loads alive
};

constexpr int kProbeWaves = 8;
constexpr int kProbeSlots = 4;   // exchange slots behind the counters (modes 0-2 use two of them)

__global__ __launch_bounds__(kWave *kProbeWaves) void step_probe_kernel(const ProbeParams p) {
    using T = _Float16;
    using E = Elem<T>;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int j;   // member index
    if (p.kind == 0) {
        if (blockIdx.x % kNumXcd != 0) return;
        j = blockIdx.x / kNumXcd;
    } else {
        j = xcd_major_id(blockIdx.x, gridDim.x);
    }
    if (j >= p.members) return;
    const int HT = p.H / p.members;   // hidden units of this member
    const int items = HT * 16 * p.NT; // (unit, batch row) values a member publishes per step
    const size_t xslot = (size_t)p.NT * p.KS * kFragBytes;
    const int shares = p.KS <= 32 ? 4 : 8;   // K-shares among the waves (4 x 2 unit halves, or 8: the real kernels' splits)
    int *my_counter = p.counters + (j % kXcdReplicas) * kXcdCounterStride;
    unsigned acc = 0;
    if (p.mode >= 3) {
        // ring of 4 slots, all sentinel at launch (host); slot v % 4 holds version v
        constexpr int R = 4;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(p.xbuf, 0, (unsigned)(R * xslot), 0x00020000);
        long long t0 = 0;
        bool dead = false;
        for (int t = 0; t < p.steps && !dead; ++t) {
            const unsigned wslot = (unsigned)(((t + 1) % R) * xslot), rslot = (unsigned)(((t + 3) % R) * xslot);
            for (int it = tid; it < items; it += kWave * kProbeWaves) {
                const unsigned off = ((it >> 4) / HT) * p.KS * kFragBytes + frag_offset<T>(it & 15, j * HT + (it >> 4) % HT);
                __builtin_amdgcn_raw_buffer_store_b16((unsigned short)((t + it) & 0x7fff), rs, wslot + off, 0, 0);
                if (t >= 1) __builtin_amdgcn_raw_buffer_store_b16((unsigned short)0xffffu, rs, rslot + off, 0, 0);
            }
            // poll version t + 1
            for (int nt = 0; nt < p.NT; ++nt) {
                int polls = 0;
                for (;;) {
                    u32x4 v[8];
#pragma unroll
                    for (int ki = 0; ki < 8; ++ki) {
                        const int ks = min(wave % shares + shares * ki, p.KS - 1);
                        const unsigned off = wslot + (unsigned)((nt * p.KS + ks) * kWave + lane) * 16u;
                        v[ki] = p.mode == 3 ? __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 16)
                                            : __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 17);
                    }
                    unsigned bad = 0;
#pragma unroll
                    for (int ki = 0; ki < 8; ++ki)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned w = v[ki][e];
                            bad |= ((w & 0xffffu) == 0xffffu) | ((w >> 16) == 0xffffu);
                            acc ^= w;
                        }
                    if (!__any(bad)) break;
                    if (++polls >= 64) {
                        polls = 0;
                        if (__hip_atomic_load(&p.hdr->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) { dead = true; break; }
                        const long long now = (long long)wall_clock64();
                        if (t0 == 0) t0 = now;
                        else if (now - t0 > p.spin_limit) {
                            if (lane == 0) {
                                p.hdr->timeout_group = 0;
                                p.hdr->timeout_step = t;
                                __hip_atomic_store(&p.hdr->abort_flag, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                            }
                            dead = true;
                            break;
                        }
                    }
                }
                if (dead) break;
            }
            dead = __syncthreads_or(dead);   // (also keeps the waves of a member within a step of each other, as the real kernels' barriers do)
        }
        if (acc == 0x9e3779b9u) p.sink[blockIdx.x] = acc;
        return;
    }
    for (int t = 0; t < p.steps; ++t) {
        // ---- publish version t + 1 ----------------------------------------------------------
        if (p.mode >= 1) {
            if (p.kind == 0) {
                const XchgL2 xw(p.xbuf + (size_t)((t + 1) & 1) * xslot, (unsigned)xslot);
                for (int it = tid; it < items; it += kWave * kProbeWaves)
                    xw.store_elem(((it >> 4) / HT) * p.KS * kFragBytes + frag_offset<T>(it & 15, j * HT + (it >> 4) % HT),
                                  E::from_f32((float)(t + it)));
            } else {
                const XchgGlobal xw(p.xbuf + (size_t)((t + 1) & 1) * xslot, (unsigned)xslot);
                for (int it = tid; it < items; it += kWave * kProbeWaves)
                    xw.store_elem(((it >> 4) / HT) * p.KS * kFragBytes + frag_offset<T>(it & 15, j * HT + (it >> 4) % HT),
                                  E::from_f32((float)(t + it)));
            }
        }
        if (p.kind == 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid < kXcdReplicas)
                __hip_atomic_fetch_add(p.counters + tid * kXcdCounterStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (wave == 0) wait_counter(my_counter, p.members * (t + 1), p.hdr, p.spin_limit, 0, t);
        } else {
            publish_version(p.counters + j, t + 1);
            if (wave == 0) wait_versions(p.counters, p.members, t + 1, p.hdr, p.spin_limit, 0, t);
        }
        __syncthreads();
        // ---- fetch the group's h_{t+1}: wave w takes k-steps w % shares, + shares, ... of every batch tile
        // (the K-shares of the real kernels), 8 blocks in flight at a time
        if (p.mode >= 2) {
            const XchgL2 xr(p.xbuf + (size_t)((t + 1) & 1) * xslot, (unsigned)xslot);
            for (int nt = 0; nt < p.NT; ++nt) {
                u32x4 v[8];
#pragma unroll
                for (int ki = 0; ki < 8; ++ki) {
                    const int ks = min(wave % shares + shares * ki, p.KS - 1);
                    const unsigned off = (unsigned)((nt * p.KS + ks) * kWave + lane) * 16u;
                    v[ki] = xr.load16_l2(off);
                }
#pragma unroll
                for (int ki = 0; ki < 8; ++ki) acc ^= v[ki][0] ^ v[ki][1] ^ v[ki][2] ^ v[ki][3];
            }
        }
    }
    if (p.mode >= 2 && acc == 0x9e3779b9u) p.sink[blockIdx.x] = acc;   // (practically never: the loads just have to be used)
}

}  // namespace fastlstm

using namespace fastlstm;

extern "C" {

size_t fastlstm_diag_step_probe_bytes(int steps, int H, int rows) {
    if (steps <= 0 || H <= 0 || H % 32 || rows <= 0 || rows % 16) return 0;
    return kWsHeaderBytes + kWsCounterBytes + (size_t)kProbeSlots * (rows / 16) * (H / 32) * kFragBytes + 4096;
}

int fastlstm_diag_step_probe(int kind, int mode, int members, int H, int rows, int steps, void *ws, size_t ws_bytes,
                             void *stream) {
    if (!ws) return FASTLSTM_ERR_NULL;
    if (kind < 0 || kind > 1 || mode < 0 || mode > 4 || (mode >= 3 && kind != 0) || members <= 0 || steps <= 0 || H <= 0 || H % 32 || H % members ||
        H / members < 4 || members > (kind == 0 ? 32 : 256) || H > 8 * 8 * 32 || rows < 16 || rows > 64 || rows % 16)
        return FASTLSTM_ERR_DIM;
    if (!aligned16(ws)) return FASTLSTM_ERR_ALIGN;
    if (ws_bytes < fastlstm_diag_step_probe_bytes(steps, H, rows)) return FASTLSTM_ERR_WORKSPACE;
    unsigned char *wsb = static_cast<unsigned char *>(ws);
    ProbeParams p{};
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.counters = reinterpret_cast<int *>(wsb + kWsHeaderBytes);
    p.xbuf = wsb + kWsHeaderBytes + kWsCounterBytes;
    p.sink = reinterpret_cast<unsigned *>(p.xbuf + (size_t)kProbeSlots * (rows / 16) * (H / 32) * kFragBytes);
    p.members = members; p.steps = steps; p.KS = H / 32; p.H = H; p.mode = mode; p.kind = kind; p.NT = rows / 16;
    p.spin_limit = spin_limit_ticks();
    int occ = 0;
    if (launch_one(step_probe_kernel, p, 0, 0, nullptr, &occ, kWave * kProbeWaves) != hipSuccess) return FASTLSTM_ERR_HIP;
    if (occ < 1) return FASTLSTM_ERR_RESIDENCY;
    // one workgroup per CU of an 8 x 32 CU device, as the real launches; the workgroups without a role return at once
    const int grid = kind == 0 ? kNumXcd * 32 : members;
    return launch_one(step_probe_kernel, p, grid, 0, static_cast<hipStream_t>(stream), nullptr, kWave * kProbeWaves) == hipSuccess
               ? FASTLSTM_OK
               : FASTLSTM_ERR_HIP;
}

}  // extern "C"

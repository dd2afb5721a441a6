// extern "C" entry points of libfastlstm_hip.so (declared in include/fastlstm_hip.h).
// Every function validates its arguments before the first HIP call.
#include <atomic>
#include <mutex>

#include "gemm.hpp"
#include "internal.hpp"
#include "recurrent_bwd.hpp"
#include "recurrent_fwd.hpp"
#include "recurrent_bwd_xcd.hpp"
#include "recurrent_bwd_wide.hpp"
#include "recurrent_bwd_wide_split.hpp"
#include "recurrent_fwd_xcd.hpp"
#include "recurrent_stream.hpp"

using namespace fastlstm;

namespace fastlstm {

// What one recurrent launch covers and stores; handed down explicitly from the entry points.
struct LaunchOpts {
    int keep = 1;            // forward: 1 = store the gate pre-activations and every cell state (the reverse
                             // pass reads them), 0 = inference (the *_infer entry points)
    int row0 = 0, rows = 0;  // rows [row0, row0 + rows) of the batch; rows == 0: all of it.  A batch with more
                             // tiles than one XCD-local launch holds runs as several launches over row ranges
    // independent recurrences side by side beyond the first two (see try_multi): n_more of them, each its
    // operand pointers in the order of the single entry point (forward: ifgo, out, cell, Wh; reverse: dout, dh, dc,
    // ifgo, cell, d_ifgo, Wh)
    int n_more = 0;
    void *const (*more)[7] = nullptr;
};

static long long *g_rec_trace = nullptr;
static std::atomic<long long> g_spin_limit{400000000ll};  // 4 s of the 100 MHz clock
static std::atomic<int> g_families{7};   // diagnostics: bit 0 = XCD-local kernels allowed, bit 1 = register-resident wide kernels, bit 2 = their reverse form with teams
long long spin_limit_ticks() { return g_spin_limit.load(); }

namespace {

int check_dims(int T, int B, int I, int H) {
    if (T <= 0 || B <= 0 || I <= 0 || H <= 0) return FASTLSTM_ERR_DIM;
    const long long lim = (1ll << 31) - 1;
    if ((long long)T * B > lim || (long long)B * 4 * H > lim || 4ll * H * std::max(I, H) > lim) return FASTLSTM_ERR_DIM;
    return FASTLSTM_OK;
}

struct DeviceInfo {
    int num_cus = 0, lds = 0;
    int xcd_round_robin = 0;   // 1: the workgroups of a launch are dealt to the 8 XCDs in turn (probed once)
    // One pinned, device-visible word per device (allocated by the first planning call): a recurrent call
    // whose launches ended with the abort flag raised sets it when that work completes on the device, and
    // the next entry on the device reports it -- a failed barrier is never silent and costs no host sync.
    int *status_host = nullptr, *status_dev = nullptr;
};

// Every workgroup reports the XCD it runs on (hardware register XCC_ID).
__global__ void xcc_probe_kernel(int *out) {
    if (threadIdx.x == 0) {
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        out[blockIdx.x] = (int)(xcc & 15u);
    }
}

// 1 when the device has 8 XCDs x 32 CUs and deals the workgroups of a launch to the XCDs in turn
// (workgroup i on XCD (i + r) % 8 with one r for the whole dispatch; the kernels check r per launch).
// Uses pinned host memory the kernel writes directly: no device allocation.
int probe_xcd_round_robin(int num_cus) {
    if (num_cus != kNumXcd * 32) return 0;
    const int n = 4 * num_cus;
    int *buf = nullptr;
    if (hipHostMalloc(reinterpret_cast<void **>(&buf), n * sizeof(int), hipHostMallocMapped) != hipSuccess) return 0;
    for (int i = 0; i < n; ++i) buf[i] = -1;
    int ok = 0;
    int *dptr = nullptr;
    if (hipHostGetDevicePointer(reinterpret_cast<void **>(&dptr), buf, 0) == hipSuccess) {
        hipLaunchKernelGGL(xcc_probe_kernel, dim3(n), dim3(64), 0, nullptr, dptr);
        if (hipGetLastError() == hipSuccess && hipDeviceSynchronize() == hipSuccess) {
            // in turn, from whichever XCD the dispatch started at
            ok = buf[0] >= 0 && buf[0] < kNumXcd;
            for (int i = 0; i < n && ok; ++i)
                if (buf[i] != (buf[0] + i) % kNumXcd) ok = 0;
        }
    }
    (void)hipHostFree(buf);
    return ok;
}

DeviceInfo g_device_cache[64];
std::mutex g_device_mu;                       // guards g_device_cache
std::atomic<int> g_status_words{0};           // devices that have a status word (0: no entry ever looks)
void device_info_set_probe(int device, int rr, int *status_host, int *status_dev) {
    std::lock_guard<std::mutex> lock(g_device_mu);
    if (device < 0 || device >= 64) return;
    g_device_cache[device].xcd_round_robin = rr;
    if (status_host && !g_device_cache[device].status_host) {
        g_device_cache[device].status_host = status_host;
        g_device_cache[device].status_dev = status_dev;
        g_status_words.fetch_add(1);
    } else if (status_host) {
        (void)hipHostFree(status_host);   // (a recurrent call has given the device its word already)
    }
}

int device_info(int device, DeviceInfo *out) {
    DeviceInfo *cache = g_device_cache;
    if (device < 0) {
        if (hipGetDevice(&device) != hipSuccess) return FASTLSTM_ERR_HIP;
    }
    if (device >= 64) return FASTLSTM_ERR_HIP;
    std::lock_guard<std::mutex> lock(g_device_mu);
    if (cache[device].num_cus == 0) {
        int cus = 0, lds = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
            hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess)
            return FASTLSTM_ERR_HIP;
        cache[device].lds = lds;
        cache[device].xcd_round_robin = -1;   // probed on first use by a planning call (synchronises once)
        cache[device].num_cus = cus;
    }
    *out = cache[device];
    return FASTLSTM_OK;
}

// The probe synchronises the device, so it runs from fastlstm_plan_device (a host-side planning
// call) and never from a launch call, which may be under stream capture.
void probe_device(int device) {
    static std::mutex mu;
    std::lock_guard<std::mutex> lock(mu);
    DeviceInfo di;
    if (device_info(device, &di) != FASTLSTM_OK || di.xcd_round_robin >= 0) return;
    int cur = 0;
    if (hipGetDevice(&cur) != hipSuccess) return;
    if (device < 0) device = cur;
    if (device != cur && hipSetDevice(device) != hipSuccess) return;
    const int rr = probe_xcd_round_robin(di.num_cus);
    int *word = nullptr, *word_dev = nullptr;
    if (hipHostMalloc(reinterpret_cast<void **>(&word), 64, hipHostMallocMapped) == hipSuccess) {
        *word = 0;
        if (hipHostGetDevicePointer(reinterpret_cast<void **>(&word_dev), word, 0) != hipSuccess) {
            (void)hipHostFree(word);
            word = word_dev = nullptr;
        }
    }
    if (device != cur) (void)hipSetDevice(cur);
    device_info_set_probe(device, rr, word, word_dev);
}

// Results of a recurrent call that are overwritten with NaN when its launches ended with the abort flag raised
// (barrier time-out, workgroup on the wrong XCD): the failing call itself has returned success long before, so the
// failure has to travel with its data -- a loss, a gradient scaler or an isfinite check trips in the same step.
struct PoisonList {
    void *p[8];
    unsigned n[8];   // elements
    int count, dtype;
    void add(void *ptr, size_t elems) {
        if (ptr && count < 8) { p[count] = ptr; n[count] = (unsigned)std::min<size_t>(elems, 1u << 24); ++count; }
    }
};

// Behind the launches of a recurrent call: carries the abort flag of its workspace to the device's status word
// (if the device has one) and poisons the call's results.
__global__ void collect_status_kernel(const WsHeader *hdr, int *status_word, const PoisonList pl) {
    if (!__hip_atomic_load(&hdr->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return;
    if (threadIdx.x == 0 && status_word) __hip_atomic_store(status_word, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    for (int k = 0; k < pl.count; ++k)
        for (unsigned i = threadIdx.x; i < pl.n[k]; i += blockDim.x) {
            if (pl.dtype == FASTLSTM_FP32) static_cast<unsigned *>(pl.p[k])[i] = 0x7fc00000u;
            else static_cast<unsigned short *>(pl.p[k])[i] = pl.dtype == FASTLSTM_FP16 ? 0x7e00 : 0x7fc0;
        }
}

// The status word of the current device says that an earlier recurrent call failed: report it once.
int take_pending_status() {
    if (g_status_words.load() == 0) return FASTLSTM_OK;   // no device has a status word yet: nothing to look at
    DeviceInfo di;
    if (device_info(-1, &di) != FASTLSTM_OK || !di.status_host) return FASTLSTM_OK;
    if (__atomic_load_n(di.status_host, __ATOMIC_RELAXED) == 0) return FASTLSTM_OK;
    __atomic_store_n(di.status_host, 0, __ATOMIC_RELAXED);
    return FASTLSTM_ERR_TIMEOUT;
}

// A caller that never plans (fastlstm_plan_device) still gets a status word: allocated by its first recurrent
// call outside stream capture (pinned host memory; no device allocation, no synchronisation).
void ensure_status_word(int device, hipStream_t stream) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return;
    int *word = nullptr, *word_dev = nullptr;
    if (hipHostMalloc(reinterpret_cast<void **>(&word), 64, hipHostMallocMapped) != hipSuccess) return;
    *word = 0;
    if (hipHostGetDevicePointer(reinterpret_cast<void **>(&word_dev), word, 0) != hipSuccess) {
        (void)hipHostFree(word);
        return;
    }
    std::lock_guard<std::mutex> lock(g_device_mu);
    if (device < 0 || device >= 64 || g_device_cache[device].status_host) {
        (void)hipHostFree(word);   // (another thread was first)
        return;
    }
    g_device_cache[device].status_host = word;
    g_device_cache[device].status_dev = word_dev;
    g_status_words.fetch_add(1);
}

// Recurrent launches of one device run one after the other, whatever streams they are enqueued on.  A
// persistent launch holds its CUs until its last step; the workgroups of a second one on another stream get
// the CUs that are left, and where that is not all of a barrier group both launches wait on each other's CUs
// until the spin limit ends them (4 s).  So the library keeps one event per device: a recurrent entry point
// records it behind its launches, and the next one on a DIFFERENT stream makes its stream wait for it first
// (hipStreamWaitEvent: no host synchronisation).  Streams under capture are left alone: a graph orders its own
// nodes, and an event recorded into a capture could not be waited for outside it.
struct StreamOrder {
    hipEvent_t event = nullptr;
    hipStream_t last = nullptr;
    bool recorded = false;
};
StreamOrder g_order[64];
std::mutex g_order_mu;

static bool capturing(hipStream_t s) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone;
}

// At the start of every recurrent entry point: the failure of an earlier call, if one is pending; the wait
// for the last recurrent call of the device where that one went to another stream.
int begin_recurrent(void *stream_) {
    if (int rc = take_pending_status()) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return FASTLSTM_OK;
    std::lock_guard<std::mutex> lock(g_order_mu);
    StreamOrder &o = g_order[device];
    if (!o.recorded || o.last == stream || capturing(stream)) return FASTLSTM_OK;
    return hipStreamWaitEvent(stream, o.event, 0) == hipSuccess ? FASTLSTM_OK : FASTLSTM_ERR_HIP;
}

// may_create: false for the entry point that must not allocate anything (it records only into an event that a
// set-up call or an earlier entry point has created)
static void order_record(int device, hipStream_t stream, bool may_create = true) {
    if (device < 0 || device >= 64 || capturing(stream)) return;
    std::lock_guard<std::mutex> lock(g_order_mu);
    StreamOrder &o = g_order[device];
    if (!o.event) {
        if (!may_create) return;
        if (hipEventCreateWithFlags(&o.event, hipEventDisableTiming) != hipSuccess) {
            o.event = nullptr;
            return;
        }
    }
    if (hipEventRecord(o.event, stream) == hipSuccess) {
        o.last = stream;
        o.recorded = true;
    }
}

// Wraps a recurrent entry point: rc of its launches; on success the status collection is enqueued behind them.
// may_allocate: false for the entry point that must not allocate anything (no status word, no event then, unless a
// set-up call made them: fastlstm_plan_device, fastlstm_noalloc_scratch_bytes or an earlier entry point).
int finish_recurrent(int rc, void *ws, void *stream, const PoisonList &poison = PoisonList{}, bool may_allocate = true) {
    if (rc != FASTLSTM_OK) return rc;
    DeviceInfo di;
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device_info(device, &di) != FASTLSTM_OK) return rc;
    if (!di.status_dev && may_allocate) {
        ensure_status_word(device, static_cast<hipStream_t>(stream));
        (void)device_info(device, &di);
    }
    collect_status_kernel<<<1, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const WsHeader *>(ws), di.status_dev, poison);
    if (hipGetLastError() != hipSuccess) return FASTLSTM_ERR_HIP;
    order_record(device, static_cast<hipStream_t>(stream), may_allocate);
    return FASTLSTM_OK;
}

// the final slab [B*H] of a [T+1][B][H] state history
static void *last_slab(void *base, int T, int B, int H, int dtype) {
    return base ? static_cast<unsigned char *>(base) + (size_t)T * B * H * elem_bytes(dtype) : nullptr;
}
static PoisonList poison_fwd(int dtype, int T, int B, int H, void *out, void *cell, void *out_b = nullptr, void *cell_b = nullptr) {
    PoisonList pl{};
    pl.dtype = dtype;
    const size_t bh = (size_t)B * H;
    pl.add(last_slab(out, T, B, H, dtype), bh); pl.add(last_slab(cell, T, B, H, dtype), bh);
    pl.add(last_slab(out_b, T, B, H, dtype), bh); pl.add(last_slab(cell_b, T, B, H, dtype), bh);
    return pl;
}

typedef hipError_t (*FwdLauncher)(const FwdParams &, int, int, int, int, int, hipStream_t, int *);
typedef hipError_t (*BwdLauncher)(const BwdParams &, int, int, int, int, int, hipStream_t, int *);
FwdLauncher fwd_launcher(int dtype) {
    return dtype == FASTLSTM_FP32 ? launch_fwd_f32 : (dtype == FASTLSTM_FP16 ? launch_fwd_f16 : launch_fwd_bf16);
}
BwdLauncher bwd_launcher(int dtype) {
    return dtype == FASTLSTM_FP32 ? launch_bwd_f32 : (dtype == FASTLSTM_FP16 ? launch_bwd_f16 : launch_bwd_bf16);
}

typedef hipError_t (*FwdXcdLauncher)(const FwdXcdParams &, int, int, int, int, int, int, hipStream_t, int *);
typedef hipError_t (*BwdXcdLauncher)(const BwdXcdParams &, int, int, int, int, int, hipStream_t, int *);
typedef hipError_t (*FwdXcdHelpLauncher)(const FwdXcdParams &, int, int, int, hipStream_t, int *);

// Shape of an XCD-local launch (see recurrent_fwd_xcd.hpp / recurrent_bwd_xcd.hpp).
struct XcdCfg {
    int mt, nkw, ntw, nwv;     // unit tiles per workgroup, k-steps per wave (share), batch tiles, waves
    int n_ht, gpx, n_groups;   // members of a group, groups per XCD, groups of the launch
    int ks;                    // k-steps of the contraction
    int lds;
    size_t xslot;              // bytes of one exchange slot (the kernels use two)
};

// The XCD-local kernels apply when the device deals workgroups to XCDs in turn, the shape fits
// and the workspace holds a ring with one slot per exchanged version.
// `launch_rows`: batch rows of this launch (0: all B_all of them).
// copies > 1: that many recurrences of this shape share the launch, so the unit tile has to leave room for all their
// groups.
bool select_xcd(int T, int B_all, int H, int dtype, bool backward, size_t ws_bytes, XcdCfg *c, int launch_rows = 0,
                int copies = 1) {
    const int B = launch_rows ? launch_rows : B_all;
    DeviceInfo di;
    if (!(g_families.load() & 1) || device_info(-1, &di) != FASTLSTM_OK || di.xcd_round_robin != 1) return false;
    const int s = elem_bytes(dtype), kstep = dtype == FASTLSTM_FP32 ? 16 : 32;
    const int K = backward ? 4 * H : H;
    if (K % kstep || (H * s) % 16) return false;
    c->ks = K / kstep;
    const int ways = backward ? 8 : 4;   // K-shares
    const int per = cdiv(c->ks, ways);
    c->nkw = per <= 4 ? 4 : (per <= 8 ? 8 : ((backward && per <= 16) ? 16 : 0));
    if (!c->nkw) return false;
    // hidden units per workgroup: the smallest tile that puts a group on one XCD and all batch tiles in one launch
    const int hts_f[3] = {8, 16, 32}, hts_b[2] = {16, 32};
    const int *hts = backward ? hts_b : hts_f;
    const int n_hts = backward ? 2 : 3, rows = backward ? 16 : 4;   // weight rows per unit tile count as rows/4 fragments
    int ht = 0;
    c->ntw = 0;
    for (int hi = 0; hi < n_hts && !ht; ++hi) {
        const int cand = hts[hi];
        const int frags = (cand / rows) * c->nkw;   // per wave (forward: halved again by the unit split of 8 waves)
        if (H % cand || H / cand > 32 || cand * s < 16 || frags > (backward ? 32 : 64)) continue;
        // groups per XCD: as many as its 32 CUs hold, and no more than the workspace has barrier counters for
        const int groups_max = kNumXcd * std::min(32 / (H / cand), kXcdMaxGroups / kNumXcd);
        if (copies * cdiv(B, 16) <= groups_max) { ht = cand; c->ntw = 1; }
        else if (copies * cdiv(B, 32) <= groups_max) { ht = cand; c->ntw = 2; }
    }
    if (!ht) return false;
    c->mt = ht / rows;
    c->nwv = backward ? 8 : (c->mt * c->nkw > 32 ? 8 : 4);
    c->n_ht = H / ht;
    c->gpx = std::min(32 / c->n_ht, kXcdMaxGroups / kNumXcd);
    const int bt = 16 * c->ntw;
    c->n_groups = cdiv(B, bt);
    if (copies * c->n_groups > kNumXcd * c->gpx) return false;   // (the tile loop above guarantees it; the kernels index counters by group)
    c->xslot = (size_t)c->n_groups * c->ntw * c->ks * kFragBytes;
    if (ws_bytes < kWsHeaderBytes + kWsCounterBytes + 2 * (size_t)copies * c->xslot) return false;
    const int gseg = ht * s;
    const int red_blocks = backward ? 8 * c->mt * c->ntw : 4 * c->mt * c->ntw;
    c->lds = red_blocks * kFragBytes + bt * (4 * gseg + 16) + 2 * bt * (gseg + 16);
#ifdef FASTLSTM_TIMELINE
    c->lds += 4096;
#endif
    return true;
}

// GEMM work of `flop` on `n_helpers` CUs inside a recurrent launch of about rec_ms: worth while when the launch, which
// lasts as long as the longer of the two, beats the recurrence followed by the same work on the whole device.  A CU
// inside the launch sustains about 3.5 TFLOP/s on the 256 x 256 16-bit tiles.
static bool helpers_keep_up(double flop, int n_helpers, double rec_ms) {
    const double helper_ms = flop / (n_helpers * 3.5e9);
    return std::max(helper_ms, rec_ms) <= rec_ms + helper_ms * n_helpers / 256.0;
}

// In-kernel input projection: possible when the XCD-local forward kernel is the 8-wave one, at
// least a quarter of the CUs have no role in the recurrence, and K1 suits the 256 x 256 16-bit
// tile kernel.  Fills the k1 fields of *p (chunking by time) and returns true.
// The second layer of a stack that shares the launch (see FwdXcdParams::n_layers).
struct SecondLayer {
    const void *Wx, *bx, *bh, *Wh;
    void *ifgo, *out, *cell;
};

bool plan_k1_helpers(const XcdCfg &c, const void *x, const void *Wx, const void *bx, const void *bh, void *ifgo, int T,
                     int B, int I, int H, int dtype, FwdXcdParams *p, const SecondLayer *second = nullptr) {
    if (dtype == FASTLSTM_FP32 || c.nwv != 8 || c.mt != 8 || c.nkw != 8) return false;
    const int layers = second ? 2 : 1;
    if (layers * c.n_groups > kNumXcd * c.gpx) return false;   // every group needs its CUs on one XCD
    const int n_helpers = kNumXcd * 32 - layers * c.n_groups * c.n_ht;
    if (n_helpers < kNumXcd * (second ? 6 : 8)) return false;
    const int max_chunks = kMaxChunks;
    const int M = T * B, N = 4 * H;
    if (!gemm16_eligible(dtype, M, N, I, I, I, false, false) || N % 8) return false;
    if (!second && !helpers_keep_up(2.0 * M * N * I, n_helpers, T * (c.ntw == 1 ? 2.3e-3 : 3.8e-3))) return false;
    // two layers: both projections on the helpers; past 1.25 x the time of the two time loops side by side the layers
    // are better run one by one, each with more helpers (config E: 1.0)
    if (second && 2.0 * M * N * (I + H) / (n_helpers * 3.5e9) > 1.25 * T * 2.4e-3) return false;
    const int tiles_m = cdiv(M, 256), tiles_n = cdiv(N, 256);
    // a chunk: whole timesteps, about one round of the helpers, at most kMaxChunks chunks
    int base = 1;
    while ((base * 256) % B) ++base;                       // row tiles that hold whole timesteps
    int ct = std::max(1, n_helpers / tiles_n / base) * base;
    // the second layer starts a chunk behind the first: no more than 64 timesteps per chunk (B = 16: a round of the
    // helpers would be 192)
    if (second) ct = std::min(ct, std::max(1, 64 * B / 256 / base) * base);
    while (cdiv(tiles_m, ct) > max_chunks) ct += base;
    const int steps = ct * 256 / B;
    if (steps < 2) return false;
    p->n_layers = layers;
    p->n_active = c.n_groups * c.n_ht;
    if (second) {
        if (!gemm16_eligible(dtype, M, N, H, H, H, false, false)) return false;
        p->ifgo2 = second->ifgo; p->out2 = second->out; p->cell2 = second->cell; p->Wh2 = second->Wh;
        p->k1b = GemmParams{};
        p->k1b.A = static_cast<const unsigned char *>(p->out) + (size_t)B * H * elem_bytes(dtype);   // out[1:] of the first layer
        p->k1b.B = second->Wx; p->k1b.C = second->ifgo; p->k1b.bias0 = second->bx; p->k1b.bias1 = second->bh;
        p->k1b.M = M; p->k1b.N = N; p->k1b.K = H;
        p->k1b.lda = H; p->k1b.ldb = H; p->k1b.ldc = N;
        p->k1b.splits = 1; p->k1b.k_per_split = H;
        p->k1_done2 = ws_chunk_counters(p->hdr, 1);
        p->out_ready = ws_chunk_counters(p->hdr, 2);
    }
    p->k1 = GemmParams{};
    p->k1.A = x; p->k1.B = Wx; p->k1.C = ifgo; p->k1.bias0 = bx; p->k1.bias1 = bh;
    p->k1.M = M; p->k1.N = N; p->k1.K = I;
    p->k1.lda = I; p->k1.ldb = I; p->k1.ldc = N;
    p->k1.splits = 1; p->k1.k_per_split = I;
    p->k1_tiles_m = tiles_m; p->k1_tiles_n = tiles_n;
    p->k1_chunk_tiles = ct; p->k1_chunk_steps = steps;
    p->k1_done = ws_chunk_counters(p->hdr, 0);
    return true;
}

// Returns 1 when the XCD-local kernel does not apply, else a fastlstm_status.  With x != nullptr
// the kernel also has to compute ifgo = x.Wx^T + b (returns 2 when that is not possible in-kernel).
int try_fwd_xcd(void *ifgo, void *out, void *cell, const void *Wh, unsigned char *wsb, size_t ws_bytes, int T, int B,
                int H, int dtype, hipStream_t stream, const void *x = nullptr, const void *Wx = nullptr,
                const void *bx = nullptr, const void *bh = nullptr, int I = 0, const SecondLayer *second = nullptr,
                bool dry_run = false, const LaunchOpts &o = LaunchOpts()) {
    XcdCfg c;
    const int copies = (second && !x) ? 2 + o.n_more : 1;   // independent recurrences side by side
    if (!select_xcd(T, B, H, dtype, false, ws_bytes, &c, o.rows, copies)) return copies > 1 ? 2 : 1;
    if (second && ws_bytes < kWsHeaderBytes + kWsCounterBytes + 2 * 2 * c.xslot) return 2;   // both layers' slots side by side
    FwdXcdParams p{};
    p.ifgo = ifgo; p.out = out; p.cell = cell; p.Wh = Wh;
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.counters = reinterpret_cast<int *>(wsb + kWsHeaderBytes);
    p.xbuf = wsb + kWsHeaderBytes + kWsCounterBytes;
    p.T = T; p.B = B; p.H = H;
    p.n_ht = c.n_ht; p.gpx = c.gpx; p.n_groups = c.n_groups; p.KS = c.ks;
    p.b_base = o.row0;
    p.spin_limit = spin_limit_ticks();
    p.keep = o.keep;
    p.trace = g_rec_trace;
    p.n_layers = 1;
    if (second && !x) {   // independent recurrences of this shape side by side (their projections are done)
        const int n = 2 + o.n_more;
        if (n > kMaxSideBySide || n * c.n_groups > kNumXcd * c.gpx) return 2;   // every group needs its CUs on one XCD
        if (ws_bytes < kWsHeaderBytes + kWsCounterBytes + 2 * (size_t)n * c.xslot) return 2;
        p.n_layers = n;
        p.ifgo2 = second->ifgo; p.out2 = second->out; p.cell2 = second->cell; p.Wh2 = second->Wh;
        for (int i = 0; i < o.n_more; ++i) {
            p.ifgo_more[i] = o.more[i][0]; p.out_more[i] = o.more[i][1]; p.cell_more[i] = o.more[i][2]; p.Wh_more[i] = o.more[i][3];
        }
    }
    if (x) {
        if (!plan_k1_helpers(c, x, Wx, bx, bh, ifgo, T, B, I, H, dtype, &p, second)) return 2;
        const int lds = std::max(c.lds, Gemm16Cfg<256, 256, 2, 2, 4, 2>::LDS_BYTES);
        FwdXcdHelpLauncher hl = dtype == FASTLSTM_FP16 ? launch_fwd_xcd_help_f16 : launch_fwd_xcd_help_bf16;
        int occ = 0;
        if (hl(p, c.ntw, 0, lds, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
        if (occ < 1) return 2;
        if (dry_run) return FASTLSTM_OK;
        if (hl(p, c.ntw, kNumXcd * 32, lds, stream, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
        return FASTLSTM_OK;
    }
    FwdXcdLauncher launch = dtype == FASTLSTM_FP32 ? launch_fwd_xcd_f32
                                                   : (dtype == FASTLSTM_FP16 ? launch_fwd_xcd_f16 : launch_fwd_xcd_bf16);
    int occ = 0;
    if (launch(p, c.mt, c.nkw, c.ntw, c.nwv, 0, c.lds, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
    if (occ < 1) return 1;
    if (dry_run) return FASTLSTM_OK;
    // one workgroup per CU of the device; those without a role return at once
    if (launch(p, c.mt, c.nkw, c.ntw, c.nwv, kNumXcd * 32, c.lds, stream, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
    return FASTLSTM_OK;
}

// Clears the part of a workspace that a recurrent call needs zeroed (a kernel, not hipMemsetAsync:
// callers may capture the stream into a graph).
__global__ void zero_words_kernel(unsigned *p, size_t n) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}

// One launch that gets a forward call ready: clears `zero_words` words of the workspace and writes the initial
// state (h0, c0, or zeros when they are null) into slot 0 of out and cell, n elements of `esz` bytes each.
__global__ void prepare_forward_kernel(unsigned *ws, size_t zero_words, unsigned char *out0, unsigned char *cell0,
                                       const unsigned char *h0, const unsigned char *c0, size_t n, int esz) {
    const size_t first = blockIdx.x * (size_t)blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = first; i < zero_words; i += stride) ws[i] = 0u;
    if (esz == 2) {
        unsigned short *o = reinterpret_cast<unsigned short *>(out0), *c = reinterpret_cast<unsigned short *>(cell0);
        const unsigned short *h = reinterpret_cast<const unsigned short *>(h0), *cc = reinterpret_cast<const unsigned short *>(c0);
        for (size_t i = first; i < n; i += stride) {
            o[i] = h ? h[i] : (unsigned short)0;
            c[i] = cc ? cc[i] : (unsigned short)0;
        }
    } else {
        unsigned *o = reinterpret_cast<unsigned *>(out0), *c = reinterpret_cast<unsigned *>(cell0);
        const unsigned *h = reinterpret_cast<const unsigned *>(h0), *cc = reinterpret_cast<const unsigned *>(c0);
        for (size_t i = first; i < n; i += stride) {
            o[i] = h ? h[i] : 0u;
            c[i] = cc ? cc[i] : 0u;
        }
    }
}

// A batch with more tiles than one XCD-local launch holds, even with 32-row tiles: rows per launch such that
// full launches use every XCD (with 32-row tiles where they fit: twice the rows of a launch for 1.1 ... 1.65
// times its step; T = 256, B = 1024, H = 512 fp16 forward 4.4 -> 2.6 ms) and the remainder fits too, or 0.
// The launches run one after the other on the stream and share the workspace.
static int xcd_rows_per_launch(int T, int B, int H, int dtype, bool backward, size_t ws_bytes) {
    const int candidates[4] = {512, 256, 128, 64};
    for (int rows : candidates) {
        if (rows >= B) continue;
        XcdCfg c;
        if (!select_xcd(T, B, H, dtype, backward, ws_bytes, &c, rows) || c.n_groups != kNumXcd * c.gpx) continue;
        if (B % rows && !select_xcd(T, B, H, dtype, backward, ws_bytes, &c, B % rows)) continue;
        return rows;
    }
    return 0;
}
// Between two launches that share a workspace: the barrier counters of the XCD-local kernels start from
// zero in every launch, and so does the XCD rotation its workgroups agree on (check_xcd_placement).
__global__ void reset_xcd_state_kernel(WsHeader *hdr, unsigned *counters, size_t n) {
    if (blockIdx.x == 0 && threadIdx.x == 0) hdr->xcd_rotation = 0;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) counters[i] = 0u;
}
static bool clear_xcd_counters(unsigned char *wsb, hipStream_t s) {
    reset_xcd_state_kernel<<<64, 256, 0, s>>>(reinterpret_cast<WsHeader *>(wsb),
                                              reinterpret_cast<unsigned *>(wsb + kWsHeaderBytes), kWsCounterBytes / 4);
    return hipGetLastError() == hipSuccess;
}

// Shape of a launch of the register-resident kernels whose barrier groups span several XCDs
// (recurrent_fwd_wide.hpp): 16 units x 16 nt batch rows per workgroup, H / 16 workgroups per group.
struct WideCfg {
    int nkw, n_ht, xpg, n_groups, ks, lds;
    int nt;   // batch tiles of 16 rows per group: the smallest of 1, 2, 4 with which the launch holds the batch
    int v;    // reverse kernel, 64-row groups: members of a team that splits K (lstm_bwd_wide_split_kernel); 0 = no teams
    size_t xslot;
};
// copies > 1: that many recurrences of this shape share the launch (groups of 16 or 32 rows only).
bool select_wide(int T, int B_all, int H, int dtype, bool backward, size_t ws_bytes, WideCfg *c, int rows = 0, int copies = 1) {
    const int B = rows ? rows : B_all;   // rows of this launch
    DeviceInfo di;
    if (!(g_families.load() & 2) || device_info(-1, &di) != FASTLSTM_OK || di.xcd_round_robin != 1 || di.num_cus < kNumXcd * 32)
        return false;
    // a weight row of 2.5 ... 4 KiB in steps of 512 bytes: H = 1280, 1536, 1792, 2048 with 16-bit elements,
    // 640, 768, 896, 1024 with fp32
    const int es = elem_bytes(dtype), kstep = dtype == FASTLSTM_FP32 ? 16 : 32;
    if ((H * es) % 512 || H * es <= 2048 || H * es > 4096) return false;
    c->nkw = (backward ? 4 * H : H) / kstep / 8;
    c->n_ht = H / 16;
    if (c->n_ht > kXcdGroupStride) return false;
    c->xpg = cdiv(c->n_ht, 32);   // XCDs per group (the last one partly used when H is not a multiple of 512)
    // groups of 16 or 32 rows where they all fit the launch: more groups = more CUs for a small batch, and a
    // CU then fetches a quarter or half of the operand bytes per step
    c->nt = copies * cdiv(B, 16) * c->xpg <= kNumXcd ? 1 : copies * cdiv(B, 32) * c->xpg <= kNumXcd ? 2 : 4;
    if (copies > 1 && c->nt == 4) return false;
    // fp32 multiplies at 1/16 of the 16-bit rate: 16 units x 64 rows per CU are more MFMA time than a step of the
    // general kernels, which spread 4 units x all rows over every CU
    if (dtype == FASTLSTM_FP32 && c->nt == 4) return false;
    c->n_groups = cdiv(B, 16 * c->nt);
    if (copies * c->n_groups * c->xpg > kNumXcd) return false;
    // ... and a small fp32 batch leaves most CUs without a share of the forward product (B = 32, H = 1024: 6.0
    // instead of 5.7 us per step; the reverse step, with four times the operand bytes, gains at every size)
    // (a remainder of rows behind full launches still runs here: the general kernel would take the whole batch)
    if (dtype == FASTLSTM_FP32 && !backward && copies * c->n_groups * c->xpg < 6 && B == B_all) return false;
    c->ks = (backward ? 4 * H : H) / kstep;
    c->xslot = (size_t)c->n_groups * c->nt * c->ks * kFragBytes;
    if (ws_bytes < kWsHeaderBytes + kWsCounterBytes + 2 * (size_t)copies * c->xslot) return false;
    const int gr = 16 * c->nt;
    const int gseg = 16 * es;
    const int tiles = gr * (4 * gseg + 16) + 2 * gr * (gseg + 16);   // gates + two state tiles of `gr` rows x 16 units
    c->lds = backward ? 8 * c->nt * kFragBytes + tiles + 8 * kWideRing * kFragBytes : 8 * 4 * c->nt * kFragBytes + tiles;
    c->v = 0;
    if (backward && c->nt == 4 && (g_families.load() & 4)) {
        const int v = 4;   // divides the k-steps per wave (20 ... 32) and the workgroups of an XCD
        const size_t partials = (size_t)c->n_groups * c->n_ht * v * 4 * kFragBytes;
        if (c->n_ht % v == 0 && ws_bytes >= kWsHeaderBytes + kWsCounterBytes + 2 * c->xslot + partials) {
            c->v = v;
            c->lds = 4 * kFragBytes + tiles + 8 * 4 * v * kFragBytes;   // the waves' sums take the place of their rings
        }
    }
    return true;
}

// Rows per launch (see xcd_rows_per_launch) for the register-resident kernels: full launches of 64-row groups
// (fp32: 32-row groups) on all XCDs.
static int wide_rows_per_launch(int T, int B, int H, int dtype, bool backward, size_t ws_bytes) {
    const int xpg = cdiv(H / 16, 32);
    const int rows = (dtype == FASTLSTM_FP32 ? 32 : 64) * (kNumXcd / std::max(1, xpg));
    if (rows >= B || rows <= 0) return 0;
    WideCfg c;
    if (!select_wide(T, B, H, dtype, backward, ws_bytes, &c, rows)) return 0;
    if (B % rows && !select_wide(T, B, H, dtype, backward, ws_bytes, &c, B % rows)) return 0;
    return rows;
}

// Returns 1 when the kernel does not apply, else a fastlstm_status.
// `second` (+ o.more): independent recurrences of the same shape side by side in the launch, as try_fwd_xcd takes them.
int try_fwd_wide(void *ifgo, void *out, void *cell, const void *Wh, unsigned char *wsb, size_t ws_bytes, int T, int B,
                 int H, int dtype, hipStream_t stream, const LaunchOpts &o = LaunchOpts(), const SecondLayer *second = nullptr,
                 bool dry_run = false) {
    WideCfg c;
    const int copies = second ? 2 + o.n_more : 1;
    if (copies > kMaxSideBySide || !select_wide(T, B, H, dtype, false, ws_bytes, &c, o.rows, copies)) return 1;
    FwdXcdParams p{};
    p.n_layers = copies;
    if (second) {
        p.ifgo2 = second->ifgo; p.out2 = second->out; p.cell2 = second->cell; p.Wh2 = second->Wh;
        for (int i = 0; i < o.n_more; ++i) {
            p.ifgo_more[i] = o.more[i][0]; p.out_more[i] = o.more[i][1]; p.cell_more[i] = o.more[i][2]; p.Wh_more[i] = o.more[i][3];
        }
    }
    p.ifgo = ifgo; p.out = out; p.cell = cell; p.Wh = Wh;
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.counters = reinterpret_cast<int *>(wsb + kWsHeaderBytes);   // here: one flag per workgroup
    p.xbuf = wsb + kWsHeaderBytes + kWsCounterBytes;
    p.T = T; p.B = B; p.H = H;
    p.n_ht = c.n_ht; p.gpx = c.xpg; p.n_groups = c.n_groups; p.KS = c.ks;
    p.b_base = o.row0;
    p.spin_limit = spin_limit_ticks();
    p.keep = o.keep;
    auto launch = dtype == FASTLSTM_FP16 ? launch_fwd_wide_f16 : dtype == FASTLSTM_BF16 ? launch_fwd_wide_bf16 : launch_fwd_wide_f32;
    int occ = 0;
    if (launch(p, c.nkw, c.nt, 0, c.lds, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
    if (occ < 1) return 1;
    if (dry_run) return FASTLSTM_OK;
    if (launch(p, c.nkw, c.nt, kNumXcd * 32, c.lds, stream, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
    return FASTLSTM_OK;
}

// `second` (7 operand pointers in the order of this call's own; + o.more): independent recurrences of the same shape
// side by side in the launch.
int try_bwd_wide(const void *dout, void *dh, void *dc, const void *ifgo, const void *cell, void *d_ifgo, const void *Wh,
                 unsigned char *wsb, size_t ws_bytes, int T, int B, int H, int dtype, hipStream_t stream,
                 const LaunchOpts &o = LaunchOpts(), void *const *second = nullptr, bool dry_run = false) {
    WideCfg c;
    const int copies = second ? 2 + o.n_more : 1;
    if (copies > kMaxSideBySide || !select_wide(T, B, H, dtype, true, ws_bytes, &c, o.rows, copies)) return 1;
    if (copies > 1) c.v = 0;   // (never set: the team form is for 64-row groups)
    BwdXcdParams p{};
    p.n_layers = copies;
    if (second) {
        p.k5.C = second[0];   // the kernels read the second recurrence's dout from there
        p.dh_lo = second[1]; p.dc_lo = second[2]; p.ifgo_lo = second[3]; p.cell_lo = second[4];
        p.d_ifgo_lo = second[5]; p.Wh_lo = second[6];
        for (int i = 0; i < o.n_more; ++i) {
            p.dout_more[i] = o.more[i][0]; p.dh_more[i] = o.more[i][1]; p.dc_more[i] = o.more[i][2]; p.ifgo_more[i] = o.more[i][3];
            p.cell_more[i] = o.more[i][4]; p.d_ifgo_more[i] = o.more[i][5]; p.Wh_more[i] = o.more[i][6];
        }
    }
    p.dout = dout; p.dh = dh; p.dc = dc; p.ifgo = ifgo; p.cell = cell; p.d_ifgo = d_ifgo; p.Wh = Wh;
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.counters = reinterpret_cast<int *>(wsb + kWsHeaderBytes);   // here: one flag per workgroup
    p.xbuf = wsb + kWsHeaderBytes + kWsCounterBytes;
    p.T = T; p.B = B; p.H = H;
    p.n_ht = c.n_ht; p.gpx = c.xpg; p.n_groups = c.n_groups; p.KSB = c.ks;
    p.b_base = o.row0;
    p.spin_limit = spin_limit_ticks();
    p.partials = p.xbuf + 2 * c.xslot;
    auto launch = c.v ? (dtype == FASTLSTM_FP16 ? launch_bwd_wide_split_f16 : launch_bwd_wide_split_bf16)
                      : (dtype == FASTLSTM_FP16 ? launch_bwd_wide_f16 : dtype == FASTLSTM_BF16 ? launch_bwd_wide_bf16 : launch_bwd_wide_f32);
    const int form = c.v ? c.v : c.nt;
    int occ = 0;
    if (launch(p, c.nkw, form, 0, c.lds, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
    if (occ < 1) return 1;
    if (dry_run) return FASTLSTM_OK;
    if (launch(p, c.nkw, form, kNumXcd * 32, c.lds, stream, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
    return FASTLSTM_OK;
}

// What the reverse launch may compute besides the recurrence (fastlstm_bwd_layer).
struct BwdExtras {
    const void *Wx, *x, *h;
    void *dx, *dWx, *dWh;
    int I;
    float *db_part = nullptr;   // [ceil(B / 16)][4H] floats: where the launch may leave the bias gradient's partial sums
};

// In-kernel dx (and, where the shapes suit the 16-bit tile kernel, dWx and dWh) by the workgroups
// without a role in the recurrence (see BwdXcdParams).  *wgrad_fused tells whether the weight
// gradients are part of the launch.
// The lower layer of a stack that shares the reverse launch (see BwdXcdParams::n_layers): its state
// gradients, saved activations, d_ifgo, weights; dx may be null (not wanted); I = its input size.
struct LowerLayer {
    void *dh, *dc;
    const void *ifgo, *cell;
    void *d_ifgo;
    const void *Wh, *Wx;
    void *dx;
    int I;
    void *scratch;          // device memory for the parked fp32 weight-gradient tiles (the wgrad workspace)
    size_t scratch_bytes;
    const void *x, *h;      // the lower layer's input and its out (for its weight gradients; may be null)
    void *dWx, *dWh;
    float *db_part = nullptr;   // as BwdExtras::db_part, for the lower layer
    const void *dout = nullptr;   // two independent recurrences side by side (no extras): the second one's dout
};

bool plan_bwd_helpers(const XcdCfg &c, const void *d_ifgo, const BwdExtras &e, int T, int B, int H, int dtype,
                      BwdXcdParams *p, bool *wgrad_fused, const LowerLayer *lower = nullptr,
                      bool *lower_wgrad_fused = nullptr) {
    *wgrad_fused = false;
    if (lower_wgrad_fused) *lower_wgrad_fused = false;
    if (dtype == FASTLSTM_FP32 || !((c.mt == 2 && c.nkw == 16) || (c.mt == 1 && c.nkw == 8))) return false;
    const int layers = lower ? 2 : 1;
    if (layers * c.n_groups > kNumXcd * c.gpx) return false;   // every group needs its CUs on one XCD
    const int n_active = c.n_groups * c.n_ht, n_helpers = kNumXcd * 32 - layers * n_active;
    if (n_helpers < kNumXcd * (lower ? 6 : 8)) return false;
    const int max_chunks = kMaxChunks;
    const int I = e.I, M = T * B, K = 4 * H;
    if (!gemm16_eligible(dtype, M, I, K, K, I, false, true) || I % 8) return false;
    // The helpers have to keep up with the recurrence: with few of them (8 idle CUs per XCD at H = 768) the launch
    // lasts as long as their share of dx, dW_x and dW_h, and launches of their own on the whole device behind the
    // recurrence are faster (T = 256, B = 128, I = H = 768: layer backward 2.3 ms inside, 1.3 ms behind).
    // A weight-gradient tile is one helper's from the first timestep to the last (2 * 256 * 256 * T * B flop), so with
    // fewer tiles than helpers (H = 384: 24 tiles) most helpers have none and the launch lasts as long as one tile.
    // Of {dx and the weight gradients inside, dx inside, nothing inside} the fastest by this estimate is taken.
    bool wgrad_inside = true;
    if (!lower) {
        const double per_cu = 3.5e9, rec_ms = T * (c.ntw == 1 ? 3.0e-3 : 5.4e-3);   // flop per ms and CU inside a launch
        // (e.dx null: the caller wants no dx; e.dWx null: no weight gradients)
        const double dx_flop = e.dx ? 2.0 * M * K * I : 0.0, wg_flop = e.dWx ? 2.0 * M * K * (I + H) : 0.0;
        const int wg_tiles = cdiv(K, 256) * (cdiv(I, 256) + cdiv(H, 256));
        const double tile_ms = cdiv(wg_tiles, n_helpers) * 2.0 * 256 * 256 * M / per_cu;
        const double all_ms = std::max(rec_ms, std::max((dx_flop + wg_flop) / (n_helpers * per_cu), tile_ms));
        const double dx_ms = std::max(rec_ms, dx_flop / (n_helpers * per_cu)) + wg_flop / (256 * per_cu);
        const double none_ms = rec_ms + (dx_flop + wg_flop) / (256 * per_cu);
        if (none_ms < std::min(all_ms, dx_ms)) return false;
        wgrad_inside = all_ms <= dx_ms;
        if ((!wgrad_inside || !e.dWx) && !e.dx) return false;   // nothing left for the helpers
    }
    const int tiles_m = cdiv(M, 256), tiles_n = cdiv(I, 256);
    // a chunk: whole timesteps, two row tiles where that is possible -- what the helpers still have to do when the
    // recurrence ends is their share of the last chunk (T = 512, B = 64, I = H = 1024: layer backward 1.674 ms with
    // chunks of 8 row tiles, 1.628 with 2) -- at most kMaxChunks chunks.  Two stacked layers keep about 8: their
    // helpers serve two recurrences, and with half the chunk the module's forward + backward at T = 2048, B = 32,
    // I = H = 1024 took 12.35 instead of 11.99 ms.
    int base = 1;
    while ((base * 256) % B) ++base;
    const int target = lower ? 8 : 2;
    int ct = base >= target ? base : (target / base) * base;
    if (lower) {
        // the lower layer runs two chunks behind the upper one: no more than 64 timesteps per chunk
        ct = std::min(ct, std::max(1, 64 * B / 256 / base) * base);
        // dx, dW_x and dW_h of both layers on the helpers: see plan_k1_helpers (config E: 1.0).  Where that is too much
        // for them, both dx alone (the upper one is the lower recurrence's operand and has to be inside): the weight
        // gradients then follow as launches of their own on the whole device (T = 512, B = 64, I = 256, H = 768 bf16,
        // two layers: reverse pass 3.6 ms as a wavefront of launches, 2.8 ms this way).
        const double dx_flop = 2.0 * M * K * I + (lower->dx ? 2.0 * M * K * lower->I : 0.0);
        const double flop = dx_flop + 2.0 * M * K * (I + H) + 2.0 * M * K * (lower->I + H);
        const double budget_ms = 1.25 * T * 3.6e-3;
        if (flop / (n_helpers * 3.5e9) > budget_ms) {
            if (dx_flop / (n_helpers * 3.5e9) > budget_ms) return false;
            wgrad_inside = false;
        }
    }
    while (cdiv(tiles_m, ct) > max_chunks) ct += base;
    p->n_layers = layers;
    if (lower) {
        if (e.I != H) return false;   // the upper layer's dx is the lower layer's dout
        p->dh_lo = lower->dh; p->dc_lo = lower->dc; p->ifgo_lo = lower->ifgo; p->cell_lo = lower->cell;
        p->d_ifgo_lo = lower->d_ifgo; p->Wh_lo = lower->Wh;
        p->k5_lo = GemmParams{};
        if (lower->dx) {
            if (!gemm16_eligible(dtype, M, lower->I, K, K, lower->I, false, true) || lower->I % 8) return false;
            p->k5_lo.A = lower->d_ifgo; p->k5_lo.B = lower->Wx; p->k5_lo.C = lower->dx;
            p->k5_lo.M = M; p->k5_lo.N = lower->I; p->k5_lo.K = K;
            p->k5_lo.lda = K; p->k5_lo.ldb = lower->I; p->k5_lo.ldc = lower->I;
            p->k5_lo.splits = 1; p->k5_lo.k_per_split = K;
        }
        p->k5_lo_tiles_n = cdiv(lower->I, 256);
        p->chunk_done_lo = ws_chunk_counters(p->hdr, 1);
        p->dx_done = ws_chunk_counters(p->hdr, 2);
    }
    p->k5 = GemmParams{};
    p->k5.A = d_ifgo; p->k5.B = e.Wx; p->k5.C = e.dx;
    p->k5.M = M; p->k5.N = I; p->k5.K = K;
    p->k5.lda = K; p->k5.ldb = I; p->k5.ldc = I;
    p->k5.splits = 1; p->k5.k_per_split = K;
    p->k5_tiles_m = tiles_m; p->k5_tiles_n = tiles_n;
    p->k5_chunk_tiles = ct; p->k5_chunk_steps = ct * 256 / B; p->k5_chunks = cdiv(tiles_m, ct);
    p->k5_tail_by_rec = (!lower && e.dx) ? 1 : 0;
    p->n_active = n_active;
    p->chunk_done = ws_chunk_counters(p->hdr, 0);
    p->wg_tiles = 0;
    if (wgrad_inside && e.dWx && gemm16_eligible(dtype, K, I, M, K, I, true, true) &&
        gemm16_eligible(dtype, K, H, M, K, H, true, true) && H % 8 == 0) {
        GemmParams g{};
        g.A = d_ifgo; g.M = K; g.K = M; g.lda = K; g.splits = 1; g.k_per_split = M;
        p->k8 = g; p->k8.B = e.x; p->k8.C = e.dWx; p->k8.N = I; p->k8.ldb = I; p->k8.ldc = I;
        p->k9 = g; p->k9.B = e.h; p->k9.C = e.dWh; p->k9.N = H; p->k9.ldb = H; p->k9.ldc = H;
        p->wg_tiles_m = cdiv(K, 256);
        p->k8_tiles_n = cdiv(I, 256); p->k9_tiles_n = cdiv(H, 256);
        p->wg_tiles = p->wg_tiles_m * (p->k8_tiles_n + p->k9_tiles_n);
        *wgrad_fused = true;
        if (lower) {   // the stacked helpers park their accumulators between chunks
            p->wg_scratch = static_cast<float *>(lower->scratch);
            const size_t tile_bytes = (size_t)256 * 256 * sizeof(float);
            const size_t upper_bytes = (size_t)std::min(p->wg_tiles, n_helpers) * tile_bytes;
            if (upper_bytes > lower->scratch_bytes) {
                p->wg_tiles = 0;
                *wgrad_fused = false;
            } else if (lower->dWx && lower->dWh && lower->x && lower->h && lower_wgrad_fused &&
                       gemm16_eligible(dtype, K, lower->I, M, K, lower->I, true, true) && lower->I % 8 == 0) {
                // the lower layer's weight gradients the same way, its tiles parked behind the upper layer's
                GemmParams lo{};
                lo.A = lower->d_ifgo; lo.M = K; lo.K = M; lo.lda = K; lo.splits = 1; lo.k_per_split = M;
                p->k8_lo = lo; p->k8_lo.B = lower->x; p->k8_lo.C = lower->dWx; p->k8_lo.N = lower->I;
                p->k8_lo.ldb = lower->I; p->k8_lo.ldc = lower->I;
                p->k9_lo = lo; p->k9_lo.B = lower->h; p->k9_lo.C = lower->dWh; p->k9_lo.N = H; p->k9_lo.ldb = H; p->k9_lo.ldc = H;
                p->k8_lo_tiles_n = cdiv(lower->I, 256);
                const int lo_tiles = p->wg_tiles_m * (p->k8_lo_tiles_n + p->k9_tiles_n);
                if (upper_bytes + (size_t)std::min(lo_tiles, n_helpers) * tile_bytes <= lower->scratch_bytes) {
                    p->wg_lo_tiles = lo_tiles;
                    p->wg_scratch_lo = p->wg_scratch + upper_bytes / sizeof(float);
                    *lower_wgrad_fused = true;
                }
            }
        }
    }
    // the bias gradient of a layer whose weight gradients are part of the launch: summed by its recurrence workgroups
    p->db_lds_off = (c.lds + 15) / 16 * 16;
    const int ipt = cdiv(16 * c.mt * 16 * c.ntw, kWave * 8);   // (unit, row) items per thread of the reverse kernel
    const bool slots_fit = p->db_lds_off + ipt * kWave * 8 * 16 <= Gemm16Cfg<256, 256, 2, 2, 4, 2>::LDS_BYTES;
    p->db_part = (*wgrad_fused && slots_fit) ? e.db_part : nullptr;
    p->db_part_lo = (lower && lower_wgrad_fused && *lower_wgrad_fused && slots_fit) ? lower->db_part : nullptr;
    return true;
}

// With `extras` the launch also computes dx (returns 2 when that is not possible in-kernel) and, if
// it can, the weight gradients: returns 0 when they were part of the launch, 3 when they are still
// to be computed.
int try_bwd_xcd(const void *dout, void *dh, void *dc, const void *ifgo, const void *cell, void *d_ifgo, const void *Wh,
                unsigned char *wsb, size_t ws_bytes, int T, int B, int H, int dtype, hipStream_t stream,
                const BwdExtras *extras = nullptr, const LowerLayer *lower = nullptr, bool dry_run = false,
                bool *lower_wgrad_fused = nullptr, const LaunchOpts &o = LaunchOpts(), int *db_done = nullptr) {
    // *db_done: bit 0 / bit 1 set when the launch leaves the bias gradient's partial sums of the (upper) layer / the
    // lower layer in extras->db_part / lower->db_part
    if (db_done) *db_done = 0;
    XcdCfg c;
    const int copies = (lower && !extras) ? 2 + o.n_more : 1;   // independent recurrences side by side
    if (!select_xcd(T, B, H, dtype, true, ws_bytes, &c, o.rows, copies)) return copies > 1 ? 2 : 1;
    if (lower && ws_bytes < kWsHeaderBytes + kWsCounterBytes + 2 * 2 * c.xslot) return 2;   // both layers' slots side by side
    BwdXcdParams p{};
    p.dout = dout; p.dh = dh; p.dc = dc; p.ifgo = ifgo; p.cell = cell; p.d_ifgo = d_ifgo; p.Wh = Wh;
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.counters = reinterpret_cast<int *>(wsb + kWsHeaderBytes);
    p.xbuf = wsb + kWsHeaderBytes + kWsCounterBytes;
    p.T = T; p.B = B; p.H = H;
    p.n_ht = c.n_ht; p.gpx = c.gpx; p.n_groups = c.n_groups; p.KSB = c.ks;
    p.b_base = o.row0;
    p.spin_limit = spin_limit_ticks();
    p.n_layers = 1;
    if (lower && !extras) {   // independent recurrences of this shape side by side
        const int n = 2 + o.n_more;
        // (32-row groups of the 16-k-step reverse kernel, H > 512, cost 1.9 x a 16-row step: no gain over one after the other)
        if (n > kMaxSideBySide || n * c.n_groups > kNumXcd * c.gpx || (c.ntw == 2 && c.nkw == 16)) return 2;
        if (ws_bytes < kWsHeaderBytes + kWsCounterBytes + 2 * (size_t)n * c.xslot) return 2;
        p.n_layers = n;
        for (int i = 0; i < o.n_more; ++i) {
            p.dout_more[i] = o.more[i][0]; p.dh_more[i] = o.more[i][1]; p.dc_more[i] = o.more[i][2]; p.ifgo_more[i] = o.more[i][3];
            p.cell_more[i] = o.more[i][4]; p.d_ifgo_more[i] = o.more[i][5]; p.Wh_more[i] = o.more[i][6];
        }
        p.dh_lo = lower->dh; p.dc_lo = lower->dc; p.ifgo_lo = lower->ifgo; p.cell_lo = lower->cell;
        p.d_ifgo_lo = lower->d_ifgo; p.Wh_lo = lower->Wh;
        p.k5.C = const_cast<void *>(lower->dout);   // the kernel reads the second recurrence's dout from there
    }
    if (extras) {
        bool wgrad_fused = false;
        if (!plan_bwd_helpers(c, d_ifgo, *extras, T, B, H, dtype, &p, &wgrad_fused, lower, lower_wgrad_fused)) return 2;
        const int lds = std::max(c.lds, Gemm16Cfg<256, 256, 2, 2, 4, 2>::LDS_BYTES);
        BwdXcdLauncher hl = dtype == FASTLSTM_FP16 ? launch_bwd_xcd_help_f16 : launch_bwd_xcd_help_bf16;
        int occ = 0;
        if (hl(p, c.mt, c.nkw, c.ntw, 0, lds, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
        if (occ < 1) return 2;
        if (dry_run) return wgrad_fused ? FASTLSTM_OK : 3;
        if (hl(p, c.mt, c.nkw, c.ntw, kNumXcd * 32, lds, stream, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
        if (db_done) *db_done = (p.db_part ? 1 : 0) | (p.db_part_lo ? 2 : 0);
        return wgrad_fused ? FASTLSTM_OK : 3;
    }
    BwdXcdLauncher launch = dtype == FASTLSTM_FP32 ? launch_bwd_xcd_f32
                                                   : (dtype == FASTLSTM_FP16 ? launch_bwd_xcd_f16 : launch_bwd_xcd_bf16);
    int occ = 0;
    if (launch(p, c.mt, c.nkw, c.ntw, 0, c.lds, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
    if (occ < 1) return 1;
    if (dry_run) return FASTLSTM_OK;
    if (launch(p, c.mt, c.nkw, c.ntw, kNumXcd * 32, c.lds, stream, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
    return FASTLSTM_OK;
}

}  // namespace
}  // namespace fastlstm

extern "C" {

static int plan_device(int device, int B, int H, int dtype, int backward, fastlstm_plan *plan, bool may_probe) {
    if (!plan) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (B <= 0 || H <= 0) return FASTLSTM_ERR_DIM;
    DeviceInfo di;
    int rc = device_info(device, &di);
    if (rc) return rc;
    if (may_probe && di.xcd_round_robin < 0) probe_device(device);
    return fastlstm_plan_for(di.num_cus, di.lds, B, H, dtype, backward, plan);
}

int fastlstm_plan_device(int device, int B, int H, int dtype, int backward, fastlstm_plan *plan) {
    return plan_device(device, B, H, dtype, backward, plan, true);
}

// The input projection's output is read back by the time loop that follows it.  Up to half the memory-side cache
// (256 MiB on this device) it is written with ordinary stores so that the loop, whose step waits for its gate tile,
// finds it there; a larger one streams out past the caches (GemmParams::keep_c).
static int gates_stay_cached(size_t rows, int H, int dtype) {
    return rows * 4 * (size_t)H * elem_bytes(dtype) <= ((size_t)128 << 20) ? 1 : 0;
}

// K1 on rows [row0, row0 + rows) of x[T*B, I] / ifgo[T*B, 4H]
static int gemm_ifgo_rows(const void *x, const void *Wx, const void *bx, const void *bh, void *ifgo, size_t row0,
                          int rows, int I, int H, int dtype, hipStream_t stream) {
    const size_t s = elem_bytes(dtype);
    // a narrow layer whose I the tile kernel does not take (no whole k-tile of 64): the streaming form of gemm_small.hpp
    // (T*B = 262144, I = H = 32: 0.062 ms on the generic kernel, 0.021 here; at I = 64 the tile kernel is the faster one)
    if (!gemm_baseline() && I % 64 != 0 && small_bwd_eligible(dtype, rows, I, H))
        return launch_small_k1(dtype, static_cast<const unsigned char *>(x) + row0 * I * s, Wx, bx, bh,
                               static_cast<unsigned char *>(ifgo) + row0 * 4 * H * s, rows, I, H, stream) == hipSuccess
                   ? FASTLSTM_OK
                   : FASTLSTM_ERR_HIP;
    GemmParams p{};
    p.A = static_cast<const unsigned char *>(x) + row0 * I * s;
    p.B = Wx;
    p.C = static_cast<unsigned char *>(ifgo) + row0 * 4 * H * s;
    p.bias0 = bx; p.bias1 = bh;
    p.M = rows; p.N = 4 * H; p.K = I;
    p.lda = I; p.ldb = I; p.ldc = 4 * H;
    p.splits = 1; p.k_per_split = I;
    p.keep_c = gates_stay_cached(rows, H, dtype);
    int tile, splits;
    gemm_plan(dtype, p.M, p.N, p.K, p.lda, p.ldb, false, false, false, &tile, &splits);
    return launch_gemm_tiled(dtype, p, false, false, tile, stream) == hipSuccess ? FASTLSTM_OK : FASTLSTM_ERR_HIP;
}

int fastlstm_gemm_ifgo(const void *x, const void *Wx, const void *bx, const void *bh, void *ifgo, int T,
                       int B, int I, int H, int dtype, void *stream) {
    if (!x || !Wx || !bx || !bh || !ifgo) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(x) || !aligned16(Wx) || !aligned16(ifgo)) return FASTLSTM_ERR_ALIGN;
    if (!gemm_baseline() && I % 64 != 0 && small_bwd_eligible(dtype, T * B, I, H))   // (see gemm_ifgo_rows)
        return launch_small_k1(dtype, x, Wx, bx, bh, ifgo, T * B, I, H, static_cast<hipStream_t>(stream)) == hipSuccess
                   ? FASTLSTM_OK
                   : FASTLSTM_ERR_HIP;
    GemmParams p{};
    p.A = x; p.B = Wx; p.C = ifgo; p.bias0 = bx; p.bias1 = bh;
    p.M = T * B; p.N = 4 * H; p.K = I;
    p.lda = I; p.ldb = I; p.ldc = 4 * H;
    p.splits = 1; p.k_per_split = I;
    p.keep_c = gates_stay_cached(T * B, H, dtype);
    int tile, splits;
    gemm_plan(dtype, p.M, p.N, p.K, p.lda, p.ldb, false, false, false, &tile, &splits);
    return launch_gemm_tiled(dtype, p, false, false, tile, static_cast<hipStream_t>(stream)) == hipSuccess
               ? FASTLSTM_OK
               : FASTLSTM_ERR_HIP;
}

// dx = d_ifgo . Wx.  With a scratch buffer (fp32 partial sums) a product with few output tiles is
// split along K so that it fills the device; without one it is a single pass.
static int gemm_dx_impl(const void *d_ifgo, const void *Wx, void *dx, int T, int B, int I, int H, int dtype,
                        void *scratch, size_t scratch_bytes, void *stream) {
    // a narrow layer: the streaming pass of gemm_small.hpp with dx alone (T*B = 262144, I = H = 64: 0.057 -> 0.03 ms)
    if (!gemm_baseline() && small_bwd_eligible(dtype, T * B, I, H))
        return launch_small_bwd(dtype, d_ifgo, Wx, nullptr, nullptr, dx, nullptr, nullptr, nullptr, nullptr, T * B, I, H,
                                static_cast<hipStream_t>(stream)) == hipSuccess
                   ? FASTLSTM_OK
                   : FASTLSTM_ERR_HIP;
    GemmParams p{};
    p.A = d_ifgo; p.B = Wx; p.C = dx;
    p.M = T * B; p.N = I; p.K = 4 * H;
    p.lda = 4 * H; p.ldb = I; p.ldc = I;
    p.splits = 1; p.k_per_split = 4 * H;
    int tile, splits;
    gemm_plan(dtype, p.M, p.N, p.K, p.lda, p.ldb, false, true, scratch != nullptr, &tile, &splits);
    if (splits > 1) {
        const int bk = tile ? 64 : gemm_bk(dtype);
        const int kps = cdiv(cdiv(p.K, splits), bk) * bk;
        splits = cdiv(p.K, kps);
        if (splits > 1 && (size_t)splits * p.M * p.N * sizeof(float) <= scratch_bytes) {
            p.splits = splits; p.k_per_split = kps; p.Cpart = static_cast<float *>(scratch);
        }
    }
    return launch_gemm_tiled(dtype, p, false, true, tile, static_cast<hipStream_t>(stream)) == hipSuccess
               ? FASTLSTM_OK
               : FASTLSTM_ERR_HIP;
}

int fastlstm_gemm_dx(const void *d_ifgo, const void *Wx, void *dx, int T, int B, int I, int H, int dtype,
                     void *stream) {
    if (!d_ifgo || !Wx || !dx) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(d_ifgo) || !aligned16(Wx) || !aligned16(dx)) return FASTLSTM_ERR_ALIGN;
    return gemm_dx_impl(d_ifgo, Wx, dx, T, B, I, H, dtype, nullptr, 0, stream);
}

int fastlstm_gemm_dx_split(const void *d_ifgo, const void *Wx, void *dx, int T, int B, int I, int H, int dtype,
                           void *scratch, size_t scratch_bytes, void *stream) {
    if (!d_ifgo || !Wx || !dx) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(d_ifgo) || !aligned16(Wx) || !aligned16(dx) || !aligned16(scratch)) return FASTLSTM_ERR_ALIGN;
    return gemm_dx_impl(d_ifgo, Wx, dx, T, B, I, H, dtype, scratch_bytes ? scratch : nullptr, scratch_bytes, stream);
}

// tile and split-K factor of a weight-gradient product C[M,N] = A^T.B with reduction length K
static void wgrad_plan(int M, int N, int K, int dtype, int *tile, int *splits, int *k_per_split) {
    gemm_plan(dtype, M, N, K, M, N, true, true, true, tile, splits);
    const int bk = *tile ? 64 : gemm_bk(dtype);
    *k_per_split = cdiv(cdiv(K, *splits), bk) * bk;
    *splits = cdiv(K, *k_per_split);
}
static int colsum_chunks(int R) { return std::max(1, std::min(256, R / 64)); }

size_t fastlstm_wgrad_workspace_bytes(int T, int B, int I, int H, int dtype) {
    if (!dtype_ok(dtype) || check_dims(T, B, I, H)) return 0;
    const int K = T * B, M = 4 * H;
    int tile, sx, sh, kps;
    wgrad_plan(M, I, K, dtype, &tile, &sx, &kps);
    wgrad_plan(M, H, K, dtype, &tile, &sh, &kps);
    size_t part = std::max(sx > 1 ? (size_t)sx * M * I : 0, sh > 1 ? (size_t)sh * M * H : 0) * sizeof(float);
    size_t cs = (size_t)colsum_chunks(K) * M * sizeof(float);
    const size_t small = small_bwd_eligible(dtype, K, I, H) ? small_bwd_workspace(K, I, H) : 0;
    return std::max(std::max(align_up(cs, 256) + align_up(part, 256), wgrad_merged_workspace(dtype, M, I, H, K)), small) + 256;
}

int fastlstm_gemm_wgrad(const void *d_ifgo, const void *x, const void *h, void *dWx, void *dWh, void *db,
                        void *ws, size_t ws_bytes, int T, int B, int I, int H, int dtype, void *stream) {
    if (!d_ifgo || !x || !h || !dWx || !dWh || !db || !ws) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(d_ifgo) || !aligned16(x) || !aligned16(h) || !aligned16(dWx) || !aligned16(dWh) ||
        !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    if (ws_bytes < fastlstm_wgrad_workspace_bytes(T, B, I, H, dtype)) return FASTLSTM_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int K = T * B, M = 4 * H;
    if (!gemm_baseline() && small_bwd_eligible(dtype, K, I, H))   // narrow layer: one streaming pass (gemm_small.hpp)
        return launch_small_bwd(dtype, d_ifgo, nullptr, x, h, nullptr, dWx, dWh, db, ws, K, I, H, s) == hipSuccess ? FASTLSTM_OK
                                                                                                                  : FASTLSTM_ERR_HIP;
    {   // both products and the bias gradient as one tile grid, d_ifgo read once
        int sp, kps;
        bool merged;
        if (!gemm_baseline() && wgrad_merged_plan(dtype, M, I, H, K, &sp, &kps, &merged))
            return launch_wgrad_merged(dtype, d_ifgo, x, h, dWx, dWh, db, ws, M, I, H, K, s) == hipSuccess ? FASTLSTM_OK
                                                                                                            : FASTLSTM_ERR_HIP;
    }
    const int chunks = colsum_chunks(K);
    float *cs_part = static_cast<float *>(ws);
    float *gemm_part = reinterpret_cast<float *>(static_cast<unsigned char *>(ws) +
                                                 align_up((size_t)chunks * M * sizeof(float), 256));
    if (launch_colsum(dtype, d_ifgo, db, cs_part, K, M, chunks, s) != hipSuccess) return FASTLSTM_ERR_HIP;
    for (int which = 0; which < 2; ++which) {
        const int N = which == 0 ? I : H;
        GemmParams p{};
        p.A = d_ifgo; p.B = which == 0 ? x : h; p.C = which == 0 ? dWx : dWh;
        p.Cpart = gemm_part;
        p.M = M; p.N = N; p.K = K;
        p.lda = M; p.ldb = N; p.ldc = N;
        int tile;
        wgrad_plan(M, N, K, dtype, &tile, &p.splits, &p.k_per_split);
        if (launch_gemm_tiled(dtype, p, true, true, tile, s) != hipSuccess) return FASTLSTM_ERR_HIP;
    }
    return FASTLSTM_OK;
}

// K5, K8, K9 and the bias gradient behind a reverse recurrence: one pass over d_ifgo for a narrow 16-bit layer
// (gemm_small.hpp), else the two stages one after the other.  dx may be null, and so may dWx, dWh, db (all three).
static int gemm_dx_wgrad_impl(const void *d_ifgo, const void *Wx, const void *x, const void *h, void *dx, void *dWx,
                              void *dWh, void *db, void *ws, size_t ws_bytes, int T, int B, int I, int H, int dtype,
                              void *stream) {
    const bool want_w = dWx != nullptr;
    if (!dx && !want_w) return FASTLSTM_OK;
    if (small_bwd_eligible(dtype, T * B, I, H) && (!want_w || ws_bytes >= small_bwd_workspace(T * B, I, H)))
        return launch_small_bwd(dtype, d_ifgo, Wx, x, h, dx, dWx, dWh, db, ws, T * B, I, H, static_cast<hipStream_t>(stream)) ==
                       hipSuccess
                   ? FASTLSTM_OK
                   : FASTLSTM_ERR_HIP;
    // (the weight-gradient workspace is free until the weight gradients start: scratch for a split along K)
    if (dx)
        if (int rc = gemm_dx_impl(d_ifgo, Wx, dx, T, B, I, H, dtype, ws, ws_bytes, stream)) return rc;
    if (!want_w) return FASTLSTM_OK;
    return fastlstm_gemm_wgrad(d_ifgo, x, h, dWx, dWh, db, ws, ws_bytes, T, B, I, H, dtype, stream);
}

int fastlstm_gemm_dx_wgrad(const void *d_ifgo, const void *Wx, const void *x, const void *h, void *dx, void *dWx, void *dWh,
                           void *db, void *ws, size_t ws_bytes, int T, int B, int I, int H, int dtype, void *stream) {
    const bool want_w = dWx || dWh || db;
    if (!d_ifgo || !Wx || !x || !h || !ws || (want_w && (!dWx || !dWh || !db))) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(d_ifgo) || !aligned16(Wx) || !aligned16(x) || !aligned16(h) || !aligned16(dx) || !aligned16(dWx) ||
        !aligned16(dWh) || !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    if (ws_bytes < fastlstm_wgrad_workspace_bytes(T, B, I, H, dtype)) return FASTLSTM_ERR_WORKSPACE;
    return gemm_dx_wgrad_impl(d_ifgo, Wx, x, h, dx, dWx, dWh, db, ws, ws_bytes, T, B, I, H, dtype, stream);
}

// The one-tile kernels of 64 hidden units (no exchange between workgroups) are bound by the vector ALU of their CU:
// a step of 16 rows x 64 units is 1024 cells of 10 exp / rcp at a quarter of the rate and ~35 other instructions
// each, on one CU, while the others idle.  Rows per workgroup 16 -> 8 -> 4 spreads the cells over 2 x / 4 x the CUs
// (the MFMAs still produce 16 columns; the lanes of the columns that do not exist take over cells of the lane's other
// row tiles, so a lane computes one cell per step, not two or four).  T = 1024, B = 256, I = H = 64, fp16, forward /
// reverse us per step: 16 rows 0.556 / 0.82, 8 rows 0.401 / 0.593, 4 rows 0.339 / 0.458.
// Returns the factor (0: 16 rows, 2, 4) for `n_rec` recurrences of B rows side by side in one launch.
static int one_tile_row_split(int B, int n_rec, int num_cus) {
    if ((long long)n_rec * cdiv(B, 4) <= num_cus) return 4;
    if ((long long)n_rec * cdiv(B, 8) <= num_cus) return 2;
    return 0;
}

// coalesced tile I/O of the general kernels needs complete, 16-byte aligned row segments and room in LDS
static bool fwd_tile_io(const fastlstm_plan &pl, int H, int dtype, int *tile_bytes) {
    const int s = elem_bytes(dtype), gseg = pl.ht * s;
    *tile_bytes = (pl.bt * (4 * gseg + 16) + 2 * pl.bt * (gseg + 16)) * (pl.wave_split != 2 ? 1 : 2);
    return gseg >= 16 && (H * s) % 16 == 0 && H % pl.ht == 0 && pl.lds_bytes + *tile_bytes <= pl.lds_limit;
}

// keep: see LaunchOpts
// others / n_others: further independent recurrences of this shape (operands in the order ifgo, out, cell, Wh) that
// share every launch -- only where the plan is the one-tile form (wave_split 2: no exchange between workgroups).
static int fwd_persistent_impl(void *ifgo, void *out, void *cell, const void *Wh, void *ws, size_t ws_bytes, int T, int B,
                               int H, int dtype, void *stream, int keep, void *const (*others)[7] = nullptr,
                               int n_others = 0) {
    if (!ifgo || !out || !cell || !Wh || !ws) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    if (!aligned16(ifgo) || !aligned16(out) || !aligned16(cell) || !aligned16(Wh) || !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, 0, &pl, false)) return rc;
    if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
    const bool sync = pl.wave_split != 2;
    if (n_others && (sync || n_others > 3)) return FASTLSTM_ERR_DIM;
    // 64 units per workgroup: batch tiles of 4 or 8 rows where that many workgroups still find a CU each
    int tile_bytes = 0;
    const bool tile_io = fwd_tile_io(pl, H, dtype, &tile_bytes);
    const int rs = (!sync && tile_io && pl.ht == 64 && pl.bt == 16) ? one_tile_row_split(B, 1 + n_others, pl.num_cus) : 0;
    const int kstep = dtype == FASTLSTM_FP32 ? 16 : 32;
    unsigned char *wsb = static_cast<unsigned char *>(ws);
    if (pl.wave_split == 3) {   // W_h does not fit on chip: pack it once, then stream it every step
        const StreamLayout l = stream_layout(pl, H, dtype, false);
        hipStream_t s = static_cast<hipStream_t>(stream);
        if (launch_pack_wh(dtype, false, Wh, wsb + l.wpack_off, H, l.KS, l.KSP, l.mt, pl.n_htiles, s) != hipSuccess)
            return FASTLSTM_ERR_HIP;
        FwdStreamParams p{};
        p.ifgo = ifgo; p.out = out; p.cell = cell;
        p.wpack = wsb + l.wpack_off;
        p.hdr = reinterpret_cast<WsHeader *>(wsb);
        p.T = T; p.B = B; p.H = H;
        p.n_bt = pl.n_btiles; p.n_ht = pl.n_htiles;
        p.flag_stride = (int)align_up((size_t)pl.n_htiles, 64);
        p.KS = l.KS; p.KSP = l.KSP;
        p.keep = keep;
        p.spin_limit = spin_limit_ticks();
        const int n_bt_total = cdiv(B, pl.bt);
        for (int c = 0, bt0 = 0; bt0 < n_bt_total; ++c, bt0 += pl.n_btiles) {
            const int n_bt = std::min(pl.n_btiles, n_bt_total - bt0);
            unsigned char *chunk = wsb + kWsHeaderBytes + kWsCounterBytes + (size_t)c * l.chunk_bytes;
            p.flags = reinterpret_cast<int *>(chunk);
            p.xbuf = chunk + l.flags_bytes;
            p.b_base = bt0 * pl.bt;
            const int grid = n_bt * pl.n_htiles;
            int occ = 0;
            if (launch_fwd_stream(dtype, p, l.mt, pl.bt / 16, 0, pl.lds_bytes, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
            if ((long long)occ * pl.num_cus < grid) return FASTLSTM_ERR_RESIDENCY;
            if (launch_fwd_stream(dtype, p, l.mt, pl.bt / 16, grid, pl.lds_bytes, s, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
        }
        return FASTLSTM_OK;
    }
    if (sync) {
        // One launch per range of rows where the batch has too many 16-row tiles for one XCD-local launch;
        // also instead of one launch with 32-row tiles of the 8-wave kernel (H = 1024, 16-bit), whose
        // 32-row step costs 2.5 x its 16-row step (the 4-wave kernels of smaller H are faster in one
        // launch with 32-row tiles).
        const LaunchOpts whole_batch{keep, 0, 0};
        auto by_row_ranges = [&](int rows) {
            for (int r0 = 0; r0 < B; r0 += rows) {
                if (r0 && !clear_xcd_counters(wsb, static_cast<hipStream_t>(stream))) return (int)FASTLSTM_ERR_HIP;
                const LaunchOpts o{keep, r0, std::min(rows, B - r0)};
                const int r = try_fwd_xcd(ifgo, out, cell, Wh, wsb, ws_bytes, T, B, H, dtype, static_cast<hipStream_t>(stream),
                                          nullptr, nullptr, nullptr, nullptr, 0, nullptr, false, o);
                if (r != FASTLSTM_OK) return r < 0 ? r : (int)FASTLSTM_ERR_RESIDENCY;
            }
            return (int)FASTLSTM_OK;
        };
        int rc = try_fwd_xcd(ifgo, out, cell, Wh, wsb, ws_bytes, T, B, H, dtype, static_cast<hipStream_t>(stream), nullptr,
                             nullptr, nullptr, nullptr, 0, nullptr, false, whole_batch);
        if (rc == 1)
            rc = try_fwd_wide(ifgo, out, cell, Wh, wsb, ws_bytes, T, B, H, dtype, static_cast<hipStream_t>(stream), whole_batch);
        if (rc == 1)
            if (const int rows = xcd_rows_per_launch(T, B, H, dtype, false, ws_bytes)) return by_row_ranges(rows);
        if (rc == 1)
            if (const int rows = wide_rows_per_launch(T, B, H, dtype, false, ws_bytes)) {
                for (int r0 = 0; r0 < B; r0 += rows) {
                    if (r0 && !clear_xcd_counters(wsb, static_cast<hipStream_t>(stream))) return FASTLSTM_ERR_HIP;
                    const LaunchOpts o{keep, r0, std::min(rows, B - r0)};
                    const int r = try_fwd_wide(ifgo, out, cell, Wh, wsb, ws_bytes, T, B, H, dtype, static_cast<hipStream_t>(stream), o);
                    if (r != FASTLSTM_OK) return r < 0 ? r : FASTLSTM_ERR_RESIDENCY;
                }
                return FASTLSTM_OK;
            }
        if (rc != 1) return rc;   // launched (0) or failed (< 0); 1: not applicable, use the general kernels
    }
    FwdParams p{};
    p.ifgo = ifgo; p.out = out; p.cell = cell; p.Wh = Wh;
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.T = T; p.B = B; p.H = H;
    p.n_ht = pl.n_htiles;
    p.flag_stride = (int)align_up((size_t)pl.n_htiles, 64);
    p.KS = cdiv(H, kstep);
    p.spin_limit = spin_limit_ticks();
    p.keep = keep;
    p.trace = g_rec_trace;
    p.n_rec = 1 + n_others;
    for (int i = 0; i < n_others; ++i) {
        p.ifgo_x[i] = others[i][0]; p.out_x[i] = others[i][1]; p.cell_x[i] = others[i][2]; p.Wh_x[i] = others[i][3];
    }
    const size_t flags_bytes = recurrent_flags_bytes(pl.n_btiles, pl.n_htiles);
    const size_t slot_bytes = recurrent_slot_bytes(H, dtype, pl.bt, pl.n_btiles, false);
    int lds_bytes = pl.lds_bytes;
    {
        p.vec_io = tile_io ? 1 : 0;
        if (p.vec_io) lds_bytes += tile_bytes;
#ifdef FASTLSTM_TIMELINE
        lds_bytes += 4096;   // room for the diagnostic time stamps of the kernel
#endif
    }
    int bt = pl.bt, n_btiles = pl.n_btiles;
    if (rs) {
        p.rs = rs;
        bt = 16 / rs;
        n_btiles = cdiv(B, bt);
    }
    const int n_bt_total = cdiv(B, bt);
    // K-split kernels keep the slice in registers when a wave's share is at most 32 fragments
    if (pl.wave_split == 0) {
        const int nkw = cdiv(p.KS, 4) <= 4 ? 4 : (cdiv(p.KS, 4) <= 8 ? 8 : 0);
        if (nkw && (pl.ht / 4) * nkw <= 32) p.w_regs = nkw;
    }
    FwdLauncher launch = fwd_launcher(dtype);
    for (int c = 0, bt0 = 0; bt0 < n_bt_total; ++c, bt0 += n_btiles) {
        const int n_bt = std::min(n_btiles, n_bt_total - bt0);
        p.flags = reinterpret_cast<int *>(wsb + kWsHeaderBytes + kWsCounterBytes + (size_t)c * flags_bytes);
        p.xbuf = wsb + pl.ws_zero_bytes + (size_t)c * 2 * slot_bytes;
        p.n_bt = pl.n_btiles;  // exchange-slot stride is sized for a full launch
        p.b_base = bt0 * bt;
        p.n_bt_launch = n_bt;
        const int grid = p.n_rec * n_bt * pl.n_htiles;
        int occ = 0;
        if (launch(p, pl.ht, pl.bt, pl.wave_split, 0, lds_bytes, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
        if (sync && (long long)occ * pl.num_cus < grid) return FASTLSTM_ERR_RESIDENCY;
        if (launch(p, pl.ht, pl.bt, pl.wave_split, grid, lds_bytes, static_cast<hipStream_t>(stream), nullptr) !=
            hipSuccess)
            return FASTLSTM_ERR_HIP;
    }
    return FASTLSTM_OK;
}

int fastlstm_fwd_persistent(void *ifgo, void *out, void *cell, const void *Wh, void *ws, size_t ws_bytes, int T, int B,
                            int H, int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    return finish_recurrent(fwd_persistent_impl(ifgo, out, cell, Wh, ws, ws_bytes, T, B, H, dtype, stream, 1), ws, stream,
                            poison_fwd(dtype, T, B, H, out, cell));
}

// others / n_others: see fwd_persistent_impl (operands in the order of this call's own seven).
static int bwd_persistent_impl(const void *dout, void *dh, void *dc, const void *ifgo, const void *cell,
                               void *d_ifgo, const void *Wh, void *ws, size_t ws_bytes, int T, int B, int H,
                               int dtype, void *stream, void *const (*others)[7] = nullptr, int n_others = 0) {
    if (!dout || !dh || !dc || !ifgo || !cell || !d_ifgo || !Wh || !ws) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    if (!aligned16(dout) || !aligned16(dh) || !aligned16(dc) || !aligned16(ifgo) || !aligned16(cell) ||
        !aligned16(d_ifgo) || !aligned16(Wh) || !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, 1, &pl, false)) return rc;
    if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
    const bool sync = pl.wave_split != 2;
    if (n_others && (sync || n_others > 3)) return FASTLSTM_ERR_DIM;
    const int kstep = dtype == FASTLSTM_FP32 ? 16 : 32;
    unsigned char *wsb = static_cast<unsigned char *>(ws);
    if (pl.wave_split == 3) {   // W_h does not fit on chip: pack Wh[:, units]^T once, then stream it every step
        const StreamLayout l = stream_layout(pl, H, dtype, true);
        hipStream_t s = static_cast<hipStream_t>(stream);
        if (launch_pack_wh(dtype, true, Wh, wsb + l.wpack_off, H, l.KS, l.KSP, l.mt, pl.n_htiles, s) != hipSuccess)
            return FASTLSTM_ERR_HIP;
        BwdStreamParams p{};
        p.dout = dout; p.dh = dh; p.dc = dc; p.ifgo = ifgo; p.cell = cell; p.d_ifgo = d_ifgo;
        p.wpack = wsb + l.wpack_off;
        p.hdr = reinterpret_cast<WsHeader *>(wsb);
        p.T = T; p.B = B; p.H = H;
        p.n_bt = pl.n_btiles; p.n_ht = pl.n_htiles;
        p.flag_stride = (int)align_up((size_t)pl.n_htiles, 64);
        p.KSB = l.KS; p.KSBP = l.KSP;
        p.spin_limit = spin_limit_ticks();
        const int n_bt_total = cdiv(B, pl.bt);
        for (int c = 0, bt0 = 0; bt0 < n_bt_total; ++c, bt0 += pl.n_btiles) {
            const int n_bt = std::min(pl.n_btiles, n_bt_total - bt0);
            unsigned char *chunk = wsb + kWsHeaderBytes + kWsCounterBytes + (size_t)c * l.chunk_bytes;
            p.flags = reinterpret_cast<int *>(chunk);
            p.xbuf = chunk + l.flags_bytes;
            p.b_base = bt0 * pl.bt;
            const int grid = n_bt * pl.n_htiles;
            int occ = 0;
            if (launch_bwd_stream(dtype, p, l.mt, pl.bt / 16, 0, pl.lds_bytes, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
            if ((long long)occ * pl.num_cus < grid) return FASTLSTM_ERR_RESIDENCY;
            if (launch_bwd_stream(dtype, p, l.mt, pl.bt / 16, grid, pl.lds_bytes, s, nullptr) != hipSuccess) return FASTLSTM_ERR_HIP;
        }
        return FASTLSTM_OK;
    }
    if (sync) {
        int rc = try_bwd_xcd(dout, dh, dc, ifgo, cell, d_ifgo, Wh, wsb, ws_bytes, T, B, H, dtype,
                             static_cast<hipStream_t>(stream));
        if (rc == 1)
            rc = try_bwd_wide(dout, dh, dc, ifgo, cell, d_ifgo, Wh, wsb, ws_bytes, T, B, H, dtype,
                              static_cast<hipStream_t>(stream));
        if (rc == 1) {   // too many batch tiles for one XCD-local launch: one launch per range of rows
            if (const int rows = xcd_rows_per_launch(T, B, H, dtype, true, ws_bytes)) {
                for (int r0 = 0; r0 < B; r0 += rows) {
                    if (r0 && !clear_xcd_counters(wsb, static_cast<hipStream_t>(stream))) return FASTLSTM_ERR_HIP;
                    const LaunchOpts o{1, r0, std::min(rows, B - r0)};
                    const int r = try_bwd_xcd(dout, dh, dc, ifgo, cell, d_ifgo, Wh, wsb, ws_bytes, T, B, H, dtype,
                                              static_cast<hipStream_t>(stream), nullptr, nullptr, false, nullptr, o);
                    if (r != FASTLSTM_OK) return r < 0 ? r : FASTLSTM_ERR_RESIDENCY;
                }
                return FASTLSTM_OK;
            }
            if (const int rows = wide_rows_per_launch(T, B, H, dtype, true, ws_bytes)) {
                for (int r0 = 0; r0 < B; r0 += rows) {
                    if (r0 && !clear_xcd_counters(wsb, static_cast<hipStream_t>(stream))) return FASTLSTM_ERR_HIP;
                    const LaunchOpts o{1, r0, std::min(rows, B - r0)};
                    const int r = try_bwd_wide(dout, dh, dc, ifgo, cell, d_ifgo, Wh, wsb, ws_bytes, T, B, H, dtype,
                                               static_cast<hipStream_t>(stream), o);
                    if (r != FASTLSTM_OK) return r < 0 ? r : FASTLSTM_ERR_RESIDENCY;
                }
                return FASTLSTM_OK;
            }
        }
        if (rc != 1) return rc;   // launched (0) or failed (< 0); 1: not applicable, use the general kernels
    }
    BwdParams p{};
    p.dout = dout; p.dh = dh; p.dc = dc; p.ifgo = ifgo; p.cell = cell; p.d_ifgo = d_ifgo; p.Wh = Wh;
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.T = T; p.B = B; p.H = H;
    p.n_ht = pl.n_htiles;
    p.flag_stride = (int)align_up((size_t)pl.n_htiles, 64);
    p.KSB = cdiv(4 * H, kstep);
    p.ht = pl.ht;
    p.spin_limit = spin_limit_ticks();
    p.trace = g_rec_trace;
    p.n_rec = 1 + n_others;
    for (int i = 0; i < n_others; ++i) {
        p.dout_x[i] = others[i][0]; p.dh_x[i] = others[i][1]; p.dc_x[i] = others[i][2]; p.ifgo_x[i] = others[i][3];
        p.cell_x[i] = others[i][4]; p.d_ifgo_x[i] = others[i][5]; p.Wh_x[i] = others[i][6];
    }
    const size_t flags_bytes = recurrent_flags_bytes(pl.n_btiles, pl.n_htiles);
    const size_t slot_bytes = recurrent_slot_bytes(H, dtype, pl.bt, pl.n_btiles, true);
    // coalesced tile I/O needs complete, 16-byte aligned row segments and room in LDS
    int lds_bytes = pl.lds_bytes;
    {
        const int s = elem_bytes(dtype), gseg = pl.ht * s;
        const int tile_bytes = (pl.bt * (4 * gseg + 16) + 2 * pl.bt * (gseg + 16)) * (sync ? 1 : 2);
        p.vec_io = (gseg >= 16 && (H * s) % 16 == 0 && H % pl.ht == 0 && lds_bytes + tile_bytes <= pl.lds_limit) ? 1 : 0;
        if (p.vec_io) lds_bytes += tile_bytes;
    }
    // 64 units per workgroup: batch tiles of 4 or 8 rows where that many workgroups still find a CU each
    int bt = pl.bt, n_btiles = pl.n_btiles;
    if (!sync && p.vec_io && pl.ht == 64 && pl.bt == 16) {
        p.rs = one_tile_row_split(B, 1 + n_others, pl.num_cus);
        bt = 16 / std::max(p.rs, 1);
        n_btiles = cdiv(B, bt);
    }
    const int n_bt_total = cdiv(B, bt);
    BwdLauncher launch = bwd_launcher(dtype);
    for (int c = 0, bt0 = 0; bt0 < n_bt_total; ++c, bt0 += n_btiles) {
        const int n_bt = std::min(n_btiles, n_bt_total - bt0);
        p.flags = reinterpret_cast<int *>(wsb + kWsHeaderBytes + kWsCounterBytes + (size_t)c * flags_bytes);
        p.xbuf = wsb + pl.ws_zero_bytes + (size_t)c * 2 * slot_bytes;
        p.n_bt = pl.n_btiles;
        p.b_base = bt0 * bt;
        p.n_bt_launch = n_bt;
        const int grid = p.n_rec * n_bt * pl.n_htiles;
        int occ = 0;
        if (launch(p, pl.ht, pl.bt, pl.wave_split, 0, lds_bytes, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
        if (sync && (long long)occ * pl.num_cus < grid) return FASTLSTM_ERR_RESIDENCY;
        if (launch(p, pl.ht, pl.bt, pl.wave_split, grid, lds_bytes, static_cast<hipStream_t>(stream), nullptr) !=
            hipSuccess)
            return FASTLSTM_ERR_HIP;
    }
    return FASTLSTM_OK;
}

int fastlstm_bwd_persistent(const void *dout, void *dh, void *dc, const void *ifgo, const void *cell,
                            void *d_ifgo, const void *Wh, void *ws, size_t ws_bytes, int T, int B, int H,
                            int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    PoisonList pl{};
    pl.dtype = dtype;
    pl.add(dh, (size_t)B * H); pl.add(dc, (size_t)B * H); pl.add(d_ifgo, (size_t)4 * H);   // (d_ifgo[0][0]: every product made of it)
    return finish_recurrent(bwd_persistent_impl(dout, dh, dc, ifgo, cell, d_ifgo, Wh, ws, ws_bytes, T, B, H, dtype, stream), ws,
                            stream, pl);
}

// n = 2 ... kMaxSideBySide recurrences of one shape (recs[r]: the operand pointers of recurrence r in the order of
// the single entry point): side by side in one launch of the XCD-local kernels where they all fit (returns 0), else
// 1 (not launched).
static int try_multi(bool backward, int n, void *const (*recs)[7], void *ws, size_t ws_bytes, int T, int B, int H, int dtype,
                     void *stream, int keep, bool dry_run) {
    if (n < 2 || n > kMaxSideBySide) return 1;
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, backward ? 1 : 0, &pl, false)) return rc;
    if (pl.wave_split == 3) return 1;
    void *const *a = recs[0], *const *b = recs[1];
    if (pl.wave_split == 2) {   // the one-tile form: no exchange between workgroups, any number of them side by side
        if (dry_run) return FASTLSTM_OK;
        return backward ? bwd_persistent_impl(a[0], a[1], a[2], a[3], a[4], a[5], a[6], ws, ws_bytes, T, B, H, dtype, stream,
                                              recs + 1, n - 1)
                        : fwd_persistent_impl(a[0], a[1], a[2], a[3], ws, ws_bytes, T, B, H, dtype, stream, keep, recs + 1, n - 1);
    }
    unsigned char *wsb = static_cast<unsigned char *>(ws);
    hipStream_t s = static_cast<hipStream_t>(stream);
    LaunchOpts o;
    o.keep = keep;
    o.n_more = n - 2;
    o.more = recs + 2;
    int rc;
    if (!backward) {
        const SecondLayer second{nullptr, nullptr, nullptr, b[3], b[0], b[1], b[2]};
        rc = try_fwd_xcd(a[0], a[1], a[2], a[3], wsb, ws_bytes, T, B, H, dtype, s, nullptr, nullptr, nullptr, nullptr, 0, &second,
                         dry_run, o);
        if (rc == 1 || rc == 2) rc = try_fwd_wide(a[0], a[1], a[2], a[3], wsb, ws_bytes, T, B, H, dtype, s, o, &second, dry_run);
    } else {
        LowerLayer lower{b[1], b[2], b[3], b[4], b[5], b[6], nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, nullptr, nullptr};
        lower.dout = b[0];
        rc = try_bwd_xcd(a[0], a[1], a[2], a[3], a[4], a[5], a[6], wsb, ws_bytes, T, B, H, dtype, s, nullptr, &lower, dry_run,
                         nullptr, o);
        if (rc == 1 || rc == 2) rc = try_bwd_wide(a[0], a[1], a[2], a[3], a[4], a[5], a[6], wsb, ws_bytes, T, B, H, dtype, s, o, b, dry_run);
    }
    return rc == 2 ? 1 : rc;
}
size_t fastlstm_multi_workspace_bytes(const fastlstm_plan *plan, int n, int T, int H, int dtype, int backward) {
    const size_t one = fastlstm_recurrent_workspace_bytes(plan, T, H, dtype, backward);
    if (!plan || one == 0 || n <= 1 || plan->wave_split >= 2) return one;
    const size_t head = kWsHeaderBytes + kWsCounterBytes;
    return one > head ? head + (size_t)n * (one - head) : one;
}

int fastlstm_multi_fused(int n, int T, int B, int H, int dtype, int backward, size_t ws_bytes) {
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    if (n < 1 || n > kMaxSideBySide) return FASTLSTM_ERR_DIM;
    void *fake[kMaxSideBySide][7];
    for (auto &r : fake)
        for (void *&q : r) q = reinterpret_cast<void *>(static_cast<size_t>(4096));   // never dereferenced
    const int rc = try_multi(backward != 0, n, fake, fake[0][0], ws_bytes, T, B, H, dtype, nullptr, 1, true);
    return rc == FASTLSTM_OK ? 1 : (rc < 0 ? rc : 0);
}

// n recurrences one after the other on one workspace, which is cleared in between
static int multi_sequential(bool backward, int n, void *const (*r)[7], void *ws, size_t ws_bytes, int T, int B, int H, int dtype,
                            void *stream, int keep) {
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, backward ? 1 : 0, &pl, false)) return rc;
    const size_t zero = pl.ring_needs_zero ? ws_bytes : std::min(ws_bytes, pl.ws_zero_bytes);
    for (int i = 0; i < n; ++i) {
        if (i) {
            zero_words_kernel<<<256, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<unsigned *>(ws), zero / 4);
            if (hipGetLastError() != hipSuccess) return FASTLSTM_ERR_HIP;
        }
        const int rc = backward ? bwd_persistent_impl(r[i][0], r[i][1], r[i][2], r[i][3], r[i][4], r[i][5], r[i][6], ws, ws_bytes, T, B,
                                                      H, dtype, stream)
                                : fwd_persistent_impl(r[i][0], r[i][1], r[i][2], r[i][3], ws, ws_bytes, T, B, H, dtype, stream, keep);
        if (rc != FASTLSTM_OK) return rc;
    }
    return FASTLSTM_OK;
}

int fastlstm_fwd_persistent_multi(int n, void *const *ifgo, void *const *out, void *const *cell, const void *const *Wh, void *ws,
                                  size_t ws_bytes, int T, int B, int H, int dtype, int keep_activations, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    if (!ifgo || !out || !cell || !Wh || !ws) return FASTLSTM_ERR_NULL;
    if (n < 1 || n > kMaxSideBySide) return FASTLSTM_ERR_DIM;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    void *recs[kMaxSideBySide][7] = {};
    for (int i = 0; i < n; ++i) {
        recs[i][0] = ifgo[i]; recs[i][1] = out[i]; recs[i][2] = cell[i]; recs[i][3] = const_cast<void *>(Wh[i]);
        for (int k = 0; k < 4; ++k) {
            if (!recs[i][k]) return FASTLSTM_ERR_NULL;
            if (!aligned16(recs[i][k])) return FASTLSTM_ERR_ALIGN;
        }
    }
    if (!aligned16(ws)) return FASTLSTM_ERR_ALIGN;
    const int keep = keep_activations ? 1 : 0;
    int rc = try_multi(false, n, recs, ws, ws_bytes, T, B, H, dtype, stream, keep, false);
    if (rc == 1) rc = multi_sequential(false, n, recs, ws, ws_bytes, T, B, H, dtype, stream, keep);
    PoisonList pl{};
    pl.dtype = dtype;
    for (int i = 0; i < n; ++i) { pl.add(last_slab(recs[i][1], T, B, H, dtype), (size_t)B * H); pl.add(last_slab(recs[i][2], T, B, H, dtype), (size_t)B * H); }
    return finish_recurrent(rc, ws, stream, pl);
}

int fastlstm_bwd_persistent_multi(int n, const void *const *dout, void *const *dh, void *const *dc, const void *const *ifgo,
                                  const void *const *cell, void *const *d_ifgo, const void *const *Wh, void *ws, size_t ws_bytes,
                                  int T, int B, int H, int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    if (!dout || !dh || !dc || !ifgo || !cell || !d_ifgo || !Wh || !ws) return FASTLSTM_ERR_NULL;
    if (n < 1 || n > kMaxSideBySide) return FASTLSTM_ERR_DIM;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    void *recs[kMaxSideBySide][7] = {};
    for (int i = 0; i < n; ++i) {
        recs[i][0] = const_cast<void *>(dout[i]); recs[i][1] = dh[i]; recs[i][2] = dc[i]; recs[i][3] = const_cast<void *>(ifgo[i]);
        recs[i][4] = const_cast<void *>(cell[i]); recs[i][5] = d_ifgo[i]; recs[i][6] = const_cast<void *>(Wh[i]);
        for (int k = 0; k < 7; ++k) {
            if (!recs[i][k]) return FASTLSTM_ERR_NULL;
            if (!aligned16(recs[i][k])) return FASTLSTM_ERR_ALIGN;
        }
    }
    if (!aligned16(ws)) return FASTLSTM_ERR_ALIGN;
    int rc = try_multi(true, n, recs, ws, ws_bytes, T, B, H, dtype, stream, 1, false);
    if (rc == 1) rc = multi_sequential(true, n, recs, ws, ws_bytes, T, B, H, dtype, stream, 1);
    PoisonList pl{};
    pl.dtype = dtype;
    for (int i = 0; i < n; ++i) { pl.add(recs[i][1], (size_t)B * H); pl.add(recs[i][5], (size_t)4 * H); }
    return finish_recurrent(rc, ws, stream, pl);
}

int fastlstm_pair_fused(int T, int B, int H, int dtype, int backward, size_t ws_bytes) {
    return fastlstm_multi_fused(2, T, B, H, dtype, backward, ws_bytes);
}

int fastlstm_fwd_persistent_pair(void *ifgo_a, void *out_a, void *cell_a, const void *Wh_a, void *ifgo_b, void *out_b,
                                 void *cell_b, const void *Wh_b, void *ws, size_t ws_bytes, int T, int B, int H, int dtype,
                                 int keep_activations, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    if (!ifgo_a || !out_a || !cell_a || !Wh_a || !ifgo_b || !out_b || !cell_b || !Wh_b || !ws) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    void *const a[7] = {ifgo_a, out_a, cell_a, const_cast<void *>(Wh_a)}, *const b[7] = {ifgo_b, out_b, cell_b, const_cast<void *>(Wh_b)};
    for (int i = 0; i < 4; ++i)
        if (!aligned16(a[i]) || !aligned16(b[i])) return FASTLSTM_ERR_ALIGN;
    if (!aligned16(ws)) return FASTLSTM_ERR_ALIGN;
    const int keep = keep_activations ? 1 : 0;
    void *recs[2][7];
    for (int i = 0; i < 7; ++i) { recs[0][i] = a[i]; recs[1][i] = b[i]; }
    int rc = try_multi(false, 2, recs, ws, ws_bytes, T, B, H, dtype, stream, keep, false);
    if (rc == 1) rc = multi_sequential(false, 2, recs, ws, ws_bytes, T, B, H, dtype, stream, keep);
    return finish_recurrent(rc, ws, stream, poison_fwd(dtype, T, B, H, out_a, cell_a, out_b, cell_b));
}

int fastlstm_bwd_persistent_pair(const void *dout_a, void *dh_a, void *dc_a, const void *ifgo_a, const void *cell_a,
                                 void *d_ifgo_a, const void *Wh_a, const void *dout_b, void *dh_b, void *dc_b,
                                 const void *ifgo_b, const void *cell_b, void *d_ifgo_b, const void *Wh_b, void *ws,
                                 size_t ws_bytes, int T, int B, int H, int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    void *const a[7] = {const_cast<void *>(dout_a), dh_a, dc_a, const_cast<void *>(ifgo_a), const_cast<void *>(cell_a), d_ifgo_a,
                        const_cast<void *>(Wh_a)};
    void *const b[7] = {const_cast<void *>(dout_b), dh_b, dc_b, const_cast<void *>(ifgo_b), const_cast<void *>(cell_b), d_ifgo_b,
                        const_cast<void *>(Wh_b)};
    for (int i = 0; i < 7; ++i) {
        if (!a[i] || !b[i]) return FASTLSTM_ERR_NULL;
        if (!aligned16(a[i]) || !aligned16(b[i])) return FASTLSTM_ERR_ALIGN;
    }
    if (!ws) return FASTLSTM_ERR_NULL;
    if (!aligned16(ws)) return FASTLSTM_ERR_ALIGN;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    void *recs[2][7];
    for (int i = 0; i < 7; ++i) { recs[0][i] = a[i]; recs[1][i] = b[i]; }
    int rc = try_multi(true, 2, recs, ws, ws_bytes, T, B, H, dtype, stream, 1, false);
    if (rc == 1) rc = multi_sequential(true, 2, recs, ws, ws_bytes, T, B, H, dtype, stream, 1);
    PoisonList pl{};
    pl.dtype = dtype;
    pl.add(dh_a, (size_t)B * H); pl.add(d_ifgo_a, (size_t)4 * H); pl.add(dh_b, (size_t)B * H); pl.add(d_ifgo_b, (size_t)4 * H);
    return finish_recurrent(rc, ws, stream, pl);
}

static int fwd_layer_impl(const void *x, const void *Wx, const void *bx, const void *bh, const void *Wh, void *ifgo,
                          void *out, void *cell, void *ws, size_t ws_bytes, int T, int B, int I, int H, int dtype,
                          void *stream, int keep) {
    if (!x || !Wx || !bx || !bh || !Wh || !ifgo || !out || !cell || !ws) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(x) || !aligned16(Wx) || !aligned16(ifgo) || !aligned16(out) || !aligned16(cell) || !aligned16(Wh) ||
        !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    // Where the XCD-local recurrence leaves CUs without a role, those workgroups compute the input
    // projection inside the same launch, earliest timesteps first, and the recurrence follows them
    // chunk by chunk; otherwise K1 and the recurrence are two launches back to back.
#ifndef FASTLSTM_TIMELINE
    {
        fastlstm_plan pl;
        if (int rc = plan_device(-1, B, H, dtype, 0, &pl, false)) return rc;
        if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
        if (pl.wave_split != 2) {
            const int rc = try_fwd_xcd(ifgo, out, cell, Wh, static_cast<unsigned char *>(ws), ws_bytes, T, B, H, dtype,
                                       static_cast<hipStream_t>(stream), x, Wx, bx, bh, I, nullptr, false,
                                       LaunchOpts{keep, 0, 0});
            if (rc <= 0) return rc;   // launched, or failed
        }
    }
#endif
    if (int rc = fastlstm_gemm_ifgo(x, Wx, bx, bh, ifgo, T, B, I, H, dtype, stream)) return rc;
    return fwd_persistent_impl(ifgo, out, cell, Wh, ws, ws_bytes, T, B, H, dtype, stream, keep);
}

int fastlstm_fwd_layer(const void *x, const void *Wx, const void *bx, const void *bh, const void *Wh, void *ifgo,
                       void *out, void *cell, void *ws, size_t ws_bytes, int T, int B, int I, int H, int dtype,
                       void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    return finish_recurrent(fwd_layer_impl(x, Wx, bx, bh, Wh, ifgo, out, cell, ws, ws_bytes, T, B, I, H, dtype, stream, 1), ws,
                            stream, poison_fwd(dtype, T, B, H, out, cell));
}

int fastlstm_fwd_layer_infer(const void *x, const void *Wx, const void *bx, const void *bh, const void *Wh, void *ifgo,
                             void *out, void *cell, void *ws, size_t ws_bytes, int T, int B, int I, int H, int dtype,
                             void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    return finish_recurrent(fwd_layer_impl(x, Wx, bx, bh, Wh, ifgo, out, cell, ws, ws_bytes, T, B, I, H, dtype, stream, 0), ws,
                            stream, poison_fwd(dtype, T, B, H, out, cell));
}

// ---- fastlstm_fwd_layer for callers that cannot allocate ---------------------------------------
// The recurrence workspace lives in a file-scope device array instead of coming in as an argument.
// In host code the array's NAME is only a stand-in (a kernel given it faults): its device address is
// looked up once per device with hipGetSymbolAddress and kept; every use below goes through that pointer.
constexpr size_t kNoAllocScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
static unsigned char *g_scratch_ptr[64];   // per device, under g_scratch_mu
static std::mutex g_scratch_mu;

// Device address of this device's copy of `scratch` (each GPU holds its own copy at its own address).
static int scratch_of_current_device(unsigned char **out) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return FASTLSTM_ERR_HIP;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return FASTLSTM_ERR_HIP;
        g_scratch_ptr[device] = static_cast<unsigned char *>(ptr);
    }
    *out = g_scratch_ptr[device];
    return FASTLSTM_OK;
}

// Also the set-up call of fastlstm_fwd_layer_noalloc for the current device: looks up the array's device address
// and creates what the failure reporting and the ordering of streams need (a pinned status word, an event), so
// that the entry point itself -- possibly under stream capture -- neither allocates nor looks anything up.
size_t fastlstm_noalloc_scratch_bytes(void) {
    unsigned char *ptr = nullptr;
    int device = -1;
    if (scratch_of_current_device(&ptr) == FASTLSTM_OK && hipGetDevice(&device) == hipSuccess) {
        DeviceInfo di;
        if (device_info(device, &di) == FASTLSTM_OK && !di.status_dev) ensure_status_word(device, nullptr);
        std::lock_guard<std::mutex> lock(g_order_mu);
        if (device >= 0 && device < 64 && !g_order[device].event &&
            hipEventCreateWithFlags(&g_order[device].event, hipEventDisableTiming) != hipSuccess)
            g_order[device].event = nullptr;
    }
    return kNoAllocScratchBytes;
}

int fastlstm_fwd_layer_noalloc(const void *x, const void *Wx, const void *bx, const void *bh, const void *Wh, void *ifgo,
                               void *out, void *cell, int T, int B, int I, int H, int dtype, void *stream) {
    if (!x || !Wx || !bx || !bh || !Wh || !ifgo || !out || !cell) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (int rc = begin_recurrent(stream)) return rc;
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, 0, &pl, false)) return rc;
    // the smallest workspace of this shape has to fit; beyond that the call uses as much of the array
    // as a ring with one slot per timestep would take (more slots = the faster kernels, as with any workspace)
    if (pl.ws_bytes > kNoAllocScratchBytes) return FASTLSTM_ERR_WORKSPACE;
    const size_t ring = fastlstm_recurrent_workspace_bytes(&pl, T, H, dtype, 0);
    const size_t use = std::min(kNoAllocScratchBytes, std::max(ring, pl.ws_bytes));
    unsigned char *ptr = nullptr;
    if (int rc = scratch_of_current_device(&ptr)) return rc;
    // the array keeps the last call's contents: clear what this call needs zeroed (a fill kernel, so the
    // call can be captured into a graph)
    const size_t zero = pl.ring_needs_zero ? use : std::min(use, pl.ws_zero_bytes);
    zero_words_kernel<<<256, 256, 0, static_cast<hipStream_t>(stream)>>>(reinterpret_cast<unsigned *>(ptr), zero / 4);
    if (hipGetLastError() != hipSuccess) return FASTLSTM_ERR_HIP;
    return finish_recurrent(fwd_layer_impl(x, Wx, bx, bh, Wh, ifgo, out, cell, ptr, use, T, B, I, H, dtype, stream, 1), ptr,
                            stream, poison_fwd(dtype, T, B, H, out, cell), false);
}

size_t fastlstm_stack2_workspace_bytes(const fastlstm_plan *plan, int T, int H, int dtype) {
    const size_t one = fastlstm_recurrent_workspace_bytes(plan, T, H, dtype, 0);
    if (!plan || one == 0 || plan->wave_split >= 2) return one;
    const size_t head = kWsHeaderBytes + kWsCounterBytes;
    return one > head ? head + 2 * (one - head) : one;
}

int fastlstm_fwd_stack2_fused(int T, int B, int I, int H, int dtype, size_t ws_bytes) {
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    unsigned char *fake = reinterpret_cast<unsigned char *>(static_cast<size_t>(4096));   // never dereferenced
    const SecondLayer second{fake, fake, fake, fake, fake, fake, fake};
    const int rc = try_fwd_xcd(fake, fake, fake, fake, fake, ws_bytes, T, B, H, dtype, nullptr, fake, fake, fake, fake, I,
                               &second, true);
    return rc == FASTLSTM_OK ? 1 : (rc < 0 ? rc : 0);
}

static int fwd_stack2_impl(const void *x, const void *Wx0, const void *bx0, const void *bh0, const void *Wh0, void *ifgo0,
                           void *out0, void *cell0, const void *Wx1, const void *bx1, const void *bh1, const void *Wh1,
                           void *ifgo1, void *out1, void *cell1, void *ws, size_t ws_bytes, int T, int B, int I, int H,
                           int dtype, void *stream, int keep) {
    if (!x || !Wx0 || !bx0 || !bh0 || !Wh0 || !ifgo0 || !out0 || !cell0 || !Wx1 || !bx1 || !bh1 || !Wh1 || !ifgo1 ||
        !out1 || !cell1 || !ws)
        return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(x) || !aligned16(Wx0) || !aligned16(ifgo0) || !aligned16(out0) || !aligned16(cell0) ||
        !aligned16(Wh0) || !aligned16(Wx1) || !aligned16(ifgo1) || !aligned16(out1) || !aligned16(cell1) ||
        !aligned16(Wh1) || !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, 0, &pl, false)) return rc;
    if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
#ifndef FASTLSTM_TIMELINE
    if (pl.wave_split != 2) {
        const SecondLayer second{Wx1, bx1, bh1, Wh1, ifgo1, out1, cell1};
        const int rc = try_fwd_xcd(ifgo0, out0, cell0, Wh0, static_cast<unsigned char *>(ws), ws_bytes, T, B, H, dtype, s, x,
                                   Wx0, bx0, bh0, I, &second, false, LaunchOpts{keep, 0, 0});
        if (rc <= 0) return rc;   // both layers in one launch, or failed
    }
#endif
    // one layer after the other, the second on the first one's out[1:]; the workspace is cleared in between
    if (int rc = fwd_layer_impl(x, Wx0, bx0, bh0, Wh0, ifgo0, out0, cell0, ws, ws_bytes, T, B, I, H, dtype, stream, keep))
        return rc;
    const size_t zero = pl.ring_needs_zero ? ws_bytes : std::min(ws_bytes, pl.ws_zero_bytes);
    zero_words_kernel<<<256, 256, 0, s>>>(static_cast<unsigned *>(ws), zero / 4);
    if (hipGetLastError() != hipSuccess) return FASTLSTM_ERR_HIP;
    const void *x1 = static_cast<const unsigned char *>(out0) + (size_t)B * H * elem_bytes(dtype);
    return fwd_layer_impl(x1, Wx1, bx1, bh1, Wh1, ifgo1, out1, cell1, ws, ws_bytes, T, B, H, H, dtype, stream, keep);
}

int fastlstm_fwd_stack2(const void *x, const void *Wx0, const void *bx0, const void *bh0, const void *Wh0, void *ifgo0,
                        void *out0, void *cell0, const void *Wx1, const void *bx1, const void *bh1, const void *Wh1,
                        void *ifgo1, void *out1, void *cell1, void *ws, size_t ws_bytes, int T, int B, int I, int H,
                        int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    return finish_recurrent(fwd_stack2_impl(x, Wx0, bx0, bh0, Wh0, ifgo0, out0, cell0, Wx1, bx1, bh1, Wh1, ifgo1, out1, cell1,
                                            ws, ws_bytes, T, B, I, H, dtype, stream, 1),
                            ws, stream, poison_fwd(dtype, T, B, H, out1, cell1, out0, cell0));
}

int fastlstm_fwd_stack2_infer(const void *x, const void *Wx0, const void *bx0, const void *bh0, const void *Wh0,
                              void *ifgo0, void *out0, void *cell0, const void *Wx1, const void *bx1, const void *bh1,
                              const void *Wh1, void *ifgo1, void *out1, void *cell1, void *ws, size_t ws_bytes, int T,
                              int B, int I, int H, int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    return finish_recurrent(fwd_stack2_impl(x, Wx0, bx0, bh0, Wh0, ifgo0, out0, cell0, Wx1, bx1, bh1, Wh1, ifgo1, out1, cell1,
                                            ws, ws_bytes, T, B, I, H, dtype, stream, 0),
                            ws, stream, poison_fwd(dtype, T, B, H, out1, cell1, out0, cell0));
}

// bytes of the partial sums that a reverse launch leaves of a layer's bias gradient (BwdXcdParams::db_part)
static size_t db_part_bytes(int B, int H) { return align_up((size_t)cdiv(B, 16) * 4 * H * sizeof(float), 256); }

static int bwd_layer_impl(const void *dout, void *dh, void *dc, const void *ifgo, const void *cell, void *d_ifgo,
                          const void *Wh, const void *Wx, const void *x, const void *h, void *dx, void *dWx, void *dWh,
                          void *db, void *ws, size_t ws_bytes, void *wgrad_ws, size_t wgrad_ws_bytes, int T, int B, int I,
                          int H, int dtype, void *stream) {
    // dx may be null (no gradient of the layer's input is wanted: K5 is skipped), and so may dWx, dWh and db,
    // all three together (frozen weights: K8, K9 and the bias sum are skipped)
    const bool want_w = dWx || dWh || db;
    if (!dout || !dh || !dc || !ifgo || !cell || !d_ifgo || !Wh || !Wx || !x || !h || !ws || !wgrad_ws ||
        (want_w && (!dWx || !dWh || !db)))
        return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(dout) || !aligned16(dh) || !aligned16(dc) || !aligned16(ifgo) || !aligned16(cell) ||
        !aligned16(d_ifgo) || !aligned16(Wh) || !aligned16(Wx) || !aligned16(x) || !aligned16(h) || !aligned16(dx) ||
        !aligned16(dWx) || !aligned16(dWh) || !aligned16(ws) || !aligned16(wgrad_ws))
        return FASTLSTM_ERR_ALIGN;
    if (wgrad_ws_bytes < fastlstm_wgrad_workspace_bytes(T, B, I, H, dtype)) return FASTLSTM_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Where the XCD-local reverse recurrence leaves CUs without a role, those workgroups compute dx
    // and the weight gradients inside the same launch, chunk of timesteps by chunk behind the
    // recurrence; otherwise the stages are launched back to back.
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, 1, &pl, false)) return rc;
    if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
    int rc = 1;
    int db_done = 0;
    if (pl.wave_split != 2 && (dx || want_w)) {
        // (the weight-gradient workspace is not used by a launch that has the weight gradients inside: it takes the
        // partial sums of the bias gradient)
        float *db_part = want_w && db_part_bytes(B, H) <= wgrad_ws_bytes ? static_cast<float *>(wgrad_ws) : nullptr;
        const BwdExtras e{Wx, x, h, dx, dWx, dWh, I, db_part};
        rc = try_bwd_xcd(dout, dh, dc, ifgo, cell, d_ifgo, Wh, static_cast<unsigned char *>(ws), ws_bytes, T, B, H, dtype,
                         s, &e, nullptr, false, nullptr, LaunchOpts(), &db_done);
        if (rc < 0) return rc;
    }
    if (rc == 0) {   // everything was part of the launch but the last step of the bias gradient ...
        if (db_done & 1)
            return launch_colsum_final(dtype, static_cast<float *>(wgrad_ws), db, 4 * H, cdiv(B, 16), s) == hipSuccess
                       ? FASTLSTM_OK
                       : FASTLSTM_ERR_HIP;
        const int chunks = colsum_chunks(T * B);   // ... or all of it
        return launch_colsum(dtype, d_ifgo, db, static_cast<float *>(wgrad_ws), T * B, 4 * H, chunks, s) == hipSuccess
                   ? FASTLSTM_OK
                   : FASTLSTM_ERR_HIP;
    }
    if (rc != 3) {   // nothing was launched: recurrence, then dx
        if (int r2 = bwd_persistent_impl(dout, dh, dc, ifgo, cell, d_ifgo, Wh, ws, ws_bytes, T, B, H, dtype, stream))
            return r2;
        return gemm_dx_wgrad_impl(d_ifgo, Wx, x, h, dx, want_w ? dWx : nullptr, dWh, db, wgrad_ws, wgrad_ws_bytes, T, B, I, H,
                                  dtype, stream);
    }
    if (!want_w) return FASTLSTM_OK;
    return fastlstm_gemm_wgrad(d_ifgo, x, h, dWx, dWh, db, wgrad_ws, wgrad_ws_bytes, T, B, I, H, dtype, stream);
}

int fastlstm_bwd_layer(const void *dout, void *dh, void *dc, const void *ifgo, const void *cell, void *d_ifgo,
                       const void *Wh, const void *Wx, const void *x, const void *h, void *dx, void *dWx, void *dWh,
                       void *db, void *ws, size_t ws_bytes, void *wgrad_ws, size_t wgrad_ws_bytes, int T, int B, int I,
                       int H, int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    PoisonList pl{};
    pl.dtype = dtype;
    if (dtype_ok(dtype) && B > 0 && H > 0 && I > 0) {
        pl.add(dh, (size_t)B * H); pl.add(dc, (size_t)B * H); pl.add(dx, (size_t)B * I); pl.add(db, (size_t)4 * H);
        pl.add(dWx, (size_t)I); pl.add(dWh, (size_t)H);
    }
    return finish_recurrent(bwd_layer_impl(dout, dh, dc, ifgo, cell, d_ifgo, Wh, Wx, x, h, dx, dWx, dWh, db, ws, ws_bytes,
                                           wgrad_ws, wgrad_ws_bytes, T, B, I, H, dtype, stream),
                            ws, stream, pl);
}

size_t fastlstm_stack2_bwd_workspace_bytes(const fastlstm_plan *plan, int T, int H, int dtype) {
    const size_t one = fastlstm_recurrent_workspace_bytes(plan, T, H, dtype, 1);
    if (!plan || one == 0 || plan->wave_split >= 2) return one;
    const size_t head = kWsHeaderBytes + kWsCounterBytes;
    return one > head ? head + 2 * (one - head) : one;
}

size_t fastlstm_stack2_bwd_wgrad_workspace_bytes(int T, int B, int I, int H, int dtype) {
    const size_t need = std::max(fastlstm_wgrad_workspace_bytes(T, B, I, H, dtype), fastlstm_wgrad_workspace_bytes(T, B, H, H, dtype));
    if (need == 0 || dtype == FASTLSTM_FP32) return need;
    // one parked 256 x 256 fp32 tile per helper and layer (see plan_bwd_helpers): with that much the one launch
    // also computes the lower layer's weight gradients
    const size_t tile_bytes = (size_t)256 * 256 * sizeof(float);
    const int rows = cdiv(4 * H, 256), helpers = kNumXcd * 32;
    const size_t upper = std::min(rows * 2 * cdiv(H, 256), helpers), lower = std::min(rows * (cdiv(I, 256) + cdiv(H, 256)), helpers);
    // ... and the partial sums of both layers' bias gradients behind them
    return std::max(need, (upper + lower) * tile_bytes) + 2 * db_part_bytes(B, H) + 256;
}

int fastlstm_bwd_stack2_fused(int T, int B, int I, int H, int dtype, size_t ws_bytes) {
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    unsigned char *fake = reinterpret_cast<unsigned char *>(static_cast<size_t>(4096));   // never dereferenced
    const BwdExtras e{fake, fake, fake, fake, fake, fake, H};
    const LowerLayer lower{fake, fake, fake, fake, fake, fake, fake, fake, I, fake, (size_t)1 << 40, fake, fake, fake, fake};
    const int rc = try_bwd_xcd(fake, fake, fake, fake, fake, fake, fake, fake, ws_bytes, T, B, H, dtype, nullptr, &e, &lower,
                               true);
    return (rc == FASTLSTM_OK || rc == 3) ? 1 : (rc < 0 ? rc : 0);
}

static int bwd_stack2_impl(const void *dout, void *dh1, void *dc1, const void *ifgo1, const void *cell1, void *d_ifgo1,
                           const void *Wh1, const void *Wx1, const void *out1, void *dWx1, void *dWh1, void *db1, void *dx1,
                           void *dh0, void *dc0, const void *ifgo0, const void *cell0, void *d_ifgo0, const void *Wh0,
                           const void *Wx0, const void *x, const void *out0, void *dx0, void *dWx0, void *dWh0, void *db0,
                           void *ws, size_t ws_bytes, void *wgrad_ws, size_t wgrad_ws_bytes, int T, int B, int I, int H,
                           int dtype, void *stream) {
    if (!dout || !dh1 || !dc1 || !ifgo1 || !cell1 || !d_ifgo1 || !Wh1 || !Wx1 || !out1 || !dWx1 || !dWh1 || !db1 || !dx1 ||
        !dh0 || !dc0 || !ifgo0 || !cell0 || !d_ifgo0 || !Wh0 || !Wx0 || !x || !out0 || !dWx0 || !dWh0 || !db0 ||
        !ws || !wgrad_ws)   // (dx0 may be null: no gradient of the stack's input is wanted)
        return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    const void *ptrs[] = {dout, dh1, dc1, ifgo1, cell1, d_ifgo1, Wh1, Wx1, out1, dWx1, dWh1, dx1, dh0, dc0, ifgo0, cell0,
                          d_ifgo0, Wh0, Wx0, x, out0, dx0, dWx0, dWh0, ws, wgrad_ws};
    for (const void *q : ptrs)
        if (!aligned16(q)) return FASTLSTM_ERR_ALIGN;
    const size_t need = std::max(fastlstm_wgrad_workspace_bytes(T, B, I, H, dtype), fastlstm_wgrad_workspace_bytes(T, B, H, H, dtype));
    if (wgrad_ws_bytes < need) return FASTLSTM_ERR_WORKSPACE;
    fastlstm_plan pl;
    if (int rc = plan_device(-1, B, H, dtype, 1, &pl, false)) return rc;
    if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the upper layer's input is the lower layer's h: x1 = out0[1:]
    const void *x1 = static_cast<const unsigned char *>(out0) + (size_t)B * H * elem_bytes(dtype);
    if (pl.wave_split != 2) {
        // the end of the weight-gradient workspace takes the two layers' partial sums of the bias gradients, the
        // parked weight-gradient tiles come before them
        const size_t dbb = db_part_bytes(B, H);
        const bool db_room = wgrad_ws_bytes >= need + 2 * dbb;
        const size_t park_bytes = db_room ? (wgrad_ws_bytes - 2 * dbb) / 256 * 256 : wgrad_ws_bytes;
        float *dbp1 = db_room ? reinterpret_cast<float *>(static_cast<unsigned char *>(wgrad_ws) + park_bytes) : nullptr;
        float *dbp0 = db_room ? reinterpret_cast<float *>(static_cast<unsigned char *>(wgrad_ws) + park_bytes + dbb) : nullptr;
        const BwdExtras e{Wx1, x1, out1, dx1, dWx1, dWh1, H, dbp1};
        const LowerLayer lower{dh0, dc0, ifgo0, cell0, d_ifgo0, Wh0, Wx0, dx0, I, wgrad_ws, park_bytes, x, out0, dWx0, dWh0, dbp0};
        bool lower_wgrad_done = false;
        int db_done = 0;
        const int rc = try_bwd_xcd(dout, dh1, dc1, ifgo1, cell1, d_ifgo1, Wh1, static_cast<unsigned char *>(ws), ws_bytes, T, B,
                                   H, dtype, s, &e, &lower, false, &lower_wgrad_done, LaunchOpts(), &db_done);
        if (rc < 0) return rc;
        if (rc == 0) {   // both recurrences, both dx and the upper weight gradients were one launch
            if (db_done & 1) {
                if (launch_colsum_final(dtype, dbp1, db1, 4 * H, cdiv(B, 16), s) != hipSuccess) return FASTLSTM_ERR_HIP;
            } else if (launch_colsum(dtype, d_ifgo1, db1, static_cast<float *>(wgrad_ws), T * B, 4 * H, colsum_chunks(T * B), s) !=
                       hipSuccess) {
                return FASTLSTM_ERR_HIP;
            }
        } else if (rc == 3) {   // ... but for the upper weight gradients (T*B not a multiple of the GEMM k-tile)
            if (int r2 = fastlstm_gemm_wgrad(d_ifgo1, x1, out1, dWx1, dWh1, db1, wgrad_ws, wgrad_ws_bytes, T, B, H, H, dtype,
                                             stream))
                return r2;
        }
        if ((rc == 0 || rc == 3) && lower_wgrad_done) {   // only the lower layer's bias gradient is left
            if (db_done & 2)
                return launch_colsum_final(dtype, dbp0, db0, 4 * H, cdiv(B, 16), s) == hipSuccess ? FASTLSTM_OK : FASTLSTM_ERR_HIP;
            return launch_colsum(dtype, d_ifgo0, db0, static_cast<float *>(wgrad_ws), T * B, 4 * H, colsum_chunks(T * B), s) ==
                           hipSuccess
                       ? FASTLSTM_OK
                       : FASTLSTM_ERR_HIP;
        }
        if (rc == 0 || rc == 3)
            return fastlstm_gemm_wgrad(d_ifgo0, x, out0, dWx0, dWh0, db0, wgrad_ws, wgrad_ws_bytes, T, B, I, H, dtype, stream);
    }
    // one layer after the other; the workspace is cleared in between
    if (int rc = bwd_layer_impl(dout, dh1, dc1, ifgo1, cell1, d_ifgo1, Wh1, Wx1, x1, out1, dx1, dWx1, dWh1, db1, ws, ws_bytes,
                                wgrad_ws, wgrad_ws_bytes, T, B, H, H, dtype, stream))
        return rc;
    const size_t zero = pl.ring_needs_zero ? ws_bytes : std::min(ws_bytes, pl.ws_zero_bytes);
    zero_words_kernel<<<256, 256, 0, s>>>(static_cast<unsigned *>(ws), zero / 4);
    if (hipGetLastError() != hipSuccess) return FASTLSTM_ERR_HIP;
    return bwd_layer_impl(dx1, dh0, dc0, ifgo0, cell0, d_ifgo0, Wh0, Wx0, x, out0, dx0, dWx0, dWh0, db0, ws, ws_bytes, wgrad_ws,
                          wgrad_ws_bytes, T, B, I, H, dtype, stream);
}

int fastlstm_bwd_stack2(const void *dout, void *dh1, void *dc1, const void *ifgo1, const void *cell1, void *d_ifgo1,
                        const void *Wh1, const void *Wx1, const void *out1, void *dWx1, void *dWh1, void *db1, void *dx1,
                        void *dh0, void *dc0, const void *ifgo0, const void *cell0, void *d_ifgo0, const void *Wh0,
                        const void *Wx0, const void *x, const void *out0, void *dx0, void *dWx0, void *dWh0, void *db0,
                        void *ws, size_t ws_bytes, void *wgrad_ws, size_t wgrad_ws_bytes, int T, int B, int I, int H,
                        int dtype, void *stream) {
    if (int rc = begin_recurrent(stream)) return rc;
    PoisonList pl{};
    pl.dtype = dtype;
    if (dtype_ok(dtype) && B > 0 && H > 0 && I > 0) {
        pl.add(dh1, (size_t)B * H); pl.add(dh0, (size_t)B * H); pl.add(dx0, (size_t)B * I); pl.add(db1, (size_t)4 * H);
        pl.add(db0, (size_t)4 * H); pl.add(dWx1, (size_t)H); pl.add(dWx0, (size_t)I); pl.add(dx1, (size_t)B * H);
    }
    return finish_recurrent(bwd_stack2_impl(dout, dh1, dc1, ifgo1, cell1, d_ifgo1, Wh1, Wx1, out1, dWx1, dWh1, db1, dx1, dh0, dc0,
                                            ifgo0, cell0, d_ifgo0, Wh0, Wx0, x, out0, dx0, dWx0, dWh0, db0, ws, ws_bytes,
                                            wgrad_ws, wgrad_ws_bytes, T, B, I, H, dtype, stream),
                            ws, stream, pl);
}

int fastlstm_recurrent_kernel_kind(int T, int B, int H, int dtype, int backward, size_t ws_bytes) {
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (T <= 0 || B <= 0 || H <= 0) return FASTLSTM_ERR_DIM;
    {
        fastlstm_plan pl;
        if (plan_device(-1, B, H, dtype, backward, &pl, false) == FASTLSTM_OK && pl.wave_split == 3) return 3;
    }
    XcdCfg c;
    if (select_xcd(T, B, H, dtype, backward != 0, ws_bytes, &c)) return 1;
    WideCfg w;
    if (select_wide(T, B, H, dtype, backward != 0, ws_bytes, &w)) return 2;
    if (xcd_rows_per_launch(T, B, H, dtype, backward != 0, ws_bytes)) return 1;
    return wide_rows_per_launch(T, B, H, dtype, backward != 0, ws_bytes) ? 2 : 0;
}

int fastlstm_recurrent_rows_per_launch(int T, int B, int H, int dtype, int backward, size_t ws_bytes) {
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (T <= 0 || B <= 0 || H <= 0) return FASTLSTM_ERR_DIM;
    {
        fastlstm_plan pl;
        if (plan_device(-1, B, H, dtype, backward, &pl, false) == FASTLSTM_OK && pl.wave_split == 3) return 0;
    }
    XcdCfg c;
    WideCfg w;
    if (select_xcd(T, B, H, dtype, backward != 0, ws_bytes, &c) || select_wide(T, B, H, dtype, backward != 0, ws_bytes, &w)) return 0;
    if (const int rows = xcd_rows_per_launch(T, B, H, dtype, backward != 0, ws_bytes)) return rows;
    return wide_rows_per_launch(T, B, H, dtype, backward != 0, ws_bytes);
}

int fastlstm_ws_status(const void *ws_head) {
    if (!ws_head) return FASTLSTM_ERR_NULL;
    const WsHeader *h = static_cast<const WsHeader *>(ws_head);
    return h->abort_flag ? FASTLSTM_ERR_TIMEOUT : FASTLSTM_OK;
}

int fastlstm_prepare_forward(void *ws, size_t zero_bytes, void *out0, void *cell0, const void *h0, const void *c0,
                             int B, int H, int dtype, void *stream) {
    if (!ws || !out0 || !cell0 || (h0 == nullptr) != (c0 == nullptr)) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (B <= 0 || H <= 0) return FASTLSTM_ERR_DIM;
    const int esz = elem_bytes(dtype);
    const size_t align = (size_t)esz - 1;
    if (!aligned16(ws) || zero_bytes % 4 || ((reinterpret_cast<size_t>(out0) | reinterpret_cast<size_t>(cell0) |
                                             reinterpret_cast<size_t>(h0) | reinterpret_cast<size_t>(c0)) & align))
        return FASTLSTM_ERR_ALIGN;
    const size_t n = (size_t)B * H;
    const int blocks = (int)std::min<size_t>(1024, (std::max(n, zero_bytes / 4) + 255) / 256);
    prepare_forward_kernel<<<blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<unsigned *>(ws), zero_bytes / 4, static_cast<unsigned char *>(out0), static_cast<unsigned char *>(cell0),
        static_cast<const unsigned char *>(h0), static_cast<const unsigned char *>(c0), n, esz);
    return hipGetLastError() == hipSuccess ? FASTLSTM_OK : FASTLSTM_ERR_HIP;
}

int fastlstm_device_status(int device, int clear) {
    if (fastlstm::g_status_words.load() == 0) return FASTLSTM_OK;
    DeviceInfo di;
    if (int rc = device_info(device, &di)) return rc;
    if (!di.status_host || __atomic_load_n(di.status_host, __ATOMIC_RELAXED) == 0) return FASTLSTM_OK;
    if (clear) __atomic_store_n(di.status_host, 0, __ATOMIC_RELAXED);
    return FASTLSTM_ERR_TIMEOUT;
}

void fastlstm_set_gemm_baseline(int on) { fastlstm::set_gemm_baseline(on); }
void fastlstm_set_kernel_families(int mask) { fastlstm::g_families.store(mask & 7); }
int fastlstm_get_kernel_families(void) { return fastlstm::g_families.load(); }

void fastlstm_set_spin_limit(long long ticks) {
    if (ticks > 0) fastlstm::g_spin_limit.store(ticks);
}

const char *fastlstm_strerror(int status) {
    switch (status) {
        case FASTLSTM_OK: return "ok";
        case FASTLSTM_ERR_NULL: return "a required pointer is NULL";
        case FASTLSTM_ERR_DIM: return "a dimension is non-positive or too large";
        case FASTLSTM_ERR_DTYPE: return "unsupported dtype (0 = fp32, 1 = fp16, 2 = bf16)";
        case FASTLSTM_ERR_ALIGN: return "a pointer is not 16-byte aligned";
        case FASTLSTM_ERR_RESIDENCY:
            return "the barrier group cannot be co-resident on this device (hidden size beyond 64 units per compute unit, "
                   "or fewer compute units than the plan assumes)";
        case FASTLSTM_ERR_WORKSPACE: return "workspace is smaller than required";
        case FASTLSTM_ERR_HIP: return "a HIP runtime call failed";
        case FASTLSTM_ERR_TIMEOUT:
            return "a recurrent launch on this device gave up a barrier wait or found a workgroup on the wrong XCD "
                   "(the results of that call are invalid)";
        default: return "unknown status";
    }
}

void fastlstm_set_gemm_trace(void *buf) { set_gemm_trace(static_cast<long long *>(buf)); }
void fastlstm_set_recurrent_trace(void *buf) { fastlstm::g_rec_trace = static_cast<long long *>(buf); }

const char *fastlstm_version(void) { return "fastlstm_hip 0.1 (gfx950)"; }

}  // extern "C"

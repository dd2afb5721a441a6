// extern "C" entry points of libfastlstm_hip.so (declared in include/fastlstm_hip.h).
// Every function validates its arguments before the first HIP call.
#include <atomic>

#include "gemm.hpp"
#include "internal.hpp"
#include "recurrent_bwd.hpp"
#include "recurrent_fwd.hpp"

using namespace fastlstm;

namespace fastlstm {

static long long *g_rec_trace = nullptr;
static std::atomic<long long> g_spin_limit{400000000ll};  // 4 s of the 100 MHz clock
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
};

int device_info(int device, DeviceInfo *out) {
    static DeviceInfo cache[64];
    if (device < 0) {
        if (hipGetDevice(&device) != hipSuccess) return FASTLSTM_ERR_HIP;
    }
    if (device >= 64) return FASTLSTM_ERR_HIP;
    if (cache[device].num_cus == 0) {
        int cus = 0, lds = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
            hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess)
            return FASTLSTM_ERR_HIP;
        cache[device].lds = lds;
        cache[device].num_cus = cus;
    }
    *out = cache[device];
    return FASTLSTM_OK;
}

typedef hipError_t (*FwdLauncher)(const FwdParams &, int, int, int, int, int, hipStream_t, int *);
typedef hipError_t (*BwdLauncher)(const BwdParams &, int, int, int, int, int, hipStream_t, int *);
FwdLauncher fwd_launcher(int dtype) {
    return dtype == FASTLSTM_FP32 ? launch_fwd_f32 : (dtype == FASTLSTM_FP16 ? launch_fwd_f16 : launch_fwd_bf16);
}
BwdLauncher bwd_launcher(int dtype) {
    return dtype == FASTLSTM_FP32 ? launch_bwd_f32 : (dtype == FASTLSTM_FP16 ? launch_bwd_f16 : launch_bwd_bf16);
}

}  // namespace
}  // namespace fastlstm

extern "C" {

int fastlstm_plan_device(int device, int B, int H, int dtype, int backward, fastlstm_plan *plan) {
    if (!plan) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (B <= 0 || H <= 0) return FASTLSTM_ERR_DIM;
    DeviceInfo di;
    int rc = device_info(device, &di);
    if (rc) return rc;
    return fastlstm_plan_for(di.num_cus, di.lds, B, H, dtype, backward, plan);
}

int fastlstm_gemm_ifgo(const void *x, const void *Wx, const void *bx, const void *bh, void *ifgo, int T,
                       int B, int I, int H, int dtype, void *stream) {
    if (!x || !Wx || !bx || !bh || !ifgo) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(x) || !aligned16(Wx) || !aligned16(ifgo)) return FASTLSTM_ERR_ALIGN;
    GemmParams p{};
    p.A = x; p.B = Wx; p.C = ifgo; p.bias0 = bx; p.bias1 = bh;
    p.M = T * B; p.N = 4 * H; p.K = I;
    p.lda = I; p.ldb = I; p.ldc = 4 * H;
    p.splits = 1; p.k_per_split = I;
    int tile, splits;
    gemm_plan(dtype, p.M, p.N, p.K, p.lda, p.ldb, false, false, false, &tile, &splits);
    return launch_gemm_tiled(dtype, p, false, false, tile, static_cast<hipStream_t>(stream)) == hipSuccess
               ? FASTLSTM_OK
               : FASTLSTM_ERR_HIP;
}

int fastlstm_gemm_dx(const void *d_ifgo, const void *Wx, void *dx, int T, int B, int I, int H, int dtype,
                     void *stream) {
    if (!d_ifgo || !Wx || !dx) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, I, H)) return rc;
    if (!aligned16(d_ifgo) || !aligned16(Wx) || !aligned16(dx)) return FASTLSTM_ERR_ALIGN;
    GemmParams p{};
    p.A = d_ifgo; p.B = Wx; p.C = dx;
    p.M = T * B; p.N = I; p.K = 4 * H;
    p.lda = 4 * H; p.ldb = I; p.ldc = I;
    p.splits = 1; p.k_per_split = 4 * H;
    int tile, splits;
    gemm_plan(dtype, p.M, p.N, p.K, p.lda, p.ldb, false, true, false, &tile, &splits);
    return launch_gemm_tiled(dtype, p, false, true, tile, static_cast<hipStream_t>(stream)) == hipSuccess
               ? FASTLSTM_OK
               : FASTLSTM_ERR_HIP;
}

// tile and split-K factor of a weight-gradient product C[M,N] = A^T.B with reduction length K
static void wgrad_plan(int M, int N, int K, int dtype, int *tile, int *splits, int *k_per_split) {
    gemm_plan(dtype, M, N, K, M, N, true, true, true, tile, splits);
    const int bk = *tile ? 64 : gemm_bk(dtype);
    *k_per_split = cdiv(cdiv(K, *splits), bk) * bk;
    *splits = cdiv(K, *k_per_split);
}
static int colsum_chunks(int R) { return std::max(1, std::min(64, R / 64)); }

size_t fastlstm_wgrad_workspace_bytes(int T, int B, int I, int H, int dtype) {
    if (!dtype_ok(dtype) || check_dims(T, B, I, H)) return 0;
    const int K = T * B, M = 4 * H;
    int tile, sx, sh, kps;
    wgrad_plan(M, I, K, dtype, &tile, &sx, &kps);
    wgrad_plan(M, H, K, dtype, &tile, &sh, &kps);
    size_t part = std::max(sx > 1 ? (size_t)sx * M * I : 0, sh > 1 ? (size_t)sh * M * H : 0) * sizeof(float);
    size_t cs = (size_t)colsum_chunks(K) * M * sizeof(float);
    return align_up(cs, 256) + align_up(part, 256) + 256;
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

int fastlstm_fwd_persistent(void *ifgo, void *out, void *cell, const void *Wh, void *ws, size_t ws_bytes,
                            int T, int B, int H, int dtype, void *stream) {
    if (!ifgo || !out || !cell || !Wh || !ws) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    if (!aligned16(ifgo) || !aligned16(out) || !aligned16(cell) || !aligned16(Wh) || !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    fastlstm_plan pl;
    if (int rc = fastlstm_plan_device(-1, B, H, dtype, 0, &pl)) return rc;
    if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
    const bool sync = pl.wave_split != 2;
    const int kstep = dtype == FASTLSTM_FP32 ? 16 : 32;
    unsigned char *wsb = static_cast<unsigned char *>(ws);
    FwdParams p{};
    p.ifgo = ifgo; p.out = out; p.cell = cell; p.Wh = Wh;
    p.hdr = reinterpret_cast<WsHeader *>(wsb);
    p.T = T; p.B = B; p.H = H;
    p.n_ht = pl.n_htiles;
    p.flag_stride = (int)align_up((size_t)pl.n_htiles, 64);
    p.KS = cdiv(H, kstep);
    p.spin_limit = spin_limit_ticks();
    p.trace = g_rec_trace;
    const int n_bt_total = cdiv(B, pl.bt);
    const size_t flags_bytes = recurrent_flags_bytes(pl.n_btiles, pl.n_htiles);
    const size_t slot_bytes = recurrent_slot_bytes(H, dtype, pl.bt, pl.n_btiles, false);
    if (sync) {  // as many ring slots as the workspace holds, up to one per version
        const int full = recurrent_full_slots(T, slot_bytes, false);
        const size_t avail = (ws_bytes - pl.ws_zero_bytes) / pl.batch_chunks / slot_bytes;
        p.n_slots = (int)std::min<size_t>(full, avail);
        // cached loads need a never-reused slot per version and 128-byte lines written by one
        // workgroup only (16-bit tiles of 4 units share their lines with the neighbour tile)
        p.coherent_loads = (p.n_slots < T + 1 || (dtype != FASTLSTM_FP32 && pl.ht == 4)) ? 1 : 0;
    }
    // coalesced tile I/O needs complete, 16-byte aligned row segments and room in LDS
    int lds_bytes = pl.lds_bytes;
    {
        const int s = elem_bytes(dtype), gseg = pl.ht * s;
        const int tile_bytes = (pl.bt * (4 * gseg + 16) + 2 * pl.bt * (gseg + 16)) * (sync ? 1 : 2);
        p.vec_io = (gseg >= 16 && (H * s) % 16 == 0 && H % pl.ht == 0 && lds_bytes + tile_bytes <= pl.lds_limit) ? 1 : 0;
        if (p.vec_io) lds_bytes += tile_bytes;
#ifdef FASTLSTM_TIMELINE
        lds_bytes += 4096;   // room for the diagnostic time stamps of the kernel
#endif
    }
    // K-split kernels keep the slice in registers when a wave's share is at most 32 fragments
    if (pl.wave_split == 0) {
        const int nkw = cdiv(p.KS, 4) <= 4 ? 4 : (cdiv(p.KS, 4) <= 8 ? 8 : 0);
        if (nkw && (pl.ht / 4) * nkw <= 32) p.w_regs = nkw;
    }
    FwdLauncher launch = fwd_launcher(dtype);
    for (int c = 0, bt0 = 0; bt0 < n_bt_total; ++c, bt0 += pl.n_btiles) {
        const int n_bt = std::min(pl.n_btiles, n_bt_total - bt0);
        p.flags = reinterpret_cast<int *>(wsb + 1024 + (size_t)c * flags_bytes);
        p.xbuf = wsb + pl.ws_zero_bytes + (size_t)c * p.n_slots * slot_bytes;
        p.n_bt = pl.n_btiles;  // exchange-slot stride is sized for a full launch
        p.b_base = bt0 * pl.bt;
        const int grid = n_bt * pl.n_htiles;
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
    if (!dout || !dh || !dc || !ifgo || !cell || !d_ifgo || !Wh || !ws) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (int rc = check_dims(T, B, H, H)) return rc;
    if (!aligned16(dout) || !aligned16(dh) || !aligned16(dc) || !aligned16(ifgo) || !aligned16(cell) ||
        !aligned16(d_ifgo) || !aligned16(Wh) || !aligned16(ws))
        return FASTLSTM_ERR_ALIGN;
    fastlstm_plan pl;
    if (int rc = fastlstm_plan_device(-1, B, H, dtype, 1, &pl)) return rc;
    if (ws_bytes < pl.ws_bytes) return FASTLSTM_ERR_WORKSPACE;
    const bool sync = pl.wave_split != 2;
    const int kstep = dtype == FASTLSTM_FP32 ? 16 : 32;
    unsigned char *wsb = static_cast<unsigned char *>(ws);
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
    const int n_bt_total = cdiv(B, pl.bt);
    const size_t flags_bytes = recurrent_flags_bytes(pl.n_btiles, pl.n_htiles);
    const size_t slot_bytes = recurrent_slot_bytes(H, dtype, pl.bt, pl.n_btiles, true);
    if (sync) {
        const int full = recurrent_full_slots(T, slot_bytes, true);
        const size_t avail = (ws_bytes - pl.ws_zero_bytes) / pl.batch_chunks / slot_bytes;
        p.n_slots = (int)std::min<size_t>(full, avail);
        p.coherent_loads = p.n_slots < T ? 1 : 0;
    }
    // coalesced tile I/O needs complete, 16-byte aligned row segments and room in LDS
    int lds_bytes = pl.lds_bytes;
    {
        const int s = elem_bytes(dtype), gseg = pl.ht * s;
        const int tile_bytes = (pl.bt * (4 * gseg + 16) + 2 * pl.bt * (gseg + 16)) * (sync ? 1 : 2);
        p.vec_io = (gseg >= 16 && (H * s) % 16 == 0 && H % pl.ht == 0 && lds_bytes + tile_bytes <= pl.lds_limit) ? 1 : 0;
        if (p.vec_io) lds_bytes += tile_bytes;
    }
    BwdLauncher launch = bwd_launcher(dtype);
    for (int c = 0, bt0 = 0; bt0 < n_bt_total; ++c, bt0 += pl.n_btiles) {
        const int n_bt = std::min(pl.n_btiles, n_bt_total - bt0);
        p.flags = reinterpret_cast<int *>(wsb + 1024 + (size_t)c * flags_bytes);
        p.xbuf = wsb + pl.ws_zero_bytes + (size_t)c * p.n_slots * slot_bytes;
        p.n_bt = pl.n_btiles;
        p.b_base = bt0 * pl.bt;
        const int grid = n_bt * pl.n_htiles;
        int occ = 0;
        if (launch(p, pl.ht, pl.bt, pl.wave_split, 0, lds_bytes, nullptr, &occ) != hipSuccess) return FASTLSTM_ERR_HIP;
        if (sync && (long long)occ * pl.num_cus < grid) return FASTLSTM_ERR_RESIDENCY;
        if (launch(p, pl.ht, pl.bt, pl.wave_split, grid, lds_bytes, static_cast<hipStream_t>(stream), nullptr) !=
            hipSuccess)
            return FASTLSTM_ERR_HIP;
    }
    return FASTLSTM_OK;
}

int fastlstm_ws_status(const void *ws_head) {
    if (!ws_head) return FASTLSTM_ERR_NULL;
    const WsHeader *h = static_cast<const WsHeader *>(ws_head);
    return h->abort_flag ? FASTLSTM_ERR_TIMEOUT : FASTLSTM_OK;
}

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
            return "the W_h slice does not fit in LDS or the barrier group cannot be co-resident";
        case FASTLSTM_ERR_WORKSPACE: return "workspace is smaller than required";
        case FASTLSTM_ERR_HIP: return "a HIP runtime call failed";
        case FASTLSTM_ERR_TIMEOUT: return "a barrier wait timed out (results are invalid)";
        default: return "unknown status";
    }
}

void fastlstm_set_gemm_trace(void *buf) { set_gemm_trace(static_cast<long long *>(buf)); }
void fastlstm_set_recurrent_trace(void *buf) { fastlstm::g_rec_trace = static_cast<long long *>(buf); }

const char *fastlstm_version(void) { return "fastlstm_hip 0.1 (gfx950)"; }

}  // extern "C"

// Host-only tiling rule for the two recurrent kernels (no HIP calls here, so
// the rule is unit-testable without a GPU).
//
// What it decides, per (B, H, dtype, direction):
//   bt x ht        batch rows x hidden units one workgroup owns,
//   n_htiles       workgroups that must exchange data every step (barrier group),
//   n_btiles       independent barrier groups per launch,
//   batch_chunks   sequential launches when the batch does not fit,
//   wave_split     how the 4 waves of a workgroup divide the per-step product.
// Constraints: the weight slice stays resident in LDS for the whole sequence and
// n_btiles * n_htiles <= num_cus, i.e. every workgroup of a barrier group is
// resident while the others spin -- the co-residency rule of the reference,
// fastlstm/configs.py:29-58 (grid <= SM count, halve the batch tiles and loop
// otherwise) with its autotune search (configs.py:146-304) replaced by a small
// cost model over a fixed menu of tiles.
#include <string.h>

#include <algorithm>

#include "internal.hpp"

namespace fastlstm {

namespace {

struct Cand {
    int bt, ht, n_ht, n_bt_total, n_bt, chunks, split, lds;
    double cost;
};

constexpr int kNoSyncMaxH = 64;  // whole W_h on one CU, barrier compiled out

int kstep_of(int dtype) { return dtype == FASTLSTM_FP32 ? 16 : 32; }

}  // namespace

// LDS request of the forward kernel for a tile choice.
int fwd_lds_bytes(int H, int dtype, int ht, int bt, int split, bool sync) {
    const int KS = cdiv(H, kstep_of(dtype));
    const int MT = cdiv(ht, 4), NT = bt / 16;
    const int P = (split == 0) ? 4 : 1;
    int lds = MT * KS * kFragBytes + kFragBytes;  // resident W_h slice + one all-zero operand block
    lds += P * MT * NT * kFragBytes;       // cross-wave reduction / re-layout buffer
    if (!sync) lds += 2 * NT * KS * kFragBytes;  // h exchange stays in LDS
    return lds;
}

// LDS request of the backward kernel.  K runs over (unit, gate) pairs: 4H.
int bwd_lds_bytes(int H, int dtype, int ht, int bt, int split, bool sync) {
    const int KSB = cdiv(4 * H, kstep_of(dtype));
    const int NT = bt / 16;
    const int P = (split == 0) ? 4 : 1;
    int lds;
    if (sync) {
        lds = KSB * ht * 64 + kFragBytes;  // [kstep][lane group][ht rows][16 B] + all-zero block
        lds += P * NT * kFragBytes;
    } else {
        (void)ht;  // the barrier-free kernel always reserves 4 unit tiles (64 units)
        lds = 4 * KSB * kFragBytes + kFragBytes + 4 * NT * kFragBytes + 2 * NT * KSB * kFragBytes;
    }
    return lds;
}

// Workspace layout: header (1 KiB) | L2 barrier counters (64 KiB) | flags of every batch chunk |
// exchange ring of every chunk.  Without a cross-CU barrier: the header only.
size_t recurrent_flags_bytes(int n_bt, int n_ht) {
    return align_up((size_t)n_bt * align_up((size_t)n_ht, 64) * sizeof(int), 1024);
}
// One ring slot = the exchange data of one timestep of one launch.
size_t recurrent_slot_bytes(int H, int dtype, int bt, int n_bt, bool backward) {
    const int KS = backward ? cdiv(4 * H, kstep_of(dtype)) : cdiv(H, kstep_of(dtype));
    return (size_t)n_bt * (bt / 16) * KS * kFragBytes;
}
size_t recurrent_ws_bytes(int H, int dtype, int bt, int n_bt, int n_ht, int chunks, bool backward, bool sync,
                          int slots) {
    if (!sync) return kWsHeaderBytes;
    return kWsHeaderBytes + kWsCounterBytes + (size_t)chunks * (recurrent_flags_bytes(n_bt, n_ht) +
                                  (size_t)slots * recurrent_slot_bytes(H, dtype, bt, n_bt, backward));
}

// k-steps are padded to the granule of the streamed K loop (4 waves x 2 chunks x 2 k-steps)
constexpr int kStreamKPadHost = 16;

StreamLayout stream_layout(const fastlstm_plan &plan, int H, int dtype, bool backward) {
    StreamLayout l;
    l.KS = cdiv(backward ? 4 * H : H, kstep_of(dtype));
    l.KSP = cdiv(l.KS, kStreamKPadHost) * kStreamKPadHost;
    l.mt = backward ? plan.ht / 16 : plan.ht / 4;
    l.flags_bytes = recurrent_flags_bytes(plan.n_btiles, plan.n_htiles);
    l.slot_bytes = (size_t)plan.n_btiles * (plan.bt / 16) * l.KSP * kFragBytes;
    l.chunk_bytes = l.flags_bytes + 2 * l.slot_bytes;
    l.wpack_off = align_up(kWsHeaderBytes + kWsCounterBytes + (size_t)plan.batch_chunks * l.chunk_bytes, 4096);
    l.wpack_bytes = (size_t)plan.n_htiles * l.mt * l.KSP * kFragBytes;
    return l;
}

}  // namespace fastlstm

using namespace fastlstm;

extern "C" int fastlstm_plan_for(int num_cus, int lds_limit, int B, int H, int dtype, int backward,
                                 fastlstm_plan *plan) {
    if (!plan) return FASTLSTM_ERR_NULL;
    if (!dtype_ok(dtype)) return FASTLSTM_ERR_DTYPE;
    if (B <= 0 || H <= 0 || num_cus <= 0 || lds_limit <= 0) return FASTLSTM_ERR_DIM;
    if ((long long)B * H > (1ll << 31) / 8 || H > (1 << 20)) return FASTLSTM_ERR_DIM;
    memset(plan, 0, sizeof(*plan));
    plan->num_cus = num_cus;
    plan->lds_limit = lds_limit;
    const int s = elem_bytes(dtype);
    const int KSTEP = kstep_of(dtype);
    const double cyc_kstep = dtype == FASTLSTM_FP32 ? 128.0 : 16.0;

    if (H <= kNoSyncMaxH) {
        // one workgroup holds all of W_h: batch tiles are fully independent, any
        // grid size is legal, waves split the W rows (forward) / unit tiles (backward)
        int ht;
        if (!backward) {
            int mtw = cdiv(cdiv(H, 4), 4);       // m-tiles per wave
            mtw = mtw <= 1 ? 1 : (mtw <= 2 ? 2 : 4);
            ht = 16 * mtw;                       // 4 waves x mtw tiles x 4 units
        } else {
            ht = 64;
        }
        const int lds = backward ? bwd_lds_bytes(H, dtype, ht, 16, 2, false)
                                 : fwd_lds_bytes(H, dtype, ht, 16, 2, false);
        if (lds > lds_limit) return FASTLSTM_ERR_RESIDENCY;
        plan->bt = 16;
        plan->ht = ht;
        plan->n_btiles = cdiv(B, 16);
        plan->n_htiles = 1;
        plan->batch_chunks = 1;
        plan->wave_split = 2;
        plan->lds_bytes = lds;
        plan->ws_bytes = recurrent_ws_bytes(H, dtype, 16, plan->n_btiles, 1, 1, backward != 0, false, 2);
        plan->ws_zero_bytes = plan->ws_bytes;
        plan->ring_needs_zero = 0;
        return FASTLSTM_OK;
    }

    const int K = backward ? 4 * H : H;
    const int KS = cdiv(K, KSTEP);
    Cand best;
    best.cost = -1;
    const int hts[3] = {4, 8, 16};
    const int bts[4] = {16, 32, 64, 128};
    for (int hi = 0; hi < 3; ++hi)
        for (int bi = 0; bi < 4; ++bi) {
            Cand c;
            c.ht = hts[hi];
            c.bt = bts[bi];
            if (bi > 0 && bts[bi - 1] >= B) continue;  // a smaller tile already covers B
            c.n_ht = cdiv(H, c.ht);
            if (c.n_ht > num_cus || c.n_ht > 1024) continue;
            c.n_bt_total = cdiv(B, c.bt);
            c.n_bt = std::min(c.n_bt_total, num_cus / c.n_ht);
            c.chunks = cdiv(c.n_bt_total, c.n_bt);
            const int NT = c.bt / 16;
            c.split = NT >= 4 ? 1 : 0;
            c.lds = backward ? bwd_lds_bytes(H, dtype, c.ht, c.bt, c.split, true)
                             : fwd_lds_bytes(H, dtype, c.ht, c.bt, c.split, true);
            if (c.lds > lds_limit) continue;
            // per-step time model, in shader cycles (2.4 GHz) + ns of barrier latency
            const double mtiles = backward ? 1.0 : c.ht / 4.0;
            const double wbytes = backward ? (double)KS * c.ht * 64 : mtiles * KS * kFragBytes;
            double t_mfma, t_lds;
            if (c.split == 0) {
                t_mfma = mtiles * NT * cdiv(KS, 4) * cyc_kstep;
                t_lds = wbytes / 128.0;
            } else {
                t_mfma = mtiles * (NT / 4) * KS * cyc_kstep;
                t_lds = 4.0 * wbytes / 128.0;
            }
            const double t_load = (double)c.bt * KS * KSTEP * s / 64.0;
            const double items = (double)c.bt * c.ht / kThreads;
            const double t_epi = 400.0 + 250.0 * std::max(1.0, items);
            const double sync_ns = 2500.0 + 6.0 * c.n_ht;
            const double step_ns = (std::max(t_mfma, std::max(t_lds, t_load)) + t_epi) / 2.4 + sync_ns;
            c.cost = step_ns * c.chunks;
            if (best.cost < 0 || c.cost < best.cost) best = c;
        }
    if (best.cost < 0) {
        // No tiling keeps the weight slices on chip: stream them every step (wave_split 3, recurrent_stream.hpp).
        // One workgroup per slice of ht units and as many batch rows as its accumulators hold, so that the
        // weights cross the memory system once per step; ht is the smallest slice that leaves the barrier group
        // co-resident.
        int ht = 0;
        for (int cand : {16, 32, 64})
            if (!ht && cdiv(H, cand) <= num_cus) ht = cand;
        if (!ht) return FASTLSTM_ERR_RESIDENCY;   // H > 64 * num_cus
        const int nt_max = 4 / (ht / 16);
        int nt = 1;
        while (nt < nt_max && nt * 16 < B) nt *= 2;
        plan->ht = ht;
        plan->bt = 16 * nt;
        plan->n_htiles = cdiv(H, ht);
        const int n_bt_total = cdiv(B, plan->bt);
        plan->n_btiles = std::min(n_bt_total, std::max(1, num_cus / plan->n_htiles));
        plan->batch_chunks = cdiv(n_bt_total, plan->n_btiles);
        plan->wave_split = 3;
        plan->lds_bytes = 4 * (backward ? ht / 16 : ht / 4) * nt * kFragBytes;   // the 4 waves' partial sums
        const StreamLayout l = stream_layout(*plan, H, dtype, backward != 0);
        plan->ws_bytes = l.wpack_off + l.wpack_bytes;
        plan->ws_zero_bytes = l.wpack_off;   // header, counters, flags and the (small) exchange slots
        plan->ring_needs_zero = 0;
        return FASTLSTM_OK;
    }
    plan->bt = best.bt;
    plan->ht = best.ht;
    plan->n_btiles = best.n_bt;
    plan->n_htiles = best.n_ht;
    plan->batch_chunks = best.chunks;
    plan->wave_split = best.split;
    plan->lds_bytes = best.lds;
    plan->ws_bytes = recurrent_ws_bytes(H, dtype, best.bt, best.n_bt, best.n_ht, best.chunks, backward != 0, true, 2);
    plan->ws_zero_bytes = kWsHeaderBytes + kWsCounterBytes + (size_t)best.chunks * recurrent_flags_bytes(best.n_bt, best.n_ht);
    plan->ring_needs_zero = (B % 16 != 0 || K % KSTEP != 0) ? 1 : 0;
    return FASTLSTM_OK;
}

extern "C" size_t fastlstm_recurrent_workspace_bytes(const fastlstm_plan *plan, int T, int H, int dtype, int backward) {
    if (!plan || T <= 0 || H <= 0 || !dtype_ok(dtype)) return 0;
    if (plan->wave_split == 2 || plan->wave_split == 3) return plan->ws_bytes;
    const size_t slot = recurrent_slot_bytes(H, dtype, plan->bt, plan->n_btiles, backward != 0);
    const int slots = 2;   // every kernel exchanges through two slots, whatever T is
    size_t ws = plan->ws_bytes;
    // the XCD-local kernels lay their ring out for batch tiles of 16 or 32 rows, which covers at most
    // 16 rows (one operand block per k-step) more than the tiles of the plan
    // (the kernels for H = 1280 ... 2048 use tiles of 64 rows: at most 48 rows more)
    const int KS = cdiv(backward ? 4 * H : H, kstep_of(dtype));
    const int margin = (dtype != FASTLSTM_FP32 && H > 1024 && H <= 2048 && H % 256 == 0) ? 3 : 1;
    ws = std::max(ws, kWsHeaderBytes + kWsCounterBytes +
                          (size_t)slots * (plan->batch_chunks * slot + (size_t)margin * KS * kFragBytes));
    // the reverse kernel of those hidden sizes exchanges partial sums among teams of up to 8 workgroups:
    // 4 KiB per (receiver, sender), 256 workgroups
    if (backward && margin == 3) ws += (size_t)256 * 8 * 4 * kFragBytes;
    return ws;
}

// Persistent reverse-time kernel for H = 1280 ... 2048 with 16-bit elements and groups of 64 batch rows:
// lstm_bwd_wide_kernel with the product split over K as well.  Same mathematics and results as
// lstm_bwd_persistent_kernel (which replaces fastlstm/kernels.py:1201-1409); the sums over K are taken in
// another order.
//
// In lstm_bwd_wide_kernel a workgroup owns 16 units and all of K = 4H, so each of the H / 16 workgroups of a
// group reads the whole d_ifgo[t] of the group's rows every step (1 MiB at H = 2048): the step is bound by
// what the L2 of an XCD can deliver to its 32 CUs (14.4 us).  Here V neighbouring workgroups form a team
// that owns 16 V units; member m keeps the weights of ALL the team's units for the m-th part of K in
// registers (the same 256 KiB per workgroup) and so reads 1 / V of d_ifgo[t].  Its products are partial sums
// for the whole team: after the multiplication it sends the other members theirs (fp32, 16 units x 64 rows
// each) through the workspace, raises a team flag, waits for the V - 1 others and adds what they sent in
// member order.  Per step and workgroup at H = 2048, V = 4: 256 KiB of operand blocks and 12 KiB of partial
// sums each way instead of 1 MiB, for one more flag round trip among V workgroups of the same XCD.
//
// The 8 waves split the member's part of K and keep the sums of all 4 V output tiles (V unit tiles x 4 batch
// tiles) in registers; after the last operand block they add them up through LDS, 4 V / 8 tiles per wave (the
// 16 KiB per wave land where the operand ring was).  Operand blocks travel L2 -> ring in LDS with LDS-direct
// loads as in lstm_bwd_wide_kernel.  Loads and ring reads are inline assembly, with the wave counting its own
// loads (s_waitcnt vmcnt(n)): the compiler would wait for every LDS-direct load it knows of before an LDS access.
#pragma once
#include <type_traits>

#include "recurrent_bwd_wide.hpp"

namespace fastlstm {

constexpr int kSplitRing = 8;   // LDS blocks (1 KiB) per wave for operand blocks in flight

// number of k-steps per wave over the whole of K: NKW = 4H / KSTEP / 8 (20, 24, 28, 32 for H = 1280 ... 2048);
// V members per team (divides NKW and 8; the 4 V accumulator tiles must fit the registers: V <= 4)
template <typename T, int NKW, int V>
__global__ __launch_bounds__(kWave * 8) void lstm_bwd_wide_split_kernel(const BwdXcdParams p) {
    static_assert(sizeof(T) == 2, "16-bit element types");
    using E = Elem<T>;
    constexpr int NWV = 8, NTHR = kWave * NWV, NT = 4;
    constexpr int HT = 16, BT = 16 * NT;
    constexpr int IPT = HT * BT / NTHR;                // (unit, batch row) items per thread
    constexpr int GSEG = HT * E::BYTES;
    constexpr int GROW = 4 * GSEG + 16, SROW = GSEG + 16;
    constexpr int PPSEG = GSEG / 16;
    constexpr int KW = NKW / V;                        // k-steps per wave in the member's part of K
    constexpr int NB = KW * NT;                        // operand blocks per wave and step
    constexpr int TILES = NT * V;                      // output tiles of a workgroup
    constexpr int TPW = TILES / NWV;                   // ... that a wave adds up
    constexpr int S = kSplitRing < NB ? kSplitRing : NB;
    static_assert(NKW % V == 0 && NWV % V == 0 && TILES % NWV == 0 && V <= 4, "team size");
    static_assert(NB >= 4 && S >= 3, "read-ahead of two blocks");
    static_assert(TILES >= S, "the waves' sums take the place of the ring");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = lane >> 4, r = lane & 15;
    const int KSB = p.KSB, H = p.H, B = p.B, T_ = p.T;

    // ---- placement: group g on XCDs g*xpg .. (hardware deals workgroup i to XCD i % 8) --------
    const int xpg = p.gpx;
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int g = xcd / xpg, j = (xcd % xpg) * 32 + slot;
    if (g >= p.n_groups || j >= p.n_ht) return;
    check_xcd_placement(p.hdr);
    const int u0 = j * HT, b0 = p.b_base + g * BT;
    const int mem = j % V, team0 = j - mem;            // the team: workgroups team0 .. team0 + V - 1 (one XCD)

    f32x4 *own = reinterpret_cast<f32x4 *>(smem);                      // [NT][64]: this member's share of its own products
    unsigned char *tiles = reinterpret_cast<unsigned char *>(own + NT * kWave);   // gates, c, dout tiles
    f32x4 *red = reinterpret_cast<f32x4 *>(tiles + BT * GROW + 2 * BT * SROW);    // [8 waves][TILES][64], and before that
    unsigned char *ring = reinterpret_cast<unsigned char *>(red) + (size_t)wave * S * kFragBytes;   // the waves' rings
    const unsigned ring_addr = (unsigned)(size_t)((FASTLSTM_LDS_PTR unsigned char *)ring);

    const T *dout = static_cast<const T *>(p.dout);
    const T *ifgo = static_cast<const T *>(p.ifgo);
    const T *cell = static_cast<const T *>(p.cell);
    T *d_ifgo = static_cast<T *>(p.d_ifgo);
    const T *Wh = static_cast<const T *>(p.Wh);

    // ---- prologue: Wh[k-part, team units]^T, gathered from global memory ----
    // fragment (unit tile v, k-step ks = mem * 8 KW + wave + 8 ki): lane (q, r) holds row r = unit
    // team0 * 16 + 16 v + r and k = ks*KSTEP + q*EPL + e, e < EPL, with k = 4 * source unit + gate
    u32x4 wreg[V][KW];
#pragma unroll
    for (int v = 0; v < V; ++v)
#pragma unroll
        for (int ki = 0; ki < KW; ++ki) {
            const int ks = mem * NWV * KW + wave + NWV * ki;
            T tmp[E::EPL];
#pragma unroll
            for (int e = 0; e < E::EPL; ++e) {
                const int k = ks * E::KSTEP + q * E::EPL + e;
                tmp[e] = Wh[((size_t)(k & 3) * H + (k >> 2)) * H + team0 * HT + v * 16 + r];
            }
            wreg[v][ki] = *reinterpret_cast<u32x4 *>(tmp);
        }

    // ---- per-thread items: it = tid + NTHR*m -> (row n, unit ul, n-tile nt) ----------------
    float dc_state[IPT], dh_rec[IPT], c1v[IPT];
    bool valid[IPT], pair_lead[IPT];
    const size_t BH = (size_t)B * H, B4H = (size_t)B * 4 * H;
#pragma unroll
    for (int m = 0; m < IPT; ++m) {
        const int it = tid + NTHR * m;
        const int n = it & 15, rest = it >> 4;
        const int ul = rest % HT, nt = rest / HT;
        const int unit = u0 + ul, b = b0 + nt * 16 + n;
        valid[m] = b < B;
        const size_t off_h = valid[m] ? (size_t)b * H + unit : (size_t)b0 * H + u0;
        pair_lead[m] = valid[m] && ((ul & 1) == 0);
        dh_rec[m] = valid[m] ? E::to_f32(static_cast<const T *>(p.dh)[off_h]) : 0.f;
        dc_state[m] = valid[m] ? E::to_f32(static_cast<const T *>(p.dc)[off_h]) : 0.f;
        c1v[m] = valid[m] ? E::to_f32(cell[(size_t)T_ * BH + off_h]) : 0.f;
    }

    // item m is (row n, unit ul, n-tile tid / 256 + 2 m): its offsets are those of item 0 plus a constant
    static_assert(NTHR == 2 * 16 * HT, "two n-tiles per round of items");
    const int it_n = tid & 15, it_ul = (tid >> 4) % HT, it_nt = tid >> 8;
    const int xoff0 = it_nt * KSB * kFragBytes + frag_offset<T>(it_n, (u0 + it_ul) * 4);   // exchange slot
    const int roff0 = ((it_nt * kWave + (it_ul >> 2) * 16 + it_n) * 4 + (it_ul & 3)) * 4;    // its sum in a [NT][64] f32x4 tile set
    const int goff0 = (it_nt * 16 + it_n) * GROW + it_ul * E::BYTES;                        // LDS tiles
    const int soff0 = (it_nt * 16 + it_n) * SROW + it_ul * E::BYTES;
    auto xoff = [&](int m) { return xoff0 + m * 2 * KSB * kFragBytes; };
    auto roff = [&](int m) { return roff0 + m * 2 * kWave * 16; };
    auto goff = [&](int m) { return goff0 + m * 32 * GROW; };
    auto soff = [&](int m) { return soff0 + m * 32 * SROW; };
    const unsigned xgrp = (unsigned)g * NT * KSB * kFragBytes;
    const size_t xslot = (size_t)p.n_groups * NT * KSB * kFragBytes;
    int *grp_flags = p.counters + (size_t)g * kXcdGroupStride;                 // one flag per workgroup of the group
    int *team_flags = p.counters + (size_t)(kNumXcd + g) * kXcdGroupStride;   // a second one for the partial sums

    // partial sums in the workspace: [group][receiver][sender][NT][64] f32x4, one slot (a sender passes the
    // next step's group barrier only after the receiver published that step, i.e. after it read this one)
    constexpr unsigned kSetBytes = NT * kFragBytes;
    const unsigned part_bytes = (unsigned)((size_t)p.n_groups * p.n_ht * V * kSetBytes);
    const XchgGlobal part(p.partials, part_bytes);
    const unsigned part_grp = (unsigned)(((size_t)g * p.n_ht) * V * kSetBytes);
    const unsigned part_mine = part_grp + (unsigned)j * V * kSetBytes;         // what the others send to this workgroup
    // wave w adds up the tiles w + 8 i = (batch tile w / V + 8 / V * i, unit tile w % V): sums of member w % V
    const int rv = wave % V, rnt = wave / V;
    const unsigned part_to = part_grp + (unsigned)((team0 + rv) * V + mem) * kSetBytes;   // my place at that member

    // ---- tile I/O: ifgo[t], cell[t], dout[t] come in with LDS-direct loads (no register holds them), issued by
    // waves 1..7 while wave 0 polls the team's flags; d_ifgo[t] leaves with buffer stores.  A tile row is a whole
    // number of 16-byte slots, the last one padding: lane l of wave instruction i of a tile fills slot 64 i + l;
    // pad slots and rows past B stay untouched (lanes switched off).  The same (instruction, lane) -> slot map
    // drains the gates tile.
    constexpr int SPRG = GROW / 16, SPRS = SROW / 16;                                          // slots per tile row
    constexpr int NG = (BT * SPRG + kWave - 1) / kWave, NS = (BT * SPRS + kWave - 1) / kWave;   // wave instructions per tile
    constexpr int DT = (NG + 2 * NS + NWV - 2) / (NWV - 1);                                     // per moving wave
    unsigned g_off[DT];
    int g_kind[DT];   // tile of item d (0 gates, 1 c, 2 dout; the same in all lanes)
    bool g_ok[DT];
    const size_t tile_org = (size_t)b0 * 4 * H + u0, state_org = (size_t)b0 * H + u0;
    const unsigned g_bytes = (unsigned)((size_t)BT * 4 * H * E::BYTES), s_bytes = (unsigned)((size_t)BT * H * E::BYTES);
#pragma unroll
    for (int i = 0; i < DT; ++i) {
        const int w = (wave - 1) + (NWV - 1) * i;
        g_kind[i] = w < NG ? 0 : (w < NG + NS ? 1 : 2);
        const int wi = w < NG ? w : (w < NG + NS ? w - NG : w - NG - NS), sl = wi * kWave + lane;
        if (g_kind[i] == 0) {
            const int row = sl / SPRG, idx = sl % SPRG;
            g_ok[i] = wave >= 1 && sl < BT * SPRG && idx < 4 * PPSEG && b0 + row < B;
            g_off[i] = g_ok[i] ? (unsigned)(((size_t)row * 4 * H + (size_t)(idx / PPSEG) * H + (idx % PPSEG) * (16 / E::BYTES)) * E::BYTES) : 0u;
        } else {
            const int row = sl / SPRS, idx = sl % SPRS;
            g_ok[i] = wave >= 1 && w < NG + 2 * NS && sl < BT * SPRS && idx < PPSEG && b0 + row < B;
            g_off[i] = g_ok[i] ? (unsigned)(((size_t)row * H + idx * (16 / E::BYTES)) * E::BYTES) : 0u;
        }
    }
    const unsigned tiles_addr = (unsigned)(size_t)((FASTLSTM_LDS_PTR unsigned char *)tiles);
    auto rsrc_of = [](const T *base, unsigned bytes) {
        const unsigned long long a = reinterpret_cast<unsigned long long>(base);
        return u32x4{(unsigned)a, (unsigned)(a >> 32) & 0xffffu, bytes, 0x00020000u};
    };
    auto request_tiles = [&](int t) {   // (the wave waits for them itself: s_waitcnt vmcnt(0) at the end of the step)
        const u32x4 rg = rsrc_of(ifgo + (size_t)t * B4H + tile_org, g_bytes);
        const u32x4 rc = rsrc_of(cell + (size_t)t * BH + state_org, s_bytes);
        const u32x4 rd = rsrc_of(dout + (size_t)t * BH + state_org, s_bytes);
#pragma unroll
        for (int i = 0; i < DT; ++i) {
            const int w = (wave - 1) + (NWV - 1) * i;
            if (g_kind[i] == 0) {
                if (g_ok[i]) dma_block_asm<false>(rg, tiles_addr + w * kFragBytes, g_off[i], 0u);
            } else if (g_kind[i] == 1) {
                if (g_ok[i]) dma_block_asm<false>(rc, tiles_addr + BT * GROW + (w - NG) * kFragBytes, g_off[i], 0u);
            } else {
                if (g_ok[i]) dma_block_asm<false>(rd, tiles_addr + BT * GROW + BT * SROW + (w - NG - NS) * kFragBytes, g_off[i], 0u);
            }
        }
    };
    auto tile_to_global = [&](int t) {
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(d_ifgo + (size_t)t * B4H + tile_org, 0, g_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < DT; ++i)
            if (g_kind[i] == 0 && g_ok[i])
                __builtin_amdgcn_raw_buffer_store_b128(
                    *reinterpret_cast<const u32x4 *>(tiles + (size_t)((wave - 1) + (NWV - 1) * i) * kFragBytes + lane * 16), rg, g_off[i], 0, 0);
    };
    request_tiles(T_ - 1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    const unsigned lane_off = (unsigned)lane * 16u;
    const unsigned ks_base = (unsigned)(mem * NWV * KW + wave);   // this wave's first k-step

    for (int s = 0; s < T_; ++s) {
        const int t = T_ - 1 - s;
        const XchgGlobal xch(p.xbuf + (size_t)(s & 1) * xslot, (unsigned)xslot);

        // ---- point-wise gate backward for this thread's items --------------------------
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            T st_d[4];
            if (valid[m]) {
                T *gl_ = reinterpret_cast<T *>(tiles + goff(m));   // the item's 4 gates in the LDS tile
                const float si = sigmoidf_<false>(E::to_f32(gl_[0]));
                const float sf = sigmoidf_<false>(E::to_f32(gl_[HT]));
                const float tg = tanhf_<false>(E::to_f32(gl_[2 * HT]));
                const float so = sigmoidf_<false>(E::to_f32(gl_[3 * HT]));
                const float tc = tanhf_<false>(c1v[m]);
                const float c0 = E::to_f32(*reinterpret_cast<const T *>(tiles + BT * GROW + soff(m)));
                const float dh = dh_rec[m] + E::to_f32(*reinterpret_cast<const T *>(tiles + BT * GROW + BT * SROW + soff(m)));
                const float dc1 = dc_state[m] + dh * so * (1.f - tc * tc);
                const float d_o = dh * tc * so * (1.f - so);
                const float d_f = dc1 * c0 * sf * (1.f - sf);
                const float d_i = dc1 * tg * si * (1.f - si);
                const float d_g = dc1 * si * (1.f - tg * tg);
                dc_state[m] = dc1 * sf;
                c1v[m] = c0;   // c_{t-1} is the next step's c_t
                st_d[0] = E::from_f32(d_i);
                st_d[1] = E::from_f32(d_f);
                st_d[2] = E::from_f32(d_g);
                st_d[3] = E::from_f32(d_o);
                gl_[0] = st_d[0];
                gl_[HT] = st_d[1];
                gl_[2 * HT] = st_d[2];
                gl_[3 * HT] = st_d[3];
            } else {
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) st_d[gt] = E::from_f32(0.f);
            }
            // exchange copy: 4 consecutive k = (unit, gate 0..3); lanes l and l+16 own units u and u+1 of
            // the same batch row, the even-unit lane writes both (16 bytes, write-through)
            const u32x2 mine = *reinterpret_cast<u32x2 *>(st_d);
            u32x2 other;
            other[0] = (unsigned)__shfl_down((int)mine[0], 16);
            other[1] = (unsigned)__shfl_down((int)mine[1], 16);
            if (pair_lead[m]) xch.store16(xgrp + xoff(m), u32x4{mine[0], mine[1], other[0], other[1]});
        }
        publish_version(grp_flags + j, s + 1);   // waits for the stores, workgroup barrier, raises the flag
        tile_to_global(t);
        if (wave == 0) wait_versions(grp_flags, p.n_ht, s + 1, p.hdr, p.spin_limit, g, s);
        __syncthreads();

        // ---- partial dh_rec(team units, rows) = Wh[k-part, team units]^T . d_ifgo[t](rows, k-part)^T ----
        // block b of the step: k-step ks_base + 8 (b / NT), batch tile b % NT.  Block b goes L2 -> ring slot
        // b % S; its 16-byte fragment is read two blocks ahead of its MFMAs; the slot is refilled with block
        // b + S right after them.
        const unsigned long long xaddr = reinterpret_cast<unsigned long long>(p.xbuf + (size_t)(s & 1) * xslot);
        const u32x4 xrs = {(unsigned)xaddr, (unsigned)(xaddr >> 32) & 0xffffu, (unsigned)xslot, 0x00020000u};
        auto request = [&](auto bc) __attribute__((always_inline)) {
            constexpr int b = decltype(bc)::value;
            constexpr int ki = b / NT, nt = b % NT;
            const unsigned soff_ = xgrp + ((unsigned)(nt * KSB) + ks_base + NWV * ki) * kFragBytes;
            dma_block_asm<true>(xrs, ring_addr + (b % S) * kFragBytes, lane_off, soff_);
        };
        static_for<0, S>(request);
        u32x4 fr[4];
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S - 1) : "memory");
        fr[0] = lds_read_b128_asm<0>(ring + lane_off);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S - 2) : "memory");
        fr[1] = lds_read_b128_asm<0>(ring + kFragBytes + lane_off);
        f32x4 acc[NT][V];
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int v = 0; v < V; ++v) acc[i][v] = f32x4{0.f, 0.f, 0.f, 0.f};
        static_for<0, NB>([&](auto bc) __attribute__((always_inline)) {
            constexpr int b = decltype(bc)::value;
            constexpr int ki = b / NT, nt = b % NT;
            if constexpr (b + 2 < NB) {
                // block b + 2 has landed when at most the loads behind it are in flight
                constexpr int issued = (S + b < NB) ? S + b : NB;
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(issued - (b + 3)) : "memory");
                fr[(b + 2) & 3] = lds_read_b128_asm<0>(ring + ((b + 2) % S) * kFragBytes + lane_off);
                lds_reads_landed_but<1>(fr[b & 3]);   // all but the read just issued: block b's fragment is here
            } else {
                lds_reads_landed_but<0>(fr[b & 3]);
            }
#pragma unroll
            for (int v = 0; v < V; ++v) acc[nt][v] = mfma_kstep<T>(wreg[v][ki], fr[b & 3], acc[nt][v]);
            if constexpr (b + S < NB) request(std::integral_constant<int, b + S>{});   // its fragment is in a register: the slot is free
        });
        // every wave is through with its ring: the 8 waves' sums of the 4 V tiles meet there
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int v = 0; v < V; ++v) red[(wave * TILES + i * V + v) * kWave + lane] = acc[i][v];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int tl = wave + NWV * i, nt = rnt + (NWV / V) * i;   // tl = nt * V + rv
            f32x4 sum = red[tl * kWave + lane];
#pragma unroll
            for (int w = 1; w < NWV; ++w) sum += red[(w * TILES + tl) * kWave + lane];
            // ... and go to their owner (this workgroup: through LDS)
            if (rv == mem) own[nt * kWave + lane] = sum;
            // (an ordinary store: the team shares one XCD, whose L2 the receivers' device-scope loads read)
            else __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, sum), part.rsrc, part_to + (unsigned)nt * kFragBytes + lane_off, 0, 0);
        }

        // ---- the team's exchange: every member gets the others' sums for its 16 units ----
        publish_version(team_flags + j, s + 1);   // (its barrier: `red` is read, the ring may fill again)
        // the next step's inputs come in meanwhile (the tiles were drained before the group barrier)
        if (s + 1 < T_) request_tiles(t - 1);
        if (wave == 0) wait_versions(team_flags + team0, V, s + 1, p.hdr, p.spin_limit, g, s);
        __syncthreads();
        float got[IPT][V];
#pragma unroll
        for (int m = 0; m < IPT; ++m)
#pragma unroll
            for (int v = 0; v < V; ++v)   // (this member's own place too, which nobody writes: no branches between the loads)
                got[m][v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                    part.rsrc, part_mine + (unsigned)v * kSetBytes + (unsigned)roff(m), 0, kAuxDevice));
#pragma unroll
        for (int m = 0; m < IPT; ++m) {
            const float mine = *reinterpret_cast<const float *>(reinterpret_cast<const unsigned char *>(own) + roff(m));
            float sum = 0 == mem ? mine : got[m][0];
#pragma unroll
            for (int v = 1; v < V; ++v) sum += v == mem ? mine : got[m][v];   // member order, whoever adds
            dh_rec[m] = sum;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's pieces of the next step's tiles are in place
        __syncthreads();                                    // ... and everybody's; `own` is read
    }

    T *dh_out = static_cast<T *>(p.dh), *dc_out = static_cast<T *>(p.dc);
#pragma unroll
    for (int m = 0; m < IPT; ++m)
        if (valid[m]) {
            const int it = tid + NTHR * m;
            const size_t off_h = (size_t)(b0 + (it >> 4) / HT * 16 + (it & 15)) * H + u0 + (it >> 4) % HT;
            dh_out[off_h] = E::from_f32(dh_rec[m]);
            dc_out[off_h] = E::from_f32(dc_state[m]);
        }
}

}  // namespace fastlstm

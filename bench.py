#!/usr/bin/env python3
"""Benchmark of the LSTM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload B|A|C|D|E] [--no-cpu] [--no-miopen]
                    [--stage all|fwd_recurrence|gemms|fwd_layer|bwd_layer]

A "step" is one pass of the workload's hot path over one batch of synthetic input
(already resident in HBM).  The default workload is BASELINE.json's headline
configuration B: single-layer fp16 FORWARD, batch 64, seq_len 512, input = hidden =
1024 (x ~ N(0,1), h0,c0 ~ N(0,0.1), weights U(+-1/32), seeded).  Prints ONE JSON
line: metric/value = batch*timesteps per second of that step, plus
  roofline      for the dominant kernel (the launch that holds the persistent recurrence), timed with
                HIP events on the launch stream: its algorithmic flops against the MFMA peak and, in
                roofline.latency_bound, its time per timestep against the measured latency floor of a
                step (barrier round trip + exchange of h_t, fastlstm_diag_step_probe),
  kernels       per-stage timings (input-projection GEMM, recurrence, and for the
                forward+backward pass: reverse recurrence, dx GEMM, weight-gradient GEMMs),
  fwd / fwd_bwd the workload timed forward and forward+backward (hot loop, mean of --steps calls),
  do_bench      the same two with the protocol of the reference's scripts/benchmark.py:118-133
                (triton.testing.do_bench: warm-up 40 ms, 160 ms of repetitions, the L2-sized buffer
                cleared before each one, one event pair per repetition, median),
  nn_lstm_rocm  torch.nn.LSTM (MIOpen) on the same GPU, same shapes and dtype,
  cpu_baseline  torch.nn.LSTM fp32 on the box's host cores (physical cores, stated) on the same workload,
  cpu_oracle    the CPU oracle (C, OpenMP) on a bounded sample.
The --stage values other than "all" launch a few repetitions of one group of kernels plus a plain
copy of known size and print nothing: they are the targets of rocprofv3 counter runs (profiles/).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: dtype, mode, B, T, I, H, layers
    "A": ("fp32", "fwd_bwd", 16, 128, 256, 256, 1),
    "B": ("fp16", "fwd", 64, 512, 1024, 1024, 1),
    "C": ("bf16", "fwd_bwd", 128, 256, 2048, 2048, 1),
    "D": ("fp16", "fwd_bwd", 256, 1024, 64, 64, 1),
    "E": ("fp16", "fwd_bwd", 32, 2048, 1024, 1024, 2),
}
PEAK_TFLOPS = {"fp16": 2500.0, "bf16": 2500.0, "fp32": 157.3}  # MI355X dense MFMA, published
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel from rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a plain
# copy of known size.  Counters cannot be read from inside this process: the figures are copied from the
# committed summaries named here (made by `rocprofv3 --pmc ... -- python3 bench.py --stage fwd_layer`).
TRAFFIC = {"B": (1411.1e6, "profiles/recurrence_lds_l2_B.md"), "D": (336.1e6, "profiles/fwd_recurrence_D_pmc.md")}


def physical_cores():
    """Physical cores this process may use: distinct (package, core) pairs of the CPUs in its affinity
    mask, capped by OMP_NUM_THREADS (the box's CPU share)."""
    allowed = os.sched_getaffinity(0)
    seen = set()
    try:
        for cpu in allowed:
            base = "/sys/devices/system/cpu/cpu%d/topology/" % cpu
            with open(base + "physical_package_id") as f:
                pkg = f.read().strip()
            with open(base + "core_id") as f:
                core = f.read().strip()
            seen.add((pkg, core))
        n = len(seen)
    except OSError:
        n = len(allowed)
    cap = os.environ.get("OMP_NUM_THREADS")
    return max(1, min(n, int(cap)) if cap else n)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="B", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-miopen", action="store_true", help="skip the nn.LSTM-on-ROCm leg")
    ap.add_argument("--stage", default="all", choices=["all", "fwd_recurrence", "gemms", "fwd_layer", "bwd_layer"],
                    help="other than all: launch only that group of kernels and a calibration copy (for counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the LSTM recurrence is not sharded across "
              "GPUs: batch rows would be split, with one all-reduce of the weight gradients); "
              "--gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import fastlstm_amd.lstm as L
    from fastlstm_amd import FastLSTM, _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    dname, mode, B, T, I, H, layers = WORKLOADS[args.workload]
    dt = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}[dname]
    code = {"fp32": 0, "fp16": 1, "bf16": 2}[dname]

    # ---- synthetic inputs (seeded, generated on the CPU in fp32, then cast) -------------
    g = torch.Generator().manual_seed(1234 + ord(args.workload) - ord("A"))
    torch.manual_seed(1234)
    model = FastLSTM(I, H, num_layers=layers)  # U(+-1/sqrt(H)) init, nn.LSTM order
    x_cpu = torch.randn(T, B, I, generator=g)
    if args.workload == "D":
        x_cpu = torch.rand(T, B, I, generator=g) * 2 - 1
    h0_cpu = torch.randn(layers, B, H, generator=g) * 0.1 if args.workload == "B" else torch.zeros(layers, B, H)
    c0_cpu = torch.randn(layers, B, H, generator=g) * 0.1 if args.workload == "B" else torch.zeros(layers, B, H)
    model = model.to(dev, dt)
    x = x_cpu.to(dev, dt)
    h0, c0 = h0_cpu.to(dev, dt), c0_cpu.to(dev, dt)

    def step_fwd():
        return model(x, (h0, c0))

    def step_fwd_bwd():
        for p in model.parameters():
            p.grad = None
        out, _ = model(x, (h0, c0))
        out.sum().backward()

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    def ev_time(fn, reps=10, warmup=2, pre=None):
        """average device time (ms) of the launches fn() makes: one HIP event pair per repetition,
        recorded on the stream the kernels are launched on (torch's current stream); pre() runs
        outside the timed region."""
        total = 0.0
        for i in range(warmup + reps):
            if pre:
                pre()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            fn()
            e.record()
            torch.cuda.synchronize()
            if i >= warmup:
                total += s.elapsed_time(e)
        return total / reps

    flush_buf = torch.empty(256 << 20, dtype=torch.uint8, device=dev)   # as triton's do_bench: 256 MB

    def do_bench(fn, warmup_ms=40.0, rep_ms=160.0):
        """triton.testing.do_bench(fn, warmup, rep, return_mode="median") restated: one untimed call,
        estimate = mean of 5 calls, n = ms / estimate repetitions; before every repetition the cache-sized
        buffer is cleared; one event pair per repetition, one synchronisation at the end; the median."""
        fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(5):
            flush_buf.zero_()
            fn()
        e.record()
        torch.cuda.synchronize()
        est = s.elapsed_time(e) / 5
        if T < 128:            # the reference scales both for small problems (scripts/benchmark.py:118-131)
            warmup_ms, rep_ms = warmup_ms * 1.5, rep_ms * 3
        if H < 128:
            warmup_ms, rep_ms = warmup_ms * 1.5, rep_ms * 3
        if B < 32:
            warmup_ms, rep_ms = warmup_ms * 1.5, rep_ms * 3
        n_warm, n_rep = max(1, int(warmup_ms / est)), max(1, int(rep_ms / est))
        for _ in range(n_warm):
            fn()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_rep)]
        for s, e in evs:
            flush_buf.zero_()
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        return statistics.median(s.elapsed_time(e) for s, e in evs), n_rep

    # ---- per-stage launches through the C ABI (layer-0 shapes) ---------------------------
    stream = torch.cuda.current_stream().cuda_stream
    Wx, Wh = model.weight_ih_l0.detach(), model.weight_hh_l0.detach()
    bx, bh = model.bias_ih_l0.detach(), model.bias_hh_l0.detach()
    ifgo0 = torch.empty(T, B, 4 * H, device=dev, dtype=dt)
    ifgo = torch.empty_like(ifgo0)
    out = torch.empty(T + 1, B, H, device=dev, dtype=dt)
    cell = torch.empty(T + 1, B, H, device=dev, dtype=dt)
    out[0], cell[0] = h0[0], c0[0]
    plan_f, plan_b = _lib.Plan(), _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 0, plan_f), "plan")
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 1, plan_b), "plan")
    # the workspaces lstm.py allocates per call (header, barrier counters, two exchange slots)
    ws_f = L._workspace(plan_f, T, H, code, False, dev)
    ws_b = L._workspace(plan_b, T, H, code, True, dev)

    def zero_ws(ws, plan):  # the part a call needs zeroed: header, counters, flags
        n = ws.numel() if plan.ring_needs_zero else min(ws.numel(), plan.ws_zero_bytes)
        ws[:n].zero_()

    def k1():
        _lib.check(lib.fastlstm_gemm_ifgo(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(),
                                          ifgo0.data_ptr(), T, B, I, H, code, stream), "k1")

    def rec_fwd():
        _lib.check(lib.fastlstm_fwd_persistent(ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), Wh.data_ptr(),
                                               ws_f.data_ptr(), ws_f.numel(), T, B, H, code, stream), "fwd")

    def rec_fwd_pre():  # the kernel overwrites ifgo in place and needs zeroed flags
        ifgo.copy_(ifgo0)
        zero_ws(ws_f, plan_f)

    def layer_fwd():   # what lstm_persistent_fwd calls: projection + recurrence, fused where CUs would idle
        _lib.check(lib.fastlstm_fwd_layer(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), Wh.data_ptr(),
                                          ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), ws_f.data_ptr(),
                                          ws_f.numel(), T, B, I, H, code, stream), "fwd_layer")

    def layer_fwd_infer():   # the same launch without the stores only a reverse pass reads
        _lib.check(lib.fastlstm_fwd_layer_infer(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), Wh.data_ptr(),
                                                ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), ws_f.data_ptr(),
                                                ws_f.numel(), T, B, I, H, code, stream), "fwd_layer_infer")

    # backward stages
    dout = torch.ones(T, B, H, device=dev, dtype=dt)
    d_ifgo = torch.empty_like(ifgo)
    dh_n = torch.zeros(B, H, device=dev, dtype=dt)
    dc_n = torch.zeros(B, H, device=dev, dtype=dt)
    dx = torch.empty(T, B, I, device=dev, dtype=dt)
    dWx, dWh_, db = torch.empty_like(Wx), torch.empty_like(Wh), torch.empty_like(bx)
    ws_w = torch.empty(lib.fastlstm_wgrad_workspace_bytes(T, B, I, H, code), dtype=torch.uint8, device=dev)

    def rec_bwd():
        _lib.check(lib.fastlstm_bwd_persistent(dout.data_ptr(), dh_n.data_ptr(), dc_n.data_ptr(), ifgo.data_ptr(),
                                               cell.data_ptr(), d_ifgo.data_ptr(), Wh.data_ptr(), ws_b.data_ptr(),
                                               ws_b.numel(), T, B, H, code, stream), "bwd")

    def rec_bwd_pre():
        zero_ws(ws_b, plan_b); dh_n.zero_(); dc_n.zero_()

    def k5():
        # (with the weight-gradient workspace as scratch, as fastlstm_bwd_layer calls it: a dx with few output
        # tiles is split along K)
        _lib.check(lib.fastlstm_gemm_dx_split(d_ifgo.data_ptr(), Wx.data_ptr(), dx.data_ptr(), T, B, I, H, code,
                                              ws_w.data_ptr(), ws_w.numel(), stream), "k5")

    def k89():
        _lib.check(lib.fastlstm_gemm_wgrad(d_ifgo.data_ptr(), x.data_ptr(), out.data_ptr(), dWx.data_ptr(),
                                           dWh_.data_ptr(), db.data_ptr(), ws_w.data_ptr(), ws_w.numel(), T, B, I, H,
                                           code, stream), "wgrad")

    def k589():   # K5 + K8 + K9 + db in one call: one pass over d_ifgo for a narrow layer (workload D), the two stages otherwise
        _lib.check(lib.fastlstm_gemm_dx_wgrad(d_ifgo.data_ptr(), Wx.data_ptr(), x.data_ptr(), out.data_ptr(), dx.data_ptr(),
                                              dWx.data_ptr(), dWh_.data_ptr(), db.data_ptr(), ws_w.data_ptr(), ws_w.numel(),
                                              T, B, I, H, code, stream), "dx + wgrad")

    def layer_bwd():   # what lstm_persistent_bwd calls: recurrence + dx + dWx + dWh + db, fused where CUs would idle
        _lib.check(lib.fastlstm_bwd_layer(dout.data_ptr(), dh_n.data_ptr(), dc_n.data_ptr(), ifgo.data_ptr(),
                                          cell.data_ptr(), d_ifgo.data_ptr(), Wh.data_ptr(), Wx.data_ptr(),
                                          x.data_ptr(), out.data_ptr(), dx.data_ptr(), dWx.data_ptr(), dWh_.data_ptr(),
                                          db.data_ptr(), ws_b.data_ptr(), ws_b.numel(), ws_w.data_ptr(), ws_w.numel(),
                                          T, B, I, H, code, stream), "bwd_layer")

    if args.stage != "all":
        # counter runs (rocprofv3 --pmc / --kernel-trace): one group of kernels, three repetitions, plus a
        # plain copy of known size (2 x 256 MiB of traffic) that calibrates FETCH_SIZE / WRITE_SIZE
        k1()
        zero_ws(ws_f, plan_f)
        layer_fwd()             # valid ifgo / out / cell for the backward stages
        cal_src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        cal_dst = torch.empty_like(cal_src)
        for _ in range(3):
            if args.stage == "fwd_recurrence":
                rec_fwd_pre()
                rec_fwd()            # the recurrence alone (ifgo complete at launch)
                zero_ws(ws_f, plan_f)
                layer_fwd()          # projection + recurrence in one launch where the library fuses them
                zero_ws(ws_f, plan_f)
                layer_fwd_infer()
            elif args.stage == "fwd_layer":
                zero_ws(ws_f, plan_f)
                layer_fwd()
            elif args.stage == "bwd_layer":
                rec_bwd_pre()
                layer_bwd()
            else:   # gemms: K1, K5, K8 + K9 (+ db) as stand-alone launches, then K5 + K8 + K9 + db as one call
                rec_bwd_pre()
                rec_bwd()            # a real d_ifgo
                k1()
                k5()
                k89()
                k589()               # K5 + K8 + K9 + db in one call
            cal_dst.copy_(cal_src)
        torch.cuda.synchronize()
        return

    headline = step_fwd if mode == "fwd" else step_fwd_bwd
    with torch.enable_grad():
        ms = timed(headline, args.steps, args.warmup)
        ms_fwd = ms if mode == "fwd" else timed(step_fwd, args.steps, args.warmup)
        ms_full = ms if mode == "fwd_bwd" else timed(step_fwd_bwd, max(3, args.steps // 2), max(2, args.warmup // 2))
        db_fwd, n_fwd = do_bench(step_fwd)
        db_full, n_full = do_bench(step_fwd_bwd)
        # the reference's stand-alone "bwd" mode (scripts/benchmark.py:79-113): lstm_persistent_bwd of the first layer
        # on random activations, which its lambda draws inside the timed call; beside it the same call on tensors
        # drawn beforehand
        Wx0, Wh0 = model.weight_ih_l0.detach(), model.weight_hh_l0.detach()
        rnd = lambda *shape: torch.randn(shape, device=dev, dtype=dt)

        def step_bwd_as_reference():
            return L.lstm_persistent_bwd(rnd(T, B, H), rnd(B, H), rnd(B, H), x, rnd(T + 1, B, H), rnd(T + 1, B, H),
                                         rnd(T, B, 4 * H), Wx0, Wh0)

        bw_args = (rnd(T, B, H), rnd(B, H), rnd(B, H), x, rnd(T + 1, B, H), rnd(T + 1, B, H), rnd(T, B, 4 * H), Wx0, Wh0)
        db_bwd_ref, n_bwd_ref = do_bench(step_bwd_as_reference)
        db_bwd, n_bwd = do_bench(lambda: L.lstm_persistent_bwd(*bw_args))
    value = B * T / (ms * 1e-3)

    t_k1 = ev_time(k1)
    t_rec = ev_time(rec_fwd, pre=rec_fwd_pre)
    t_layer = ev_time(layer_fwd, pre=lambda: zero_ws(ws_f, plan_f))
    t_infer = ev_time(layer_fwd_infer, pre=lambda: zero_ws(ws_f, plan_f))
    kernels = {"gemm_ifgo_ms": round(t_k1, 4), "recurrent_fwd_ms": round(t_rec, 4),
               "recurrent_fwd_us_per_step": round(t_rec * 1e3 / T, 3),
               "fwd_layer_ms": round(t_layer, 4), "fwd_layer_infer_ms": round(t_infer, 4),
               "gemm_ifgo_tflops": round(2.0 * T * B * I * 4 * H / (t_k1 * 1e-3) / 1e12, 2),
               "gemm_ifgo_frac_of_mfma_peak": round(2.0 * T * B * I * 4 * H / (t_k1 * 1e-3) / 1e12 / PEAK_TFLOPS[dname], 4),
               "plan_fwd": plan_f.as_dict(), "plan_bwd": plan_b.as_dict()}
    torch.cuda.synchronize()
    _lib.check(lib.fastlstm_ws_status(ws_f[:64].cpu().numpy().tobytes()), "forward barrier status")

    t_rb = ev_time(rec_bwd, reps=5, pre=rec_bwd_pre)
    t_k5 = ev_time(k5, reps=5)
    t_k89 = ev_time(k89, reps=5)
    t_k589 = ev_time(k589, reps=5)
    t_lb = ev_time(layer_bwd, reps=5, pre=rec_bwd_pre)
    torch.cuda.synchronize()
    _lib.check(lib.fastlstm_ws_status(ws_b[:64].cpu().numpy().tobytes()), "backward barrier status")
    gf = 2.0 * T * B * I * 4 * H
    gw = 2.0 * T * B * 4 * H * (I + H)
    kernels.update({
        "recurrent_bwd_ms": round(t_rb, 4), "recurrent_bwd_us_per_step": round(t_rb * 1e3 / T, 3),
        "gemm_dx_ms": round(t_k5, 4),
        "gemm_dx_tflops": round(gf / (t_k5 * 1e-3) / 1e12, 2),
        "gemm_dx_frac_of_mfma_peak": round(gf / (t_k5 * 1e-3) / 1e12 / PEAK_TFLOPS[dname], 4),
        "gemm_wgrad_ms": round(t_k89, 4),
        "gemm_wgrad_tflops": round(gw / (t_k89 * 1e-3) / 1e12, 2),
        "gemm_wgrad_frac_of_mfma_peak": round(gw / (t_k89 * 1e-3) / 1e12 / PEAK_TFLOPS[dname], 4),
        "gemm_dx_wgrad_ms": round(t_k589, 4),
        "bwd_layer_ms": round(t_lb, 4),
    })
    # the same three stages with the tile kernel in its earlier form (one tile per workgroup, symmetric main loop,
    # LDS-staged ordinary stores, weight gradients as two products + a column-sum pass), same operands, same process:
    # box-to-box variation is larger than several of the steps in between
    if dname != "fp32":
        try:
            lib.fastlstm_set_gemm_baseline(1)
            tb1, tb5, tb89 = ev_time(k1, reps=5), ev_time(k5, reps=5), ev_time(k89, reps=5)
        finally:
            lib.fastlstm_set_gemm_baseline(0)
        kernels["gemm_earlier_form_ms"] = {"ifgo": round(tb1, 4), "dx": round(tb5, 4), "wgrad": round(tb89, 4)}
        kernels["gemm_gain_over_earlier_form"] = {"ifgo": round(tb1 / t_k1, 3), "dx": round(tb5 / t_k5, 3),
                                                  "wgrad": round(tb89 / t_k89, 3)}
    # yardstick for the three GEMM stages: the vendor library (torch.matmul = hipBLASLt / rocBLAS) on the same
    # operands and shapes, timed the same way; not part of any measured step
    if dname != "f32":
        x2, d2, h2 = x.reshape(T * B, I), d_ifgo.reshape(T * B, 4 * H), out[:T].reshape(T * B, H)
        bias = torch.zeros(4 * H, dtype=x.dtype, device=dev)
        t_l1 = ev_time(lambda: torch.addmm(bias, x2, Wx.t()), reps=5)
        t_l5 = ev_time(lambda: torch.mm(d2, Wx), reps=5)
        t_l89 = ev_time(lambda: (torch.mm(d2.t(), x2), torch.mm(d2.t(), h2), d2.sum(0)), reps=5)
        kernels["library_gemm_ms"] = {"ifgo": round(t_l1, 4), "dx": round(t_l5, 4), "wgrad": round(t_l89, 4)}

    # ---- roofline of the dominant kernel of the headline (forward) path ------------------
    # XCD-local path with idle CUs: ONE launch does projection + recurrence (fastlstm_fwd_layer);
    # otherwise the recurrence launch dominates.  The flops are priced against the MFMA peak; what bounds
    # the launch is the latency of T sequential steps, measured below.
    rec_flops = 2.0 * B * H * 4 * H * T          # algorithmic flops of the recurrence
    k1_flops = 2.0 * T * B * I * 4 * H           # ... of the input projection
    kind = lib.fastlstm_recurrent_kernel_kind(T, B, H, code, 0, ws_f.numel())
    xcd_local = kind == 1
    fused = xcd_local and t_layer < 0.9 * (t_k1 + t_rec)
    traffic, traffic_src = TRAFFIC.get(args.workload, (None, None))
    if fused:
        flops, t_dom, kname = rec_flops + k1_flops, t_layer, "lstm_fwd_xcd_kernel<..., HELP=true> (projection + recurrence)"
        alg = "2*B*H*4H*T + 2*T*B*I*4H flop per launch = %.1f GFLOP" % (flops / 1e9)
    else:
        flops, t_dom = rec_flops, t_rec
        kname = {0: "lstm_fwd_persistent_kernel", 1: "lstm_fwd_xcd_kernel", 2: "lstm_fwd_wide_kernel"}[kind]
        alg = "2*B*H*4H*T flop per launch = %.1f GFLOP" % (flops / 1e9)
        if args.workload == "B":
            traffic, traffic_src = None, None
    ach = flops / (t_dom * 1e-3) / 1e12
    roofline = {"kernel": kname, "bound": "mfma", "achieved": round(ach, 2),
                "peak": PEAK_TFLOPS[dname], "unit": "TFLOP/s", "frac": round(ach / PEAK_TFLOPS[dname], 4),
                "traffic": traffic, "traffic_source": traffic_src,
                "algorithmic": alg, "launch_ms": round(t_dom, 4),
                "note": "the launch is latency-bound, not MFMA-bound: T sequential steps, each a cross-CU exchange "
                        + ("through the L2 of one XCD" if xcd_local else "through device memory")
                        + "; see latency_bound"}

    if plan_f.wave_split == 2:
        # one hidden tile per workgroup (H <= 64): no exchange between CUs at all; the kernel streams the
        # gate tiles through (read + write-back) and writes out / cell -- priced against HBM
        sz = 2 if dname != "fp32" else 4
        # (64 units: batch tiles of 4 or 8 rows where that many workgroups find a CU each, as the library decides)
        rows_wg = 16 if H != 64 else (4 if -(-B // 4) <= plan_f.num_cus else 8 if -(-B // 8) <= plan_f.num_cus else 16)
        nbytes = sz * (2.0 * T * B * 4 * H + 2.0 * T * B * H + 4.0 * H * H)
        ach = nbytes / (t_rec * 1e-3) / 1e9
        roofline = {"kernel": "lstm_fwd_persistent_kernel<SPLIT=2> (one hidden tile per workgroup)", "bound": "hbm",
                    "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                    "traffic": traffic, "traffic_source": traffic_src,
                    "algorithmic": "s*(2*T*B*4H + 2*T*B*H + 4H*H) bytes per launch = %.1f MB" % (nbytes / 1e6),
                    "launch_ms": round(t_rec, 4),
                    "note": "latency-bound, not HBM-bound: %d independent workgroups (%d batch rows each) walk through "
                            "T sequential steps; us/step is in kernels.recurrent_fwd_us_per_step" % (-(-B // rows_wg), rows_wg)}
    elif dname != "fp32" and H % 32 == 0 and H <= 2048:
        # ---- the latency floor of a step, measured with the recurrence's own barrier and exchange code ----
        # (fastlstm_diag_step_probe: 16-bit h tiles; one group is timed alone on an otherwise idle device)
        if kind == 1:
            pk, members, rows = 0, min(32, H // 8), 16   # the smallest unit tile that keeps a group on one XCD
        elif kind == 2:
            pk, members, rows = 1, H // 16, 64
        else:
            pk, members, rows = 1, plan_f.n_htiles, min(64, max(16, plan_f.bt // 16 * 16))
        while H % members:
            members -= 1
        steps_p = 512
        ws_p = torch.zeros(lib.fastlstm_diag_step_probe_bytes(steps_p, H, rows), dtype=torch.uint8, device=dev)
        probe = {}
        for pm, name in ((0, "empty_barrier_us"), (1, "barrier_plus_publish_us"), (2, "barrier_publish_fetch_us")):
            def run(pm=pm):
                _lib.check(lib.fastlstm_diag_step_probe(pk, pm, members, H, rows, steps_p, ws_p.data_ptr(), ws_p.numel(),
                                                        stream), "step probe")
            probe[name] = round(ev_time(run, reps=5, warmup=2, pre=lambda: ws_p[:70000].zero_()) * 1e3 / steps_p, 3)
        torch.cuda.synchronize()
        _lib.check(lib.fastlstm_ws_status(ws_p[:64].cpu().numpy().tobytes()), "step probe status")
        mfma_us = 2.0 * B * H * 4 * H / (PEAK_TFLOPS[dname] * 1e12) * 1e6
        bound = probe["barrier_publish_fetch_us"]
        per_step = t_dom * 1e3 / T
        roofline["latency_bound"] = {
            "bound": "latency", "per_step_bound_us": bound, "achieved_us_per_step": round(per_step, 3),
            "frac": round(bound / per_step, 4),
            "recurrence_alone_us_per_step": round(t_rec * 1e3 / T, 3),
            "frac_recurrence_alone": round(bound / (t_rec * 1e3 / T), 4),
            "mfma_time_per_step_at_peak_us": round(mfma_us, 3),
            "probe": dict(probe, group="XCD-local, L2 counters" if pk == 0 else "flag group over all XCDs",
                          members=members, rows=rows, steps=steps_p),
            "note": "per_step_bound_us = publish h_t + barrier round trip + fetch of the group's h_t, timed with the "
                    "kernels' own code and no arithmetic (fastlstm_diag_step_probe mode 2); frac = bound / achieved"}

    res = {
        "metric": "lstm_%s_batch_timesteps_per_s" % mode, "value": round(value, 1), "unit": "batch*timesteps/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dname, "data": "synthetic",
        "config": {"workload": "%s: %d-layer LSTM %s %s, B=%d T=%d I=%d H=%d" % (args.workload, layers, dname, mode, B, T, I, H)},
        "fwd": {"ms": round(ms_fwd, 4), "bt_per_s": round(B * T / (ms_fwd * 1e-3), 1)},
        "fwd_bwd": {"ms": round(ms_full, 4), "bt_per_s": round(B * T / (ms_full * 1e-3), 1)},
        "do_bench": {"fwd_ms": round(db_fwd, 4), "fwd_reps": n_fwd, "fwd_bwd_ms": round(db_full, 4), "fwd_bwd_reps": n_full,
                     "fwd_bt_per_s": round(B * T / (db_fwd * 1e-3), 1), "fwd_bwd_bt_per_s": round(B * T / (db_full * 1e-3), 1),
                     "bwd_ms": round(db_bwd, 4), "bwd_reps": n_bwd, "bwd_with_randn_inside_ms": round(db_bwd_ref, 4),
                     "bwd_note": "lstm_persistent_bwd of one layer on random activations (scripts/benchmark.py:79-113); "
                                 "the reference's lambda draws the six random tensors inside the timed call (second figure)",
                     "protocol": "median; warm-up 40 ms, 160 ms of repetitions, 256 MB buffer cleared before each, one "
                                 "event pair per repetition (the reference's scripts/benchmark.py:118-133)"},
        "roofline": roofline, "kernels": kernels,
    }

    # ---- torch.nn.LSTM on the same GPU (MIOpen): the 1.5x target's denominator -----------
    if not args.no_miopen:
        try:
            ref = torch.nn.LSTM(I, H, num_layers=layers).to(dev, dt)
            with torch.no_grad():
                for n, p in model.named_parameters():
                    getattr(ref, n).copy_(p)

            def ref_fwd():
                return ref(x, (h0, c0))

            def ref_full():
                for p in ref.parameters():
                    p.grad = None
                o, _ = ref(x, (h0, c0))
                o.sum().backward()

            r_f = timed(ref_fwd, max(3, min(20, args.steps // 2)), 2)
            r_b = timed(ref_full, max(3, min(20, args.steps // 2)), 2)
            res["nn_lstm_rocm"] = {"fwd_ms": round(r_f, 4), "fwd_bwd_ms": round(r_b, 4),
                                   "speedup_fwd": round(r_f / ms_fwd, 3), "speedup_fwd_bwd": round(r_b / ms_full, 3)}
        except Exception as exc:  # MIOpen may not support a configuration
            res["nn_lstm_rocm"] = {"error": str(exc)[:200]}

    # ---- CPU baselines ---------------------------------------------------------------------
    if not args.no_cpu:
        import numpy as np

        cores = physical_cores()
        torch.set_num_threads(cores)
        cpu_model = torch.nn.LSTM(I, H, num_layers=layers)   # fp32, the module's parameters
        with torch.no_grad():
            for n, p in model.named_parameters():
                getattr(cpu_model, n).copy_(p.float().cpu())

        def cpu_pass(ts):
            xs = x_cpu[:ts]
            t0 = time.perf_counter()
            if mode == "fwd":
                with torch.no_grad():
                    cpu_model(xs, (h0_cpu, c0_cpu))
            else:
                for p in cpu_model.parameters():
                    p.grad = None
                o, _ = cpu_model(xs, (h0_cpu, c0_cpu))
                o.sum().backward()
            return time.perf_counter() - t0

        probe_t = min(T, 16)
        per_step = cpu_pass(probe_t) / probe_t
        per_step = min(per_step, cpu_pass(probe_t) / probe_t)
        ts = int(max(probe_t, min(T, 4.0 / max(per_step, 1e-9))))      # a pass of at most ~4 s
        passes = int(max(3, min(10, 12.0 / max(per_step * ts, 1e-9))))   # >= 3 passes, ~12 s in all
        times = sorted(cpu_pass(ts) for _ in range(passes))
        el = times[len(times) // 2]
        res["cpu_baseline"] = {"value": round(B * ts / el, 1), "unit": "batch*timesteps/s", "cores": cores,
                               "kind": "port",
                               "sample": "torch.nn.LSTM fp32 (the parity target the reference's tests use) on the host, "
                                         "%d physical cores = torch threads, same weights and inputs, all %d layer(s), "
                                         "first %d of %d timesteps, %s; median of %d passes (%.3f s each)"
                                         % (cores, layers, ts, T, mode, passes, el)}

        from oracle import lstm_oracle as orc

        a = [model.get_parameter(n).detach().float().cpu().numpy()
             for n in ("weight_ih_l0", "bias_ih_l0", "weight_hh_l0", "bias_hh_l0")]

        def oracle_run(ts):
            t0 = time.perf_counter()
            o, c, p = orc.forward(x_cpu[:ts].numpy(), h0_cpu[0].numpy(), c0_cpu[0].numpy(), a[0], a[1], a[2], a[3],
                                  dtype=np.float32)
            if mode == "fwd_bwd":
                orc.backward(np.ones((ts, B, H), np.float32), None, None, x_cpu[:ts].numpy(), o, c, p, a[0], a[2],
                             dtype=np.float32)
            return time.perf_counter() - t0

        probe_t = min(T, 4)
        per_step = oracle_run(probe_t) / probe_t
        ts = int(max(probe_t, min(T, 5.0 / max(per_step, 1e-9))))
        el = oracle_run(ts)
        res["cpu_oracle"] = {"value": round(B * ts / el, 1), "unit": "batch*timesteps/s",
                             "threads": int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)),
                             "sample": "C/OpenMP fp32 oracle (the parity checker), layer 0, first %d of %d timesteps, %s; "
                                       "one pass of %.1f s" % (ts, T, mode, el)}

    print(json.dumps(res))


if __name__ == "__main__":
    main()

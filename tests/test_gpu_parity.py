"""GPU parity tests (run with -m gpu on an MI355X).  Everything goes through the C ABI
of libfastlstm_hip.so via the Python mirror of the reference's interface.

Tolerances (north star): fp32 rtol = atol = 1e-4 against torch.nn.LSTM with identical
weights; fp16/bf16 <= 2e-2 relative (error max-norm / reference max-norm) against an
fp32/fp64 evaluation with the same 16-bit-rounded weights and inputs.
"""
import os

import numpy as np
import pytest
import torch

import fastlstm_amd.lstm as L
from fastlstm_amd import FastLSTM, PersistentLSTMfn, _lib
from helpers import elementwise_ratio, make_problem, nn_lstm_reference, rel_err, to_np

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FP32_TOL = 1e-4
HALF_TOL = 2e-2
RM = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
FWD_KEYS = ["x", "h0", "c0", "Wx", "bx", "Wh", "bh"]


@pytest.fixture(scope="module", autouse=True)
def _gpu_setup():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    old = L.CHECK_STATUS
    L.CHECK_STATUS = True  # every recurrent launch is checked for barrier time-outs
    yield
    L.CHECK_STATUS = old


@pytest.fixture(autouse=True)
def _all_kernel_families():
    yield
    _lib.load().fastlstm_set_kernel_families(7)   # whatever a test switched off is back on for the next one


def npy(t):
    return t.detach().double().cpu().numpy()


def dev(t, dt=None):
    return None if t is None else (t.to(dt) if dt else t).cuda()


def assert_close32(got, want, scale_atol=1.0):
    want = torch.as_tensor(np.asarray(want)) if not torch.is_tensor(want) else want
    torch.testing.assert_close(got.detach().cpu().double(), want.double(), rtol=FP32_TOL,
                               atol=FP32_TOL * scale_atol)


def within(got, want, tol, what=None):
    """The 16-bit bar: max-norm relative error below tol.  The fp32 bar (tol == FP32_TOL): additionally every
    ELEMENT inside rtol = atol = 1e-4."""
    e = rel_err(got, want)
    assert e < tol, (what, e)
    if tol == FP32_TOL:
        r = elementwise_ratio(got, want, FP32_TOL, FP32_TOL)
        assert r <= 1.0, (what, "element-wise", r)


def _max_norm_only(got, want, tol):
    assert rel_err(got, want) < tol, rel_err(got, want)


def assert_elementwise32(rows, what):
    """rows: (name, got, want).  Prints the worst |got - want| / (1e-4 + 1e-4*|want|) of every tensor
    and asserts that each ELEMENT is inside rtol = atol = 1e-4 (no scaling by the tensor's magnitude)."""
    worst = 0.0
    for name, got, want in rows:
        r = elementwise_ratio(got, want, FP32_TOL, FP32_TOL)
        print("    %s %-16s worst |err| / (atol + rtol*|ref|) = %.3f" % (what, name, r))
        worst = max(worst, r)
        assert r <= 1.0, (what, name, r)
    return worst


# --------------------------------------------------------------------------------------
# 1. the reference's own integration grid (tests/test_lstm.py:160-220): 2 layers, I = 123,
#    ragged B and H, fp32, module outputs and every parameter gradient vs nn.LSTM
# --------------------------------------------------------------------------------------
@pytest.mark.parametrize("seq_size", [10, 100])
@pytest.mark.parametrize("batch_size", [4, 44, 100])
@pytest.mark.parametrize("hidden_size", [16, 65, 257])
def test_fastlstm_module_vs_nn_lstm(seq_size, batch_size, hidden_size):
    input_size, num_layers = 123, 2
    torch.manual_seed(123)
    m1 = FastLSTM(input_size, hidden_size, num_layers=num_layers, version="persistent").cuda()
    torch.manual_seed(123)
    m2 = torch.nn.LSTM(input_size, hidden_size, num_layers=num_layers)  # CPU fp32 oracle
    x = torch.randn(seq_size, batch_size, input_size)
    y1, (hn1, cn1) = m1(x.cuda())
    y2, (hn2, cn2) = m2(x)
    assert_close32(y1, y2)
    assert_close32(hn1, hn2)
    assert_close32(cn1, cn2)
    assert not hn1.requires_grad and not cn1.requires_grad  # nested tuple => no grad (lstm.py:522)
    y1.sum().backward()
    y2.sum().backward()
    rows = [("y", y1, y2), ("h_n", hn1, hn2), ("c_n", cn1, cn2)]
    rows += [(n + ".grad", p.grad, getattr(m2, n).grad) for n, p in m1.named_parameters()]
    assert_elementwise32(rows, "T%d B%d H%d" % (seq_size, batch_size, hidden_size))


# --------------------------------------------------------------------------------------
# 2. every stage through the C ABI against the CPU oracle, all dtypes, ragged shapes
# --------------------------------------------------------------------------------------
STAGE_CASES = [
    # T, B, I, H, dtype
    (7, 5, 11, 13, torch.float32),        # tiny, everything ragged, barrier-free form
    (9, 12, 128, 213, torch.float32),     # the reference's unit-test shape (test_lstm.py:46-69)
    (5, 33, 70, 300, torch.float32),
    (6, 20, 64, 64, torch.float16),       # config D's hidden size: batch tiles of 4 rows, one cell per lane
    (1, 16, 32, 64, torch.float16),       # one-tile form, tile-moving waves' loop: a single step (nothing but its remainder path)
    (3, 33, 16, 32, torch.bfloat16),      # ... fewer steps than one pass of the unrolled loop, a ragged last batch tile
    (13, 50, 64, 16, torch.float16),      # ... three passes and a remainder of one, 16 units (one row tile per workgroup)
    (9, 16, 64, 64, torch.float32),       # ... fp32 pieces (two per row segment)
    (3, 1100, 32, 64, torch.float16),     # ... 64 units with more rows than CUs x 4: batch tiles of 8 rows (the last one ragged)
    (2, 2100, 16, 64, torch.bfloat16),    # ... and more than CUs x 8: batch tiles of 16 rows
    (6, 20, 40, 72, torch.float16),       # H % 8 == 0 but not a tile multiple
    (5, 7, 30, 100, torch.bfloat16),      # H % 8 != 0: unaligned rows in every kernel
    (4, 64, 256, 1024, torch.float16),    # config B tiles
    (3, 128, 128, 2048, torch.bfloat16),  # config C tiles (waves split the batch)
    (3, 300, 64, 1024, torch.float16),    # large batch: XCD-local launches over ranges of 128 rows (128 + 128 + 44)
    (4, 200, 64, 1024, torch.bfloat16),   # forward in two row ranges (128 + 72), reverse in one launch of 32-row tiles
    (3, 200, 64, 2048, torch.float16),    # register-resident kernels over two row ranges (128 + 72)
    (3, 40, 64, 512, torch.float32),
    (3, 200, 64, 1024, torch.float32),    # register-resident fp32 kernels over two row ranges (128 + 72)
    (2, 2100, 16, 96, torch.float16),     # 3 members per group: 10 groups would fit an XCD's CUs, the workspace has
                                          # barrier counters for 8 per XCD -- 66 tiles of 32 rows must not run as one launch
]


@pytest.mark.parametrize("T,B,I,H,dt", STAGE_CASES)
def test_stages_vs_oracle(oracle, T, B, I, H, dt):
    p = make_problem(T, B, I, H, seed=T * 1000 + H)
    pr = {k: (v.to(dt).double() if v is not None else None) for k, v in p.items()}  # rounded inputs
    g = {k: dev(v, dt) for k, v in p.items()}
    rm = RM[dt]
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    o_out, o_cell, o_ifgo = oracle.forward(*to_np(pr, FWD_KEYS), round_mode=rm)
    out, cell, ifgo = L.lstm_persistent_fwd(g["x"], g["h0"], g["c0"], g["Wx"], g["bx"], g["Wh"], g["bh"])
    assert out.shape == (T + 1, B, H) and cell.shape == (T + 1, B, H) and ifgo.shape == (T, B, 4 * H)
    assert torch.equal(out[0], g["h0"]) and torch.equal(cell[0], g["c0"])
    for name, got, want in (("out", out, o_out), ("cell", cell, o_cell), ("ifgo", ifgo, o_ifgo)):
        within(got, want, tol, name)
    # backward, fed with the GPU's own stored activations so that the stage is isolated
    dout, dh_n, dc_n, x, Wx, Wh = to_np(pr, ["dout", "dh_n", "dc_n", "x", "Wx", "Wh"])
    r = oracle.backward(dout, dh_n, dc_n, x, npy(out), npy(cell), npy(ifgo), Wx, Wh, round_mode=rm)
    dh_buf, dc_buf = g["dh_n"].clone(), g["dc_n"].clone()
    d_x, dh0, dc0, dWx, dbx, dWh, dbh = L.lstm_persistent_bwd(g["dout"], dc_buf, dh_buf, g["x"], out, cell, ifgo,
                                                             g["Wx"], g["Wh"])
    assert dh0 is dh_buf and dc0 is dc_buf and dbx is dbh  # in-place state grads, shared db (lstm.py:334, 501)
    for name, got, want in (("dx", d_x, r["dx"]), ("dh0", dh0, r["dh0"]), ("dc0", dc0, r["dc0"]),
                            ("dWx", dWx, r["dWx"]), ("dWh", dWh, r["dWh"]), ("db", dbx, r["db"])):
        within(got, want, tol, name)


STREAM_CASES = [
    # T, B, I, H, dtype: hidden sizes whose W_h does not fit on chip -- the weight slices are streamed every step
    # (the reference reloads its weights per step above H = 128, fastlstm/lstm.py:70-72)
    (5, 20, 64, 2560, torch.float16),     # 160 slices of 16 units, 32-row batch tile
    (4, 64, 32, 4096, torch.float16),     # 256 slices, one 64-row batch tile: every CU streams 512 KiB per step
    (5, 24, 40, 1536, torch.float32),     # fp32 past 1024
    (4, 70, 32, 2100, torch.bfloat16),    # ragged H (rows not 16-byte aligned, padded k-steps) and two batch chunks
    (3, 150, 16, 2304, torch.float16),    # three sequential launches over the batch
    (3, 16, 16, 5000, torch.float16),     # slices of 32 units
]


@pytest.mark.parametrize("T,B,I,H,dt", STREAM_CASES)
def test_streamed_weights_vs_oracle(oracle, T, B, I, H, dt):
    plan = _lib.Plan()
    _lib.check(_lib.load().fastlstm_plan_device(0, B, H, RM[dt], 0, plan), "plan")
    assert plan.wave_split == 3
    assert _lib.load().fastlstm_recurrent_kernel_kind(T, B, H, RM[dt], 0, plan.ws_bytes) == 3
    p = make_problem(T, B, I, H, seed=T * 1000 + H)
    pr = {k: (v.to(dt).double() if v is not None else None) for k, v in p.items()}
    g = {k: dev(v, dt) for k, v in p.items()}
    rm = RM[dt]
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    o_out, o_cell, o_ifgo = oracle.forward(*to_np(pr, FWD_KEYS), round_mode=rm)
    out, cell, ifgo = L.lstm_persistent_fwd(g["x"], g["h0"], g["c0"], g["Wx"], g["bx"], g["Wh"], g["bh"])
    for name, got, want in (("out", out, o_out), ("cell", cell, o_cell), ("ifgo", ifgo, o_ifgo)):
        within(got, want, tol, name)
    out_i, cell_i, _ = L.lstm_persistent_fwd(g["x"], g["h0"], g["c0"], g["Wx"], g["bx"], g["Wh"], g["bh"],
                                             keep_activations=False)
    assert torch.equal(out_i, out) and torch.equal(cell_i[-1], cell[-1])   # the inference form: same bits
    dout, dh_n, dc_n, x, Wx, Wh = to_np(pr, ["dout", "dh_n", "dc_n", "x", "Wx", "Wh"])
    r = oracle.backward(dout, dh_n, dc_n, x, npy(out), npy(cell), npy(ifgo), Wx, Wh, round_mode=rm)
    d_x, dh0, dc0, dWx, dbx, dWh, dbh = L.lstm_persistent_bwd(g["dout"], g["dc_n"].clone(), g["dh_n"].clone(), g["x"], out,
                                                             cell, ifgo, g["Wx"], g["Wh"])
    for name, got, want in (("dx", d_x, r["dx"]), ("dh0", dh0, r["dh0"]), ("dc0", dc0, r["dc0"]),
                            ("dWx", dWx, r["dWx"]), ("dWh", dWh, r["dWh"]), ("db", dbx, r["db"])):
        within(got, want, tol, name)


def _random_shape(rng):
    """One (T, B, I, H, dtype) from four families: barrier-free sizes, ragged mid sizes, the tile
    multiples that select the XCD-local / register-resident kernels, and batches of many launches'
    worth of rows."""
    import random  # noqa: F401  (rng is a random.Random)
    kind = rng.choice(["small", "mid", "mid", "tile", "tile", "bigB"])
    dt = rng.choice([torch.float32, torch.float16, torch.bfloat16])
    if kind == "small":
        return rng.randint(1, 40), rng.randint(1, 70), rng.randint(1, 90), rng.randint(1, 64), dt
    if kind == "mid":
        return rng.randint(1, 24), rng.randint(1, 130), rng.randint(1, 300), rng.randint(65, 700), dt
    if kind == "tile":
        H = rng.choice([128, 256, 384, 512, 768, 1024, 1024, 1280, 1536, 1792, 2048])
        if dt == torch.float32:
            H = min(H, 1024)
        return (rng.randint(1, 6), rng.choice([1, 8, 16, 31, 32, 33, 64, 65, 96, 128, 160, 200, 256, 300, 400]),
                rng.choice([64, 100, 256, 1024]), H, dt)
    return rng.randint(1, 4), rng.randint(200, 700), rng.randint(8, 128), rng.choice([64, 200, 256, 512, 1024]), dt


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_vs_oracle(oracle, seed):
    """40 seeded random shapes per seed through both layer entry points, each stage against the oracle
    (the backward fed with the GPU's stored activations), with the status word checked after every launch."""
    import random
    rng = random.Random(seed)
    old, L.CHECK_STATUS = L.CHECK_STATUS, True
    try:
        for case in range(40):
            T, B, I, H, dt = _random_shape(rng)
            tag = f"seed {seed} case {case}: T={T} B={B} I={I} H={H} {dt}"
            print(tag, flush=True)
            p = make_problem(T, B, I, H, seed=seed * 1000 + case)
            pr = {k: v.to(dt).double() for k, v in p.items()}
            g = {k: dev(v, dt) for k, v in p.items()}
            rm, tol = RM[dt], (FP32_TOL if dt == torch.float32 else HALF_TOL)
            o_out, o_cell, o_ifgo = oracle.forward(*to_np(pr, FWD_KEYS), round_mode=rm)
            out, cell, ifgo = L.lstm_persistent_fwd(g["x"], g["h0"], g["c0"], g["Wx"], g["bx"], g["Wh"], g["bh"])
            for name, got, want in (("out", out, o_out), ("cell", cell, o_cell), ("ifgo", ifgo, o_ifgo)):
                within(got, want, tol, (tag, name))
            dout, dh_n, dc_n, x, Wx, Wh = to_np(pr, ["dout", "dh_n", "dc_n", "x", "Wx", "Wh"])
            r = oracle.backward(dout, dh_n, dc_n, x, npy(out), npy(cell), npy(ifgo), Wx, Wh, round_mode=rm)
            got = L.lstm_persistent_bwd(g["dout"], g["dc_n"].clone(), g["dh_n"].clone(), g["x"], out, cell, ifgo,
                                        g["Wx"], g["Wh"])
            for name, k in (("dx", 0), ("dh0", 1), ("dc0", 2), ("dWx", 3), ("db", 4), ("dWh", 5)):
                within(got[k], r[name], tol, (tag, name))
    finally:
        L.CHECK_STATUS = old


@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 4, 3), (130, 260, 70), (257, 123, 515), (512, 1024, 256),
                                   (700, 1024, 256), (1120, 4096, 1024),   # T*B no multiple of 64: the tile kernel's weight-gradient loop ends past it
                                   (7200, 2112, 2624)])   # more tiles than CUs, ragged in both directions: persistent workgroups, both epilogue forms
def test_gemm_stages_vs_matmul(dt, M, N, K):
    """K1 (x.Wx^T + b), K5 (d.Wx) and K8/K9 (d^T.x) against float64 matmul; shapes chosen
    so that T*B = M, 4H = N (K1) etc. hit ragged tiles, unaligned rows and split-K."""
    # (fp32, the 7200-term case: a sum of 7200 products of unit-variance terms carries ~3e-4 of fp32 rounding whatever
    # the order, so the element-wise 1e-4 bound says nothing about the kernel there: max-norm only)
    within = globals()["within"] if not (dt == torch.float32 and M > 4096) else (
        lambda got, want, tol, what=None: _max_norm_only(got, want, tol))
    lib = _lib.load()
    g = torch.Generator().manual_seed(M + N + K)
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    H = max(1, N // 4)
    T, B, I = 1, M, K
    x = torch.randn(T, B, I, generator=g).to(dt).cuda()
    Wx = (torch.randn(4 * H, I, generator=g) * 0.1).to(dt).cuda()
    bx = torch.randn(4 * H, generator=g).to(dt).cuda()
    bh = torch.randn(4 * H, generator=g).to(dt).cuda()
    code = RM[dt]
    st = torch.cuda.current_stream().cuda_stream
    ifgo = torch.empty(T, B, 4 * H, dtype=dt, device="cuda")
    _lib.check(lib.fastlstm_gemm_ifgo(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), ifgo.data_ptr(),
                                      T, B, I, H, code, st), "k1")
    want = x.double().view(B, I) @ Wx.double().T + bx.double() + bh.double()
    within(ifgo.reshape(B, -1), want, tol)
    d = torch.randn(T, B, 4 * H, generator=g).to(dt).cuda()
    dx = torch.empty(T, B, I, dtype=dt, device="cuda")
    _lib.check(lib.fastlstm_gemm_dx(d.data_ptr(), Wx.data_ptr(), dx.data_ptr(), T, B, I, H, code, st), "k5")
    want = d.double().view(B, -1) @ Wx.double()
    within(dx.reshape(B, I), want, tol)
    scratch = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")   # ... split along K where that fills the device
    dx.zero_()
    _lib.check(lib.fastlstm_gemm_dx_split(d.data_ptr(), Wx.data_ptr(), dx.data_ptr(), T, B, I, H, code,
                                          scratch.data_ptr(), scratch.numel(), st), "k5 split")
    within(dx.reshape(B, I), want, tol)
    h = torch.randn(T + 1, B, H, generator=g).to(dt).cuda()
    dbx, dbh, dWx, dWh = L.Wgrad(d, x, h)
    assert dbx is dbh
    d2 = d.double().view(B, -1)
    within(dWx, (d2.T @ x.double().view(B, I)), tol)
    within(dWh, (d2.T @ h[:-1].double().view(B, H)), tol)
    within(dbx, d2.sum(0), tol)


@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,B,I,H", [(64, 64, 64, 64),      # whole blocks, every tile in use
                                     (100, 33, 32, 48),     # last block ragged (3300 rows), unused G, I and H tiles
                                     (30, 20, 16, 16),      # one G tile per wave pair, one column tile
                                     (256, 256, 64, 64),    # more blocks than workgroups: accumulators carried over blocks
                                     (9, 20, 64, 64),       # fewer rows than the one-pass form takes
                                     (40, 40, 80, 64),      # I too wide for it
                                     (40, 40, 64, 128)])    # H too wide for it
@pytest.mark.parametrize("want", ["all", "dx", "dw"])
def test_gemm_dx_wgrad_vs_matmul(dt, T, B, I, H, want):
    """fastlstm_gemm_dx_wgrad (one pass over d_ifgo for narrow 16-bit layers, the two stages otherwise) against float64
    matmul, with either half of the results not asked for; what is not asked for stays untouched."""
    if want != "all" and (T, B) not in ((100, 33), (40, 40)):
        pytest.skip("the partial forms on one shape per path")
    lib = _lib.load()
    code, tol = RM[dt], (FP32_TOL if dt == torch.float32 else HALF_TOL)
    g = torch.Generator().manual_seed(T * 7 + B * 5 + I * 3 + H)
    d = (torch.randn(T, B, 4 * H, generator=g) * 0.5).to(dt).cuda()
    x = torch.randn(T, B, I, generator=g).to(dt).cuda()
    h = (torch.rand(T + 1, B, H, generator=g) * 2 - 1).to(dt).cuda()
    Wx = (torch.randn(4 * H, I, generator=g) * 0.2).to(dt).cuda()
    nb = lib.fastlstm_wgrad_workspace_bytes(T, B, I, H, code)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    mark = 12345.0
    dx = torch.full((T, B, I), mark, dtype=dt, device="cuda")
    dWx, dWh, db = (torch.full(sh, mark, dtype=dt, device="cuda") for sh in ((4 * H, I), (4 * H, H), (4 * H,)))
    w_dx, w_dw = want in ("all", "dx"), want in ("all", "dw")
    _lib.check(lib.fastlstm_gemm_dx_wgrad(d.data_ptr(), Wx.data_ptr(), x.data_ptr(), h.data_ptr(), dx.data_ptr() if w_dx else None,
                                          dWx.data_ptr() if w_dw else None, dWh.data_ptr() if w_dw else None,
                                          db.data_ptr() if w_dw else None, ws.data_ptr(), nb, T, B, I, H, code,
                                          torch.cuda.current_stream().cuda_stream), "fastlstm_gemm_dx_wgrad")
    D = d.double().view(T * B, -1)
    if want == "all":   # K1 on the same shape (I no multiple of 64 and a narrow layer: the streaming form)
        bx, bh = torch.randn(4 * H, generator=g).to(dt).cuda(), torch.randn(4 * H, generator=g).to(dt).cuda()
        ifgo = torch.full((T, B, 4 * H), mark, dtype=dt, device="cuda")
        _lib.check(lib.fastlstm_gemm_ifgo(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), ifgo.data_ptr(), T, B, I, H,
                                          code, torch.cuda.current_stream().cuda_stream), "fastlstm_gemm_ifgo")
        within(ifgo.view(T * B, -1), x.double().view(T * B, I) @ Wx.double().T + bx.double() + bh.double(), tol)
    if w_dx:
        within(dx.view(T * B, I), D @ Wx.double(), tol)
        dx2 = torch.full_like(dx, mark)   # K5 by its own entry point (a narrow layer: the same streaming pass, dx alone)
        _lib.check(lib.fastlstm_gemm_dx(d.data_ptr(), Wx.data_ptr(), dx2.data_ptr(), T, B, I, H, code,
                                        torch.cuda.current_stream().cuda_stream), "fastlstm_gemm_dx")
        within(dx2.view(T * B, I), D @ Wx.double(), tol)
    else:
        assert bool((dx == mark).all())
    if w_dw:
        within(dWx, D.T @ x.double().view(T * B, I), tol)
        within(dWh, D.T @ h[:T].double().reshape(T * B, H), tol)
        within(db, D.sum(0), tol)
    else:
        assert all(bool((t == mark).all()) for t in (dWx, dWh, db))
    if w_dx and w_dw:   # the host wrapper, same call
        got = L.DxWgrad(d, Wx, x, h)
        assert got[1] is got[2]
        for a, b_ in zip((got[0], got[1], got[3], got[4]), (dx, db, dWx, dWh)):
            assert torch.equal(a, b_)


def test_gemm_earlier_form_switch_agrees():
    """fastlstm_set_gemm_baseline(1): the stand-alone products in the tile kernel's earlier form (what bench.py times
    beside the current one) -- same results to rounding, and the switch goes back."""
    lib = _lib.load()
    dt, code = torch.float16, RM[torch.float16]
    T, B, I, H = 4, 320, 512, 256
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, B, I, generator=g).to(dt).cuda()
    Wx = (torch.randn(4 * H, I, generator=g) * 0.1).to(dt).cuda()
    bx, bh = torch.randn(4 * H, generator=g).to(dt).cuda(), torch.randn(4 * H, generator=g).to(dt).cuda()
    d = torch.randn(T, B, 4 * H, generator=g).to(dt).cuda()
    h = torch.randn(T + 1, B, H, generator=g).to(dt).cuda()
    st = torch.cuda.current_stream().cuda_stream
    res = []
    try:
        for on in (0, 1):
            lib.fastlstm_set_gemm_baseline(on)
            ifgo = torch.empty(T, B, 4 * H, dtype=dt, device="cuda")
            dx = torch.empty(T, B, I, dtype=dt, device="cuda")
            _lib.check(lib.fastlstm_gemm_ifgo(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), ifgo.data_ptr(),
                                              T, B, I, H, code, st), "k1")
            _lib.check(lib.fastlstm_gemm_dx(d.data_ptr(), Wx.data_ptr(), dx.data_ptr(), T, B, I, H, code, st), "k5")
            res.append((ifgo, dx) + tuple(L.Wgrad(d, x, h)[1:]))
    finally:
        lib.fastlstm_set_gemm_baseline(0)
    torch.cuda.synchronize()
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])   # same products in the same order
    for a, b in zip(res[0][2:], res[1][2:]):
        within(a, b.double(), HALF_TOL)
    want = x.double().view(T * B, I) @ Wx.double().T + bx.double() + bh.double()
    within(res[1][0].reshape(T * B, -1), want, HALF_TOL)


def test_gpu_matches_golden_vectors():
    z = np.load(os.path.join(ROOT, "tests", "golden", "lstm_golden.npz"))
    for name in ("tiny", "ragged", "nostate", "onestep"):
        t = lambda k: torch.from_numpy(z["%s/in/%s" % (name, k)]).cuda() if "%s/in/%s" % (name, k) in z.files else None
        x, h0, c0 = t("x").requires_grad_(True), t("h0"), t("c0")
        ws = [t(k).requires_grad_(True) for k in ("Wx", "bx", "Wh", "bh")]
        if h0 is not None:
            h0.requires_grad_(True); c0.requires_grad_(True)
        out, (hn, cn) = PersistentLSTMfn.apply(x, h0, c0, *ws)
        assert_close32(out, z[name + "/out/out"])
        assert_close32(hn, z[name + "/out/h_n"])
        assert_close32(cn, z[name + "/out/c_n"])
        # the fixture's gradients belong to loss = sum(out*dout) + sum(h_n*dh_n) + sum(c_n*dc_n): the
        # differentiable-state Function delivers dh_n / dc_n to the reverse kernel
        out, hn, cn = L.PersistentLSTMStatefn.apply(x, h0, c0, *ws)
        ((out * t("dout")).sum() + (hn * t("dh_n")).sum() + (cn * t("dc_n")).sum()).backward()
        grads = [("dx", x), ("dWx", ws[0]), ("dbx", ws[1]), ("dWh", ws[2]), ("dbh", ws[3])]
        if h0 is not None:
            grads += [("dh0", h0), ("dc0", c0)]
        for key, leaf in grads:
            assert_close32(leaf.grad, z["%s/out/%s" % (name, key)])


# --------------------------------------------------------------------------------------
# 3. autograd boundary semantics (fastlstm/lstm.py:504-538)
# --------------------------------------------------------------------------------------
def test_autograd_function_contract():
    T, B, I, H = 6, 5, 9, 20
    p = make_problem(T, B, I, H, seed=3, dtype=torch.float32)
    ref = nn_lstm_reference(p, with_state_grads=False, dtype=torch.float32)
    x = p["x"].cuda().requires_grad_(True)
    h0, c0 = p["h0"].cuda().requires_grad_(True), p["c0"].cuda().requires_grad_(True)
    Wx, bx, Wh, bh = (p[k].cuda().requires_grad_(True) for k in ("Wx", "bx", "Wh", "bh"))
    out, (hn, cn) = PersistentLSTMfn.apply(x, h0, c0, Wx, bx, Wh, bh)
    assert out.shape == (T, B, H) and hn.shape == (B, H) and cn.shape == (B, H)
    (out * p["dout"].cuda()).sum().backward()
    for got, key in ((x.grad, "dx"), (h0.grad, "dh0"), (c0.grad, "dc0"), (Wx.grad, "dWx"), (Wh.grad, "dWh"),
                     (bx.grad, "dbx"), (bh.grad, "dbh")):
        assert_close32(got, ref[key])
    # h_0 = None: no state gradients, zeros initial state (lstm.py:535-537)
    x2 = p["x"].cuda().requires_grad_(True)
    out2, _ = PersistentLSTMfn.apply(x2, None, None, Wx, bx, Wh, bh)
    out0, _ = PersistentLSTMfn.apply(x2, torch.zeros(B, H).cuda(), torch.zeros(B, H).cuda(), Wx, bx, Wh, bh)
    assert torch.equal(out2, out0)
    # 2-D input is one timestep (lstm.py:33-34) == nn.LSTMCell
    o1, (h1, c1) = PersistentLSTMfn.apply(p["x"][0].cuda(), h0, c0, Wx, bx, Wh, bh)
    cellm = torch.nn.LSTMCell(I, H)
    with torch.no_grad():
        cellm.weight_ih.copy_(p["Wx"]); cellm.weight_hh.copy_(p["Wh"]); cellm.bias_ih.copy_(p["bx"]); cellm.bias_hh.copy_(p["bh"])
        hr, cr = cellm(p["x"][0], (p["h0"], p["c0"]))
    assert o1.shape == (1, B, H)
    assert_close32(h1, hr); assert_close32(c1, cr)


@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16])
def test_prepare_forward_clears_the_workspace_and_sets_the_initial_state(dt):
    """fastlstm_prepare_forward = `ws[:n].zero_(); out[0] = h0; cell[0] = c0` (or zeros) in one launch."""
    lib = _lib.load()
    B, H, code = 37, 72, RM[dt]
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device="cuda").manual_seed(5)
    for with_state in (True, False):
        ws = torch.full((70000,), 0xAB, dtype=torch.uint8, device="cuda")
        out = torch.randn(3, B, H, device="cuda", generator=g).to(dt)
        cell = torch.randn(3, B, H, device="cuda", generator=g).to(dt)
        out_before, cell_before = out.clone(), cell.clone()
        h0 = torch.randn(B, H, device="cuda", generator=g).to(dt) if with_state else None
        c0 = torch.randn(B, H, device="cuda", generator=g).to(dt) if with_state else None
        _lib.check(lib.fastlstm_prepare_forward(ws.data_ptr(), 66560, out.data_ptr(), cell.data_ptr(),
                                                h0.data_ptr() if with_state else None, c0.data_ptr() if with_state else None,
                                                B, H, code, st), "prepare")
        torch.cuda.synchronize()
        assert int(ws[:66560].max()) == 0 and int(ws[66560:].min()) == 0xAB
        assert torch.equal(out[0], h0 if with_state else torch.zeros_like(out[0]))
        assert torch.equal(cell[0], c0 if with_state else torch.zeros_like(cell[0]))
        assert torch.equal(out[1:], out_before[1:]) and torch.equal(cell[1:], cell_before[1:])
    assert lib.fastlstm_prepare_forward(ws.data_ptr(), 64, out.data_ptr(), cell.data_ptr(), out.data_ptr(), None,
                                        B, H, code, st) == _lib.ERR_NULL


def test_module_takes_a_state_of_another_dtype_and_layout():
    """An initial state that is not a dense tensor of the compute dtype goes through torch's conversion
    (`out[0] = h_0`, fastlstm/lstm.py:88-90) instead of the one-launch preparation: same results."""
    torch.manual_seed(11)
    m = FastLSTM(24, 40).to("cuda", torch.float16)
    x = torch.randn(6, 5, 24, device="cuda", dtype=torch.float16)
    h0 = torch.randn(1, 5, 40, device="cuda") * 0.3
    c0 = torch.randn(1, 40, 5, device="cuda").transpose(1, 2) * 0.3          # strided, fp32
    y1, (h1, c1) = m(x, (h0, c0))
    y2, (h2, c2) = m(x, (h0.half(), c0.half().contiguous()))
    assert torch.equal(y1, y2) and torch.equal(h1, h2) and torch.equal(c1, c2)


def test_recurrence_vanishes_with_zero_wh(oracle):
    T, B, I, H = 5, 20, 32, 96
    p = make_problem(T, B, I, H, seed=5, dtype=torch.float32)
    p["Wh"] = torch.zeros_like(p["Wh"])
    out, cell, ifgo = L.lstm_persistent_fwd(*(dev(p[k]) for k in FWD_KEYS))
    pre = torch.nn.functional.linear(p["x"].double(), p["Wx"].double(), (p["bx"] + p["bh"]).double())
    assert_close32(ifgo, pre)


def test_runs_are_bit_reproducible():
    T, B, I, H = 12, 48, 64, 320
    p = make_problem(T, B, I, H, seed=8, dtype=torch.float16)
    g = {k: dev(v) for k, v in p.items()}
    res = []
    for _ in range(2):
        out, cell, ifgo = L.lstm_persistent_fwd(*(g[k] for k in FWD_KEYS))
        r = L.lstm_persistent_bwd(g["dout"], g["dc_n"].clone(), g["dh_n"].clone(), g["x"], out, cell, ifgo, g["Wx"], g["Wh"])
        res.append([out, cell, ifgo, *r])
    for a, b in zip(*res):
        assert torch.equal(a, b)


def test_backward_is_linear_in_upstream_gradient():
    T, B, I, H = 10, 16, 48, 128
    p = make_problem(T, B, I, H, seed=9, dtype=torch.float32)
    g = {k: dev(v) for k, v in p.items()}
    out, cell, ifgo = L.lstm_persistent_fwd(*(g[k] for k in FWD_KEYS))
    z = lambda: torch.zeros(B, H, device="cuda")
    a = L.lstm_persistent_bwd(g["dout"], z(), z(), g["x"], out, cell, ifgo, g["Wx"], g["Wh"])
    b = L.lstm_persistent_bwd(g["dout"] * 2, z(), z(), g["x"], out, cell, ifgo, g["Wx"], g["Wh"])
    for u, v in zip(a, b):
        torch.testing.assert_close(v, 2 * u, rtol=1e-5, atol=1e-6)


def test_batch_larger_than_one_launch(oracle):
    """B = 1100 with H = 1024 needs more than one launch of the barrier groups
    (batch_chunks > 1, kernels.py:514/663 of the reference)."""
    T, B, I, H = 2, 1100, 16, 1024
    plan = _lib.Plan()
    _lib.check(_lib.load().fastlstm_plan_device(0, B, H, 1, 0, plan), "plan")
    assert plan.batch_chunks > 1
    p = make_problem(T, B, I, H, seed=12)
    dt = torch.float16
    pr = {k: (v.to(dt).double() if v is not None else None) for k, v in p.items()}
    g = {k: dev(v, dt) for k, v in p.items()}
    o_out, o_cell, _ = oracle.forward(*to_np(pr, FWD_KEYS), round_mode=1)
    out, cell, ifgo = L.lstm_persistent_fwd(*(g[k] for k in FWD_KEYS))
    assert rel_err(out, o_out) < HALF_TOL
    r = oracle.backward(*to_np(pr, ["dout", "dh_n", "dc_n", "x"]), npy(out), npy(cell), npy(ifgo),
                        *to_np(pr, ["Wx", "Wh"]), round_mode=1)
    res = L.lstm_persistent_bwd(g["dout"], g["dc_n"].clone(), g["dh_n"].clone(), g["x"], out, cell, ifgo, g["Wx"], g["Wh"])
    assert rel_err(res[1], r["dh0"]) < HALF_TOL
    assert rel_err(res[5], r["dWh"]) < HALF_TOL


def test_autocast_and_training_step():
    """Mixed precision as scripts/overfit.py of the reference uses it: fp32 parameters,
    autocast to bf16 inside the Function (lstm.py:509-515), fp32 gradients back."""
    torch.manual_seed(0)
    m = FastLSTM(24, 96).cuda()
    head = torch.nn.Linear(96, 1).cuda()
    opt = torch.optim.Adam(list(m.parameters()) + list(head.parameters()), lr=1e-2)
    x = torch.randn(20, 8, 24).cuda()
    y = torch.randn(20, 8, 1).cuda()
    losses = []
    for _ in range(30):
        opt.zero_grad()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, (hn, cn) = m(x)
            assert out.dtype == torch.bfloat16
            loss = torch.nn.functional.mse_loss(head(out).float(), y)
        loss.backward()
        assert m.weight_hh_l0.grad.dtype == torch.float32
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < 0.7 * losses[0], losses


def test_barrier_timeout_is_reported_not_hung():
    """Failure path forced from the host: with a spin limit of one tick a wait that is not
    satisfied at its first poll gives up, raises the abort flag (which ends every other
    wait too) and the grid drains; the status word reports it.  The kernel exits normally."""
    lib = _lib.load()
    T, B, H, code = 64, 16, 512, 1
    plan = _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 0, plan), "plan")
    assert plan.n_htiles > 1
    ifgo = torch.randn(T, B, 4 * H, device="cuda").half()
    out = torch.zeros(T + 1, B, H, device="cuda").half()
    cell = torch.zeros(T + 1, B, H, device="cuda").half()
    Wh = (torch.randn(4 * H, H, device="cuda") * 0.03).half()
    st = torch.cuda.current_stream().cuda_stream

    def launch():
        ws = torch.zeros(plan.ws_bytes, dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_fwd_persistent(ifgo.clone().data_ptr(), out.data_ptr(), cell.data_ptr(), Wh.data_ptr(),
                                               ws.data_ptr(), ws.numel(), T, B, H, code, st), "fwd")
        torch.cuda.synchronize()  # returns: the grid drained
        return lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes())

    try:
        lib.fastlstm_set_spin_limit(1)
        assert launch() == _lib.ERR_TIMEOUT
    finally:
        lib.fastlstm_set_spin_limit(400000000)
    # the device's sticky status word saw it too (no sync needed to read it); the next entry point on the
    # device reports the failure once, before launching anything, and the one after is healthy
    assert lib.fastlstm_device_status(0, 0) == _lib.ERR_TIMEOUT
    ws = torch.zeros(plan.ws_bytes, dtype=torch.uint8, device="cuda")
    args = (ifgo.clone().data_ptr(), out.data_ptr(), cell.data_ptr(), Wh.data_ptr(), ws.data_ptr(), ws.numel(), T, B, H, code, st)
    assert lib.fastlstm_fwd_persistent(*args) == _lib.ERR_TIMEOUT
    assert lib.fastlstm_device_status(0, 0) == _lib.OK
    assert launch() == _lib.OK  # and the next launch is healthy
    assert lib.fastlstm_device_status(0, 0) == _lib.OK
    assert torch.isfinite(out.float()).all()


WIDE_CASES = [
    # T, B, H, dtype: hidden sizes whose barrier groups span several XCDs (weights in registers, 64-row groups)
    (5, 128, 2048, torch.bfloat16),   # config C's B and H: two groups of 128 workgroups
    (4, 100, 1536, torch.float16),    # 96 workgroups per group, ragged second group
    (3, 40, 2048, torch.float16),     # one partly filled group
    (4, 128, 1280, torch.float16),    # 80 workgroups per group over three XCDs, the third partly used
    (3, 70, 1792, torch.bfloat16),    # 112 workgroups per group over four XCDs
    (6, 128, 1536, torch.bfloat16),   # two full groups of three XCDs
    # batches that fit the launch as groups of 16 rows (one batch tile per workgroup)
    (4, 32, 2048, torch.bfloat16),    # two 16-row groups of four XCDs each
    (3, 20, 1536, torch.float16),     # ragged second group
    (3, 9, 1792, torch.bfloat16),     # one partly filled group
    (4, 32, 1280, torch.float16),     # three XCDs per group, the third partly used
    # ... and as groups of 32 rows
    (3, 64, 2048, torch.float16),
    (4, 50, 1536, torch.bfloat16),    # ragged second group
    # fp32 at H = 640 ... 1024 (the same bytes per weight row): groups of 16 or 32 rows on two XCDs
    (4, 64, 1024, torch.float32),     # four 16-row groups
    (3, 100, 768, torch.float32),     # 32-row groups, the last one ragged
    (3, 20, 640, torch.float32),      # the second XCD of a group partly used
]


@pytest.mark.parametrize("T,B,H,dt", WIDE_CASES)
def test_wide_kernels_agree_with_general_kernels_and_oracle(oracle, T, B, H, dt):
    """H = 1280 ... 2048 (fp32: 640 ... 1024): the C ABI runs the register-resident kernels whose groups span several XCDs
    (kernel kind 2), or -- with that family switched off -- the general kernels; both must meet the
    oracle on the same inputs.  So must both forms of the reverse kernel for groups of 64 rows: every
    workgroup sums over all of K, or teams of workgroups split K and exchange partial sums."""
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dt]
    rm = RM[dt]
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    p = make_problem(T, B, 64, H, seed=5 + H + B)
    pr = {k: (v.to(dt).double() if v is not None else None) for k, v in p.items()}
    g = {k: dev(v, dt) for k, v in p.items()}
    o_out, o_cell, o_ifgo = oracle.forward(*to_np(pr, FWD_KEYS), round_mode=rm)
    st = torch.cuda.current_stream().cuda_stream
    plans = [_lib.Plan(), _lib.Plan()]
    for bw in (0, 1):
        _lib.check(lib.fastlstm_plan_device(0, B, H, code, bw, plans[bw]), "plan")
    ifgo0 = torch.empty(T, B, 4 * H, device="cuda", dtype=dt)
    _lib.check(lib.fastlstm_gemm_ifgo(g["x"].data_ptr(), g["Wx"].data_ptr(), g["bx"].data_ptr(), g["bh"].data_ptr(),
                                      ifgo0.data_ptr(), T, B, 64, H, code, st), "k1")
    results = {}
    for kind in ("general", "wide", "teams"):
        lib.fastlstm_set_kernel_families({"general": 0, "wide": 3, "teams": 7}[kind])
        sizes = [lib.fastlstm_recurrent_workspace_bytes(plans[bw], T, H, code, bw) for bw in (0, 1)]
        small32 = dt == torch.float32 and B <= 32   # (a small fp32 batch keeps the general forward kernel)
        assert lib.fastlstm_recurrent_kernel_kind(T, B, H, code, 0, sizes[0]) == (0 if kind == "general" or small32 else 2)
        assert lib.fastlstm_recurrent_kernel_kind(T, B, H, code, 1, sizes[1]) in ((0,) if kind == "general" else (0, 2))
        ifgo = ifgo0.clone()
        out = torch.empty(T + 1, B, H, device="cuda", dtype=dt)
        cell = torch.empty_like(out)
        out[0], cell[0] = g["h0"], g["c0"]
        ws = torch.zeros(sizes[0], dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_fwd_persistent(ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), g["Wh"].data_ptr(),
                                               ws.data_ptr(), ws.numel(), T, B, H, code, st), "fwd")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK
        for name, got, want in (("out", out, o_out), ("cell", cell, o_cell), ("ifgo", ifgo, o_ifgo)):
            within(got, want, tol, (kind, name))
        d_ifgo = torch.empty_like(ifgo)
        dh, dc = g["dh_n"].clone(), g["dc_n"].clone()
        wsb = torch.zeros(sizes[1], dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_bwd_persistent(g["dout"].data_ptr(), dh.data_ptr(), dc.data_ptr(), ifgo.data_ptr(),
                                               cell.data_ptr(), d_ifgo.data_ptr(), g["Wh"].data_ptr(), wsb.data_ptr(),
                                               wsb.numel(), T, B, H, code, st), "bwd")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(wsb[:64].cpu().numpy().tobytes()) == _lib.OK
        dout, dh_n, dc_n, x, Wx, Wh = to_np(pr, ["dout", "dh_n", "dc_n", "x", "Wx", "Wh"])
        r = oracle.backward(dout, dh_n, dc_n, x, npy(out), npy(cell), npy(ifgo), Wx, Wh, round_mode=rm)
        for name, got, want in (("d_ifgo", d_ifgo, r["d_ifgo"]), ("dh0", dh, r["dh0"]), ("dc0", dc, r["dc0"])):
            within(got, want, tol, (kind, name))
        results[kind] = (out, cell, ifgo, d_ifgo, dh, dc)
    for other in ("wide", "teams"):
        for a, b in zip(results["general"], results[other]):   # other summation orders of the same sums
            within(a, b, tol)


@pytest.mark.parametrize("H,dt", [(2048, torch.bfloat16), (1280, torch.float16), (1024, torch.float32), (640, torch.float32)])
def test_register_resident_kernels_at_the_batch_sizes_where_their_form_changes(H, dt):
    """Rows per group (16, 32, 64), launches over row ranges, the team form of the reverse kernel and the fp32
    limits all switch on the batch size: around every threshold the C ABI's choice must agree with the general
    kernels on the same inputs (outputs, states, stored activations, d_ifgo and the state gradients)."""
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dt]
    tol = 2 * FP32_TOL if dt == torch.float32 else HALF_TOL
    st = torch.cuda.current_stream().cuda_stream
    T = 3

    def run(B, families):
        lib.fastlstm_set_kernel_families(families)
        gen = torch.Generator(device="cuda").manual_seed(B * 7 + H)
        rnd = lambda *shape, s=1.0: (torch.randn(*shape, device="cuda", generator=gen) * s).to(dt)
        ifgo, Wh = rnd(T, B, 4 * H, s=0.5), rnd(4 * H, H, s=H ** -0.5)
        out = torch.zeros(T + 1, B, H, device="cuda", dtype=dt)
        cell = torch.zeros_like(out)
        out[0], cell[0] = rnd(B, H, s=0.1), rnd(B, H, s=0.1)
        plans = [_lib.Plan(), _lib.Plan()]
        ws = []
        for bw in (0, 1):
            _lib.check(lib.fastlstm_plan_device(0, B, H, code, bw, plans[bw]), "plan")
            ws.append(torch.zeros(lib.fastlstm_recurrent_workspace_bytes(plans[bw], T, H, code, bw), dtype=torch.uint8, device="cuda"))
        kinds = tuple(lib.fastlstm_recurrent_kernel_kind(T, B, H, code, bw, ws[bw].numel()) for bw in (0, 1))
        _lib.check(lib.fastlstm_fwd_persistent(ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), Wh.data_ptr(),
                                               ws[0].data_ptr(), ws[0].numel(), T, B, H, code, st), "fwd")
        dout, d_ifgo = rnd(T, B, H), torch.empty_like(ifgo)
        dh, dc = rnd(B, H, s=0.1), rnd(B, H, s=0.1)
        _lib.check(lib.fastlstm_bwd_persistent(dout.data_ptr(), dh.data_ptr(), dc.data_ptr(), ifgo.data_ptr(), cell.data_ptr(),
                                               d_ifgo.data_ptr(), Wh.data_ptr(), ws[1].data_ptr(), ws[1].numel(), T, B, H, code, st), "bwd")
        torch.cuda.synchronize()
        for w in ws:
            assert lib.fastlstm_ws_status(w[:64].cpu().numpy().tobytes()) == _lib.OK
        return kinds, (out, cell, ifgo, d_ifgo, dh, dc)

    seen = set()
    for B in (1, 16, 17, 32, 33, 64, 65, 128, 129, 144, 260):
        kinds0, want = run(B, 0)
        kinds, got = run(B, 7)
        assert kinds0 == (0, 0) and kinds[1] == 2, (B, kinds0, kinds)
        seen.add(kinds)
        for name, a, b in zip(("out", "cell", "ifgo", "d_ifgo", "dh0", "dc0"), got, want):
            within(a, npy(b), tol, (B, name))
    assert (2, 2) in seen


@pytest.mark.parametrize("kw", [dict(num_layers=2), dict(num_layers=3, bidirectional=True)])
def test_dropout_between_layers(kw):
    """nn.LSTM's `dropout`: on the outputs of every layer but the last, in training mode only.  (MIOpen draws its
    own mask, so the check is against the same layers composed by hand under the same seed.)"""
    T, B, I, H, dt, p = 7, 16, 24, 128, torch.float16, 0.4
    torch.manual_seed(3)
    m = FastLSTM(I, H, dropout=p, **kw).to("cuda", dt)
    plain = FastLSTM(I, H, **kw).to("cuda", dt)
    plain.load_state_dict(m.state_dict())
    x = torch.randn(T, B, I, device="cuda", dtype=dt)
    m.eval()
    plain.eval()
    assert torch.equal(m(x)[0], plain(x)[0])            # no dropout outside training
    m.train()
    plain.train()
    D = 2 if kw.get("bidirectional") else 1
    singles = []
    for layer in range(kw["num_layers"]):
        one = FastLSTM(I if layer == 0 else D * H, H, bidirectional=D == 2).to("cuda", dt)
        sd = {k.replace("_l%d" % layer, "_l0"): v for k, v in m.state_dict().items() if "_l%d" % layer in k}
        one.load_state_dict(sd)
        singles.append(one.train())
    torch.manual_seed(17)
    got, (h_n, _) = m(x)
    torch.manual_seed(17)
    y = x
    for layer, one in enumerate(singles):
        y = one(y)[0]
        if layer + 1 < len(singles):
            y = torch.nn.functional.dropout(y, p, True)
    assert torch.equal(got, y)
    assert not torch.equal(got, plain(x)[0])
    assert h_n.shape == (kw["num_layers"] * D, B, H)
    got.float().sum().backward()
    assert all(q.grad is not None and torch.isfinite(q.grad.float()).all() for q in m.parameters())
    with pytest.raises(ValueError):
        FastLSTM(I, H, dropout=1.0)


PAIR_CASES = [
    # T, B, I, H, dtype, one launch expected
    (6, 32, 96, 512, torch.float16, True),
    (5, 40, 64, 256, torch.float32, True),
    (4, 64, 128, 1024, torch.bfloat16, True),     # config B's tiles: 4 + 4 groups on the 8 XCDs
    (3, 200, 64, 1024, torch.float16, False),     # 7 + 7 groups of 32 rows do not fit: one after the other
    (4, 24, 48, 72, torch.float16, False),        # general kernels: one after the other
    (5, 16, 64, 2048, torch.bfloat16, True),      # register-resident kernels: one 16-row group each, 4 XCDs per group
    (4, 32, 64, 1536, torch.float16, True),       # ... one 32-row group each on 3 XCDs (alone: two 16-row groups)
    (3, 24, 64, 1024, torch.float32, True),       # ... fp32
    (3, 64, 64, 2048, torch.float16, False),      # 64-row groups: one after the other
    (6, 200, 48, 64, torch.float16, True),        # one hidden tile per workgroup: both recurrences' workgroups in one grid
    (3, 600, 32, 64, torch.bfloat16, True),       # ... of 8-row batch tiles (2 x 150 of 4 rows are more than the CUs)
    (5, 33, 16, 32, torch.float32, True),
]


@pytest.mark.parametrize("T,B,I,H,dt,fused", PAIR_CASES)
def test_two_recurrences_side_by_side_equal_two_calls(T, B, I, H, dt, fused):
    """fastlstm_fwd_persistent_pair / fastlstm_bwd_persistent_pair (the two directions of a bidirectional layer in
    one launch) against two calls of the single-layer ops on the same operands: the same kernels do the same sums
    in the same order, so the time loops' results are the same bits; dx and the weight gradients come from
    stand-alone GEMM launches here and from the layer call there (another order of the same sums)."""
    assert L.pair_runs_in_one_launch(T, B, H, dt, "cuda") == fused
    assert L.pair_runs_in_one_launch(T, B, H, dt, "cuda", backward=True) == fused
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    sides = []
    for seed in (11, 12):
        p = make_problem(T, B, I, H, seed=seed + H)
        sides.append({k: dev(v, dt) for k, v in p.items()})
    a, b = sides
    fwd_keys = ("x", "h0", "c0", "Wx", "bx", "Wh", "bh")
    got = L.lstm_persistent_fwd_pair(*(a[k] for k in fwd_keys), *(b[k] for k in fwd_keys))
    want = L.lstm_persistent_fwd(*(a[k] for k in fwd_keys)) + L.lstm_persistent_fwd(*(b[k] for k in fwd_keys))
    # (the register-resident kernels take 32-row groups for two recurrences where one alone gets 16-row groups: the
    # eight partial sums of a tile are then added starting from another wave's -- fp32 results agree to rounding)
    same_bits = lambda x_, y_: torch.equal(x_, y_) if not (dt == torch.float32 and H >= 640) else rel_err(x_, npy(y_)) < 1e-6
    for name, g_, w_ in zip(("out_a", "cell_a", "ifgo_a", "out_b", "cell_b", "ifgo_b"), got, want):
        assert same_bits(g_, w_), name
    ga, gb = L.lstm_persistent_bwd_pair(a["dout"], (a["dh_n"], a["dc_n"]), a["x"], got[0], got[1], got[2], a["Wx"], a["Wh"],
                                        b["dout"], (b["dh_n"], b["dc_n"]), b["x"], got[3], got[4], got[5], b["Wx"], b["Wh"])
    for side, g_, (out, cell, ifgo) in ((a, ga, want[:3]), (b, gb, want[3:])):
        w_ = L.lstm_persistent_bwd(side["dout"], side["dc_n"].clone(), side["dh_n"].clone(), side["x"], out, cell, ifgo,
                                   side["Wx"], side["Wh"])
        for name, x_, y_ in zip(("d_x", "dh_0", "dc_0", "dWx", "dbx", "dWh", "dbh"), g_, w_):
            if name in ("dh_0", "dc_0"):
                assert same_bits(x_, y_), name
            else:
                within(x_, npy(y_), tol, name)


XCD_CASES = [
    # T, B, H, dtype          (hidden tile, members, batch tiles) of the XCD-local launch
    (20, 64, 1024, torch.float16),    # config B: 32 units x 32 members, 8 waves
    (9, 40, 512, torch.bfloat16),     # 16 units x 32 members, ragged batch
    (7, 100, 256, torch.float32),     # fp32, 7 batch tiles on 7 XCDs
    (5, 300, 256, torch.float16),     # 32-row batch tiles, two groups per XCD
    (6, 16, 128, torch.float16),      # small H: 8 units (forward) / 16 units (backward) per workgroup
]


@pytest.mark.parametrize("T,B,H,dt", XCD_CASES)
def test_xcd_local_kernels_agree_with_general_kernels_and_oracle(oracle, T, B, H, dt):
    """The C ABI picks the XCD-local kernels where the shape allows, and the general kernels when that
    family is switched off; both must meet the oracle, on the same inputs."""
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dt]
    rm = RM[dt]
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    p = make_problem(T, B, H, H, seed=77 + H)
    pr = {k: (v.to(dt).double() if v is not None else None) for k, v in p.items()}
    g = {k: dev(v, dt) for k, v in p.items()}
    o_out, o_cell, o_ifgo = oracle.forward(*to_np(pr, FWD_KEYS), round_mode=rm)
    st = torch.cuda.current_stream().cuda_stream
    plans = [_lib.Plan(), _lib.Plan()]
    for bw in (0, 1):
        _lib.check(lib.fastlstm_plan_device(0, B, H, code, bw, plans[bw]), "plan")
    ifgo0 = torch.empty(T, B, 4 * H, device="cuda", dtype=dt)
    _lib.check(lib.fastlstm_gemm_ifgo(g["x"].data_ptr(), g["Wx"].data_ptr(), g["bx"].data_ptr(), g["bh"].data_ptr(),
                                      ifgo0.data_ptr(), T, B, H, H, code, st), "k1")
    results = {}
    for kind in ("general", "xcd"):
        lib.fastlstm_set_kernel_families(0 if kind == "general" else 7)
        sizes = [lib.fastlstm_recurrent_workspace_bytes(plans[bw], T, H, code, bw) for bw in (0, 1)]
        for bw in (0, 1):
            assert lib.fastlstm_recurrent_kernel_kind(T, B, H, code, bw, sizes[bw]) == (1 if kind == "xcd" else 0)
        ifgo = ifgo0.clone()
        out = torch.empty(T + 1, B, H, device="cuda", dtype=dt)
        cell = torch.empty_like(out)
        out[0], cell[0] = g["h0"], g["c0"]
        ws = torch.zeros(sizes[0], dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_fwd_persistent(ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), g["Wh"].data_ptr(),
                                               ws.data_ptr(), ws.numel(), T, B, H, code, st), "fwd")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK
        for name, got, want in (("out", out, o_out), ("cell", cell, o_cell), ("ifgo", ifgo, o_ifgo)):
            within(got, want, tol, (kind, name))
        d_ifgo = torch.empty_like(ifgo)
        dh, dc = g["dh_n"].clone(), g["dc_n"].clone()
        wsb = torch.zeros(sizes[1], dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_bwd_persistent(g["dout"].data_ptr(), dh.data_ptr(), dc.data_ptr(), ifgo.data_ptr(),
                                               cell.data_ptr(), d_ifgo.data_ptr(), g["Wh"].data_ptr(), wsb.data_ptr(),
                                               wsb.numel(), T, B, H, code, st), "bwd")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(wsb[:64].cpu().numpy().tobytes()) == _lib.OK
        dout, dh_n, dc_n, x, Wx, Wh = to_np(pr, ["dout", "dh_n", "dc_n", "x", "Wx", "Wh"])
        r = oracle.backward(dout, dh_n, dc_n, x, npy(out), npy(cell), npy(ifgo), Wx, Wh, round_mode=rm)
        for name, got, want in (("d_ifgo", d_ifgo, r["d_ifgo"]), ("dh0", dh, r["dh0"]), ("dc0", dc, r["dc0"])):
            within(got, want, tol, (kind, name))
        results[kind] = (out, cell, ifgo, d_ifgo, dh, dc)
    for a, b in zip(results["general"], results["xcd"]):   # two summation orders of the same sums
        within(a, b, tol)


@pytest.mark.parametrize("T,B,I,H,dt", [(96, 64, 1024, 1024, torch.float16),    # helpers compute K1 inside the launch
                                        (40, 32, 512, 1024, torch.bfloat16),   # same, 8 timesteps per row tile
                                        (12, 40, 96, 512, torch.float16),      # 4-wave kernel: two launches
                                        (9, 20, 50, 72, torch.float32),        # general kernels
                                        (40, 48, 64, 64, torch.float16),       # 64 units, one tile: batch tiles of 4 rows
                                        (131, 100, 48, 64, torch.bfloat16),    # ... a ragged batch tile
                                        (1, 16, 8, 64, torch.float16),         # ... one step
                                        (7, 1100, 32, 64, torch.bfloat16),     # ... batch tiles of 8 rows, T % 4 = 3
                                        (6, 2100, 40, 64, torch.float16),      # ... batch tiles of 16 rows, T % 4 = 2
                                        (5, 20, 64, 32, torch.float16)])       # 32 units
def test_fwd_layer_equals_projection_then_recurrence(T, B, I, H, dt):
    """fastlstm_fwd_layer must give bit-identical results to fastlstm_gemm_ifgo followed by
    fastlstm_fwd_persistent, whichever way it schedules the two stages."""
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dt]
    p = make_problem(T, B, I, H, seed=5 + T)
    g = {k: dev(v, dt) for k, v in p.items()}
    st = torch.cuda.current_stream().cuda_stream
    plan = _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 0, plan), "plan")
    nbytes = lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 0)
    res = []
    for fused in (False, True):
        ifgo = torch.empty(T, B, 4 * H, device="cuda", dtype=dt)
        out = torch.empty(T + 1, B, H, device="cuda", dtype=dt)
        cell = torch.empty_like(out)
        out[0], cell[0] = g["h0"], g["c0"]
        ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        if fused:
            _lib.check(lib.fastlstm_fwd_layer(g["x"].data_ptr(), g["Wx"].data_ptr(), g["bx"].data_ptr(),
                                              g["bh"].data_ptr(), g["Wh"].data_ptr(), ifgo.data_ptr(), out.data_ptr(),
                                              cell.data_ptr(), ws.data_ptr(), ws.numel(), T, B, I, H, code, st), "layer")
        else:
            _lib.check(lib.fastlstm_gemm_ifgo(g["x"].data_ptr(), g["Wx"].data_ptr(), g["bx"].data_ptr(),
                                              g["bh"].data_ptr(), ifgo.data_ptr(), T, B, I, H, code, st), "k1")
            _lib.check(lib.fastlstm_fwd_persistent(ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(),
                                                   g["Wh"].data_ptr(), ws.data_ptr(), ws.numel(), T, B, H, code, st), "fwd")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK
        res.append((out, cell, ifgo))
    for a, b in zip(*res):
        assert torch.equal(a, b)


@pytest.mark.parametrize("T,B,I,H,dt,one_launch", [
    (200, 32, 1024, 1024, torch.float16, True),    # config E's layer shape: 4 chunks of 64 timesteps
    (131, 16, 512, 1024, torch.bfloat16, True),    # one group per layer, I != H, ragged last chunk
    (3, 24, 256, 1024, torch.float16, True),       # shorter than a chunk
    (30, 64, 256, 1024, torch.float16, False),     # 2 x 4 groups leave no idle CUs: one layer after the other
    (9, 20, 50, 72, torch.float32, False),         # general kernels
    (70, 64, 128, 832, torch.bfloat16, True),      # 48 idle CUs (6 per XCD)
])
def test_fwd_stack2_equals_two_layer_calls(T, B, I, H, dt, one_launch):
    """fastlstm_fwd_stack2 must give bit-identical results to fastlstm_fwd_layer for the first layer
    followed by fastlstm_fwd_layer for the second on out0[1:], whether it runs the two layers in one
    launch (the second a chunk of timesteps behind the first) or one after the other."""
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dt]
    p0 = make_problem(T, B, I, H, seed=21 + T)
    p1 = make_problem(T, B, H, H, seed=22 + T)
    g0 = {k: dev(v, dt) for k, v in p0.items()}
    g1 = {k: dev(v, dt) for k, v in p1.items()}
    st = torch.cuda.current_stream().cuda_stream
    plan = _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 0, plan), "plan")
    n1 = lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 0)
    n2 = lib.fastlstm_stack2_workspace_bytes(plan, T, H, code)
    assert lib.fastlstm_fwd_stack2_fused(T, B, I, H, code, n2) == (1 if one_launch else 0)

    def buffers(g):
        ifgo = torch.empty(T, B, 4 * H, device="cuda", dtype=dt)
        out = torch.empty(T + 1, B, H, device="cuda", dtype=dt)
        cell = torch.empty_like(out)
        out[0], cell[0] = g["h0"], g["c0"]
        return ifgo, out, cell

    def layer(x, g, bufs, in_size):
        ifgo, out, cell = bufs
        ws = torch.zeros(n1, dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_fwd_layer(x.data_ptr(), g["Wx"].data_ptr(), g["bx"].data_ptr(), g["bh"].data_ptr(),
                                          g["Wh"].data_ptr(), ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(),
                                          ws.data_ptr(), ws.numel(), T, B, in_size, H, code, st), "layer")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK

    ref0, ref1 = buffers(g0), buffers(g1)
    layer(g0["x"], g0, ref0, I)
    layer(ref0[1][1:], g1, ref1, H)
    got0, got1 = buffers(g0), buffers(g1)
    ws = torch.zeros(n2, dtype=torch.uint8, device="cuda")
    _lib.check(lib.fastlstm_fwd_stack2(
        g0["x"].data_ptr(), g0["Wx"].data_ptr(), g0["bx"].data_ptr(), g0["bh"].data_ptr(), g0["Wh"].data_ptr(),
        got0[0].data_ptr(), got0[1].data_ptr(), got0[2].data_ptr(),
        g1["Wx"].data_ptr(), g1["bx"].data_ptr(), g1["bh"].data_ptr(), g1["Wh"].data_ptr(),
        got1[0].data_ptr(), got1[1].data_ptr(), got1[2].data_ptr(), ws.data_ptr(), ws.numel(), T, B, I, H, code, st), "stack2")
    torch.cuda.synchronize()
    assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK
    for a, b in zip(ref0 + ref1, got0 + got1):
        assert torch.equal(a, b)


@pytest.mark.parametrize("T,B,I,H,dt", [(256, 16, 96, 640, torch.float16), (384, 32, 64, 256, torch.float32),
                                        (320, 48, 128, 512, torch.bfloat16),
                                        (389, 32, 64, 256, torch.float32),      # 6 chunks of 64 behind a prefix of 5 timesteps
                                        (263, 16, 96, 640, torch.float16)])     # 4 chunks of 65 behind 3
def test_two_layers_as_a_wavefront_of_chunked_pair_launches(T, B, I, H, dt):
    """Shapes whose two time loops fit the device side by side but which the library's own two-layer launch does
    not take: lstm_persistent_fwd_stack2 / lstm_persistent_bwd_stack2 cut the sequence into chunks and run the
    upper layer's chunk k - 1 beside the lower layer's chunk k.  Against the layer-by-layer ops: the same bits with
    fp32 (the weight gradients: another order of the same sums); with 16-bit elements a chunk starts from the
    stored cell state where the one-launch loop carries it in fp32, hence a tolerance."""
    assert not L.stack2_runs_in_one_launch(T, B, I, H, dt, "cuda")
    assert L.stack2_wavefront_chunks(T, B, H, dt, "cuda") >= 2 and L.stack2_wavefront_chunks(T, B, H, dt, "cuda", backward=True) >= 2
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    g0 = {k: dev(v, dt) for k, v in make_problem(T, B, I, H, seed=41 + T).items()}
    g1 = {k: dev(v, dt) for k, v in make_problem(T, B, H, H, seed=42 + T).items()}
    keys = ("h0", "c0", "Wx", "bx", "Wh", "bh")
    got = L.lstm_persistent_fwd_stack2(g0["x"], *(g0[k] for k in keys), *(g1[k] for k in keys))
    ref0 = L.lstm_persistent_fwd(g0["x"], *(g0[k] for k in keys))
    ref1 = L.lstm_persistent_fwd(ref0[0][1:], *(g1[k] for k in keys))
    for name, a, b in zip(("out0", "cell0", "ifgo0", "out1", "cell1", "ifgo1"), got, ref0 + ref1):
        if dt == torch.float32:
            assert torch.equal(a, b), name
        else:
            within(a, npy(b), tol, name)
    # the reverse pass on the layer-by-layer activations, both ways
    out0, cell0, ifgo0, out1, cell1, ifgo1 = ref0 + ref1
    r0, r1 = L.lstm_persistent_bwd_stack2(g1["dout"], g0["x"], out0, cell0, ifgo0, g0["Wx"], g0["Wh"], out1, cell1, ifgo1,
                                          g1["Wx"], g1["Wh"], d_state0=(g0["dh_n"], g0["dc_n"]), d_state1=(g1["dh_n"], g1["dc_n"]))
    w1 = L.lstm_persistent_bwd(g1["dout"], g1["dc_n"].clone(), g1["dh_n"].clone(), out0[1:], out1, cell1, ifgo1, g1["Wx"], g1["Wh"])
    w0 = L.lstm_persistent_bwd(w1[0], g0["dc_n"].clone(), g0["dh_n"].clone(), g0["x"], out0, cell0, ifgo0, g0["Wx"], g0["Wh"])
    for side, got_, want_ in (("upper", r1, w1), ("lower", r0, w0)):
        for name, a, b in zip(("d_x", "dh_0", "dc_0", "dWx", "dbx", "dWh", "dbh"), got_, want_):
            within(a, npy(b), tol, (side, name))


@pytest.mark.parametrize("L_,T,B,I,H,dt", [(4, 256, 16, 64, 256, torch.float32), (3, 256, 16, 96, 384, torch.float16),
                                           (4, 320, 32, 64, 256, torch.bfloat16),
                                           (3, 197, 16, 64, 256, torch.float32)])   # 3 chunks of 65 behind a prefix of 2
def test_three_and_four_layers_as_a_wavefront(L_, T, B, I, H, dt):
    """lstm_persistent_fwd_stack / lstm_persistent_bwd_stack (launch k runs layer l's chunk k - l for every layer,
    fastlstm_*_persistent_multi) against the layer-by-layer ops: the same bits with fp32 (weight gradients: another
    order of the same sums), a tolerance with 16-bit elements (the cell state is rounded at chunk boundaries)."""
    assert L.stack_wavefront_chunks(L_, T, B, H, dt, "cuda") >= 2 and L.stack_wavefront_chunks(L_, T, B, H, dt, "cuda", backward=True) >= 2
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    gs = [{k: dev(v, dt) for k, v in make_problem(T, B, I if l == 0 else H, H, seed=51 + l + T).items()} for l in range(L_)]
    keys = ("h0", "c0", "Wx", "bx", "Wh", "bh")
    got = L.lstm_persistent_fwd_stack(gs[0]["x"], [tuple(g[k] for k in keys) for g in gs])
    ref, xin = [], gs[0]["x"]
    for g in gs:
        ref.append(L.lstm_persistent_fwd(xin, *(g[k] for k in keys)))
        xin = ref[-1][0][1:]
    for l in range(L_):
        for name, a, b in zip(("out", "cell", "ifgo"), got[l], ref[l]):
            if dt == torch.float32:
                assert torch.equal(a, b), (l, name)
            else:
                within(a, npy(b), tol, (l, name))
    # the reverse pass on the layer-by-layer activations, both ways
    d_states = [(g["dh_n"], g["dc_n"]) for g in gs]
    res = L.lstm_persistent_bwd_stack(gs[-1]["dout"], gs[0]["x"], ref, [(g["Wx"], g["Wh"]) for g in gs], d_states)
    dh = gs[-1]["dout"]
    for l in range(L_ - 1, -1, -1):
        g = gs[l]
        xin = gs[0]["x"] if l == 0 else ref[l - 1][0][1:]
        want = L.lstm_persistent_bwd(dh, g["dc_n"].clone(), g["dh_n"].clone(), xin, *ref[l], g["Wx"], g["Wh"])
        for name, a, b in zip(("d_x", "dh_0", "dc_0", "dWx", "dbx", "dWh", "dbh"), res[l], want):
            within(a, npy(b), tol, (l, name))
        dh = want[0]


@pytest.mark.parametrize("L_,T,B,I,H,dt", [(3, 130, 48, 64, 576, torch.bfloat16),    # a pair and the lowest layer alone
                                           (4, 70, 16, 128, 768, torch.float16)])   # two pairs
def test_deep_stack_reverse_pass_pair_by_pair(L_, T, B, I, H, dt):
    """From a hidden size that depends on the batch, lstm_persistent_bwd_stack runs the library's two-layer reverse
    launches from the top down instead of a wavefront: against the layer-by-layer ops on the same activations."""
    lib = _lib.load()
    code = {torch.float16: 1, torch.bfloat16: 2}[dt]
    plan = _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 1, plan), "plan")
    assert H >= L._pairs_min_hidden(B)
    assert lib.fastlstm_bwd_stack2_fused(T, B, H, H, code, lib.fastlstm_stack2_bwd_workspace_bytes(plan, T, H, code)) == 1
    gs = [{k: dev(v, dt) for k, v in make_problem(T, B, I if l == 0 else H, H, seed=71 + l + T).items()} for l in range(L_)]
    keys = ("h0", "c0", "Wx", "bx", "Wh", "bh")
    acts, xin = [], gs[0]["x"]
    for g in gs:
        acts.append(L.lstm_persistent_fwd(xin, *(g[k] for k in keys)))
        xin = acts[-1][0][1:]
    res = L.lstm_persistent_bwd_stack(gs[-1]["dout"], gs[0]["x"], acts, [(g["Wx"], g["Wh"]) for g in gs],
                                      [(g["dh_n"], g["dc_n"]) for g in gs])
    dh = gs[-1]["dout"]
    for l in range(L_ - 1, -1, -1):
        g = gs[l]
        xin = gs[0]["x"] if l == 0 else acts[l - 1][0][1:]
        want = L.lstm_persistent_bwd(dh, g["dc_n"].clone(), g["dh_n"].clone(), xin, *acts[l], g["Wx"], g["Wh"])
        for name, a, b in zip(("d_x", "dh_0", "dc_0", "dWx", "dbx", "dWh", "dbh"), res[l], want):
            assert rel_err(a, npy(b)) < HALF_TOL, (l, name)
        dh = want[0]


def test_four_layer_module_through_the_wavefront_matches_nn_lstm():
    T, B, I, H, dt = 256, 16, 48, 256, torch.float16
    assert L.stack_wavefront_chunks(4, T, B, H, dt, "cuda") >= 2
    torch.manual_seed(6)
    m = FastLSTM(I, H, num_layers=5).to("cuda", dt)     # four layers as one wavefront, the fifth alone
    ref = torch.nn.LSTM(I, H, num_layers=5).to("cuda", dt)
    ref.load_state_dict(m.state_dict())
    x = (torch.randn(T, B, I, device="cuda") * 0.5).to(dt).requires_grad_(True)
    w = torch.randn(T, B, H, device="cuda").to(dt)
    res = []
    for mod in (m, ref):
        x.grad = None
        out, (h_n, c_n) = mod(x)
        (out * w).sum().backward()
        res.append([out.detach(), h_n.detach(), c_n.detach(), x.grad.clone()] + [q.grad.clone() for q in mod.parameters()])
    for name, a, b in zip(["out", "h_n", "c_n", "dx"] + [n for n, _ in m.named_parameters()], *res):
        assert rel_err(a, npy(b)) < 3 * HALF_TOL, name
    with torch.no_grad():
        out_i, (h_i, c_i) = m(x)
    assert rel_err(out_i, npy(res[0][0])) < HALF_TOL and rel_err(h_i, npy(res[0][1])) < HALF_TOL


@pytest.mark.parametrize("layers,dt", [(2, torch.float16), (3, torch.bfloat16)])
def test_stacked_module_through_the_wavefront_matches_nn_lstm(layers, dt):
    T, B, I, H = 256, 16, 64, 384
    assert L.stack2_wavefront_chunks(T, B, H, dt, "cuda") >= 2
    torch.manual_seed(5)
    m = FastLSTM(I, H, num_layers=layers).to("cuda", dt)
    ref = torch.nn.LSTM(I, H, num_layers=layers).to("cuda", dt)
    ref.load_state_dict(m.state_dict())
    x = (torch.randn(T, B, I, device="cuda") * 0.5).to(dt).requires_grad_(True)
    w = torch.randn(T, B, H, device="cuda").to(dt)
    res = []
    for mod in (m, ref):
        x.grad = None
        out, (h_n, c_n) = mod(x)
        (out * w).sum().backward()
        res.append([out.detach(), h_n.detach(), c_n.detach(), x.grad.clone()] + [q.grad.clone() for q in mod.parameters()])
    for name, a, b in zip(["out", "h_n", "c_n", "dx"] + [n for n, _ in m.named_parameters()], *res):
        assert rel_err(a, npy(b)) < 3 * HALF_TOL, name


def test_two_layer_module_one_launch_matches_layer_by_layer():
    """FastLSTM with two layers of a shape that runs as one launch: outputs, final states and all
    gradients equal those of the layer-by-layer path (two PersistentLSTMfn nodes), bit for bit."""
    T, B, I, H = 130, 32, 1024, 1024
    assert L.stack2_runs_in_one_launch(T, B, I, H, torch.float16, torch.device("cuda", 0))
    torch.manual_seed(3)
    m = L.FastLSTM(I, H, num_layers=2, device="cuda", dtype=torch.float16)
    x = (torch.randn(T, B, I, device="cuda") * 0.5).half().requires_grad_(True)
    w = torch.randn(T, B, H, device="cuda").half()
    out, (h_n, c_n) = m(x)
    (out * w).sum().backward()
    got = [out.detach(), h_n.detach(), c_n.detach(), x.grad.clone()] + [q.grad.clone() for q in m.parameters()]
    x.grad = None
    m.zero_grad(set_to_none=True)
    y = x
    hs, cs = [], []
    for k in range(2):
        y, (h_i, c_i) = L.PersistentLSTMfn.apply(y, None, None, getattr(m, f"weight_ih_l{k}"), getattr(m, f"bias_ih_l{k}"),
                                                 getattr(m, f"weight_hh_l{k}"), getattr(m, f"bias_hh_l{k}"))
        hs.append(h_i)
        cs.append(c_i)
    (y * w).sum().backward()
    want = [y.detach(), torch.stack(hs).detach(), torch.stack(cs).detach(), x.grad.clone()] + [q.grad.clone() for q in m.parameters()]
    names = ["out", "h_n", "c_n", "dx"] + [n for n, _ in m.named_parameters()]
    for name, a, b in zip(names, got, want):
        if name.startswith("weight"):   # weight gradients: sums over T*B in a different order
            assert rel_err(a, b.double().cpu().numpy()) < HALF_TOL, name
        else:
            assert torch.equal(a, b), name


@pytest.mark.parametrize("T,B,I,H,dt,one_launch", [
    (200, 32, 1024, 1024, torch.float16, True),    # config E's layer shape, 4 chunks
    (131, 16, 512, 1024, torch.bfloat16, True),    # I != H, ragged chunk
    (3, 24, 256, 1024, torch.float16, True),       # shorter than a chunk
    (30, 64, 256, 1024, torch.float16, False),     # no idle CUs for two layers: one layer after the other
    (9, 20, 50, 72, torch.float32, False),         # general kernels
    (70, 64, 256, 768, torch.bfloat16, True),      # 64 idle CUs: both dx inside, the weight gradients behind the launch
    (45, 64, 128, 832, torch.float16, True),       # 48 idle CUs
])
def test_bwd_stack2_equals_two_layer_calls(T, B, I, H, dt, one_launch):
    """fastlstm_bwd_stack2 must give the results of fastlstm_bwd_layer for the upper layer followed by
    fastlstm_bwd_layer for the lower layer on the upper layer's dx: bit-identical d_ifgo, dx, dh_0, dc_0
    and db of both layers; dWx and dWh to the rounding of a different summation order."""
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dt]
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    g0 = {k: dev(v, dt) for k, v in make_problem(T, B, I, H, seed=31 + T).items()}
    g1 = {k: dev(v, dt) for k, v in make_problem(T, B, H, H, seed=32 + T).items()}
    out0, cell0, ifgo0 = L.lstm_persistent_fwd(g0["x"], g0["h0"], g0["c0"], g0["Wx"], g0["bx"], g0["Wh"], g0["bh"])
    out1, cell1, ifgo1 = L.lstm_persistent_fwd(out0[1:], g1["h0"], g1["c0"], g1["Wx"], g1["bx"], g1["Wh"], g1["bh"])
    st = torch.cuda.current_stream().cuda_stream
    plan = _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 1, plan), "plan")
    n1 = lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 1)
    n2 = lib.fastlstm_stack2_bwd_workspace_bytes(plan, T, H, code)
    assert lib.fastlstm_bwd_stack2_fused(T, B, I, H, code, n2) == (1 if one_launch else 0)
    wws = torch.empty(max(lib.fastlstm_wgrad_workspace_bytes(T, B, I, H, code),
                          lib.fastlstm_wgrad_workspace_bytes(T, B, H, H, code)), dtype=torch.uint8, device="cuda")
    G = 4 * H
    new = lambda *shape: torch.empty(shape, device="cuda", dtype=dt)

    def outputs():
        return dict(d_ifgo1=new(T, B, G), dx1=new(T, B, H), dh1=g1["dh_n"].clone(), dc1=g1["dc_n"].clone(), db1=new(G),
                    dWx1=new(G, H), dWh1=new(G, H), d_ifgo0=new(T, B, G), dx0=new(T, B, I), dh0=g0["dh_n"].clone(),
                    dc0=g0["dc_n"].clone(), db0=new(G), dWx0=new(G, I), dWh0=new(G, H))

    p = lambda t: t.data_ptr()
    x1 = out0[1:]
    ref = outputs()
    for (dout, o, x, h, Wx, Wh, ifgo, cell, sfx, insz) in (
            (g1["dout"], ref, x1, out1, g1["Wx"], g1["Wh"], ifgo1, cell1, "1", H),
            (ref["dx1"], ref, g0["x"], out0, g0["Wx"], g0["Wh"], ifgo0, cell0, "0", I)):
        ws = torch.zeros(n1, dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_bwd_layer(p(dout), p(o["dh" + sfx]), p(o["dc" + sfx]), p(ifgo), p(cell), p(o["d_ifgo" + sfx]),
                                          p(Wh), p(Wx), p(x), p(h), p(o["dx" + sfx]), p(o["dWx" + sfx]), p(o["dWh" + sfx]),
                                          p(o["db" + sfx]), p(ws), ws.numel(), p(wws), wws.numel(), T, B, insz, H, code, st),
                   "bwd_layer")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK
    got = outputs()
    ws = torch.zeros(n2, dtype=torch.uint8, device="cuda")
    _lib.check(lib.fastlstm_bwd_stack2(
        p(g1["dout"]), p(got["dh1"]), p(got["dc1"]), p(ifgo1), p(cell1), p(got["d_ifgo1"]), p(g1["Wh"]), p(g1["Wx"]), p(out1),
        p(got["dWx1"]), p(got["dWh1"]), p(got["db1"]), p(got["dx1"]), p(got["dh0"]), p(got["dc0"]), p(ifgo0), p(cell0),
        p(got["d_ifgo0"]), p(g0["Wh"]), p(g0["Wx"]), p(g0["x"]), p(out0), p(got["dx0"]), p(got["dWx0"]), p(got["dWh0"]),
        p(got["db0"]), p(ws), ws.numel(), p(wws), wws.numel(), T, B, I, H, code, st), "bwd_stack2")
    torch.cuda.synchronize()
    assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK
    for k in ref:
        if k.startswith("dW") or k.startswith("db"):   # sums over T*B, in an order that depends on the launch form
            within(got[k], ref[k].double().cpu().numpy(), tol, k)
        else:
            assert torch.equal(got[k], ref[k]), k


@pytest.mark.parametrize("T,B,I,H,dt", [(96, 64, 1024, 1024, torch.float16),    # helpers compute dx inside the launch
                                        (40, 32, 512, 1024, torch.bfloat16),
                                        (24, 48, 256, 512, torch.float16),     # 16 units per workgroup
                                        (9, 20, 50, 72, torch.float32),        # general kernels, two launches
                                        (35, 32, 1024, 1024, torch.float16),   # T*B = 1120: no multiple of 64
                                        (67, 20, 256, 512, torch.bfloat16)])
def test_bwd_layer_equals_separate_stages(T, B, I, H, dt):
    """fastlstm_bwd_layer must give the results of fastlstm_bwd_persistent, fastlstm_gemm_dx and
    fastlstm_gemm_wgrad run one after the other, whichever way it schedules the stages: bit-identical
    d_ifgo, dx, dh_0, dc_0, db; dWx and dWh to the rounding of a different summation order."""
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dt]
    tol = FP32_TOL if dt == torch.float32 else HALF_TOL
    p = make_problem(T, B, I, H, seed=11 + T)
    g = {k: dev(v, dt) for k, v in p.items()}
    out, cell, ifgo = L.lstm_persistent_fwd(g["x"], g["h0"], g["c0"], g["Wx"], g["bx"], g["Wh"], g["bh"])
    st = torch.cuda.current_stream().cuda_stream
    plan = _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 1, plan), "plan")
    nbytes = lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 1)
    wbytes = lib.fastlstm_wgrad_workspace_bytes(T, B, I, H, code)
    res = []
    for fused in (False, True):
        d_ifgo = torch.empty_like(ifgo)
        dx = torch.empty(T, B, I, device="cuda", dtype=dt)
        dWx, dWh, db = torch.empty_like(g["Wx"]), torch.empty_like(g["Wh"]), torch.empty_like(g["bx"])
        dh, dc = g["dh_n"].clone(), g["dc_n"].clone()
        ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        wws = torch.empty(wbytes, dtype=torch.uint8, device="cuda")
        if fused:
            _lib.check(lib.fastlstm_bwd_layer(g["dout"].data_ptr(), dh.data_ptr(), dc.data_ptr(), ifgo.data_ptr(),
                                              cell.data_ptr(), d_ifgo.data_ptr(), g["Wh"].data_ptr(), g["Wx"].data_ptr(),
                                              g["x"].data_ptr(), out.data_ptr(), dx.data_ptr(), dWx.data_ptr(),
                                              dWh.data_ptr(), db.data_ptr(), ws.data_ptr(), ws.numel(), wws.data_ptr(),
                                              wws.numel(), T, B, I, H, code, st), "layer")
        else:
            _lib.check(lib.fastlstm_bwd_persistent(g["dout"].data_ptr(), dh.data_ptr(), dc.data_ptr(), ifgo.data_ptr(),
                                                   cell.data_ptr(), d_ifgo.data_ptr(), g["Wh"].data_ptr(), ws.data_ptr(),
                                                   ws.numel(), T, B, H, code, st), "bwd")
            _lib.check(lib.fastlstm_gemm_dx(d_ifgo.data_ptr(), g["Wx"].data_ptr(), dx.data_ptr(), T, B, I, H, code, st), "dx")
            _lib.check(lib.fastlstm_gemm_wgrad(d_ifgo.data_ptr(), g["x"].data_ptr(), out.data_ptr(), dWx.data_ptr(),
                                               dWh.data_ptr(), db.data_ptr(), wws.data_ptr(), wws.numel(), T, B, I, H,
                                               code, st), "wgrad")
        torch.cuda.synchronize()
        assert lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes()) == _lib.OK
        res.append((d_ifgo, dx, dh, dc, db, dWx, dWh))
    for i, (a, b) in enumerate(zip(*res)):
        if i < 4:
            assert torch.equal(a, b), i
        else:   # db, dWx, dWh: the stand-alone stage sums over T*B in another order (split along K)
            within(a, b, tol, i)


def test_xcd_local_barrier_timeout_is_reported_not_hung():
    """The host-forced failure path of the L2 counter barrier: same contract as the flag barrier."""
    lib = _lib.load()
    T, B, H, code = 64, 16, 512, 1
    plan = _lib.Plan()
    _lib.check(lib.fastlstm_plan_device(0, B, H, code, 0, plan), "plan")
    nbytes = lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 0)
    assert lib.fastlstm_recurrent_kernel_kind(T, B, H, code, 0, nbytes) == 1
    ifgo = torch.randn(T, B, 4 * H, device="cuda").half()
    out = torch.zeros(T + 1, B, H, device="cuda").half()
    cell = torch.zeros(T + 1, B, H, device="cuda").half()
    Wh = (torch.randn(4 * H, H, device="cuda") * 0.03).half()
    st = torch.cuda.current_stream().cuda_stream

    def launch():
        ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        _lib.check(lib.fastlstm_fwd_persistent(ifgo.clone().data_ptr(), out.data_ptr(), cell.data_ptr(), Wh.data_ptr(),
                                               ws.data_ptr(), ws.numel(), T, B, H, code, st), "fwd")
        torch.cuda.synchronize()  # returns: the grid drained
        return lib.fastlstm_ws_status(ws[:64].cpu().numpy().tobytes())

    try:
        lib.fastlstm_set_spin_limit(1)
        assert launch() == _lib.ERR_TIMEOUT
    finally:
        lib.fastlstm_set_spin_limit(400000000)
    assert lib.fastlstm_device_status(0, 1) == _lib.ERR_TIMEOUT   # read and cleared
    assert launch() == _lib.OK
    assert lib.fastlstm_device_status(0, 0) == _lib.OK
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("T,B,I,H,dt", [(70, 32, 256, 1024, torch.float16),     # two stacked layers per launch
                                        (6, 128, 128, 2048, torch.bfloat16),    # register-resident H = 2048 kernels
                                        (4, 300, 64, 1024, torch.float16)])     # XCD-local launches over ranges of rows
def test_stacked_and_wide_launches_drain_on_timeout(T, B, I, H, dt):
    """Host-forced failure path for the launches with chunk counters and multi-XCD flag barriers:
    with a spin limit of one poll every wait gives up, the grids drain, the status word reports the
    time-out (the host mirror raises), and the next call is healthy."""
    lib = _lib.load()
    torch.manual_seed(T)
    x = (torch.randn(T, B, I, device="cuda") * 0.5).to(dt)
    mk = lambda *shape: ((torch.rand(*shape, device="cuda") * 2 - 1) / H ** 0.5).to(dt)
    W0, U0, W1, U1, b = mk(4 * H, I), mk(4 * H, H), mk(4 * H, H), mk(4 * H, H), mk(4 * H)
    dh = torch.randn(T, B, H, device="cuda").to(dt)

    def run():
        o = L.lstm_persistent_fwd_stack2(x, None, None, W0, b, U0, b, None, None, W1, b, U1, b)
        torch.cuda.synchronize()
        r = L.lstm_persistent_bwd_stack2(dh, x, o[0], o[1], o[2], W0, U0, o[3], o[4], o[5], W1, U1)
        torch.cuda.synchronize()
        return o, r

    old = L.CHECK_STATUS
    try:
        L.CHECK_STATUS = True
        lib.fastlstm_set_spin_limit(1)
        with pytest.raises(RuntimeError):
            run()
    finally:
        lib.fastlstm_set_spin_limit(400000000)
    assert lib.fastlstm_device_status(0, 0) == _lib.OK   # the host mirror cleared the sticky word when it raised
    try:
        o, r = run()   # healthy again, still with status checks
    finally:
        L.CHECK_STATUS = old
    assert all(torch.isfinite(t.float()).all() for t in o)
    assert torch.isfinite(r[0][0].float()).all() and torch.isfinite(r[1][3].float()).all()


# --------------------------------------------------------------------------------------
# 3b. options beyond the reference's module (its README.md:92-93 lists them as unsupported):
#     nn.LSTM's bias / batch_first / bidirectional and gradients through h_n, c_n
# --------------------------------------------------------------------------------------
def _option_pair(I, H, layers, dt, seed, **kw):
    torch.manual_seed(seed)
    m = FastLSTM(I, H, num_layers=layers, **kw)
    kw.pop("state_grads", None)
    ref = torch.nn.LSTM(I, H, num_layers=layers, **kw)
    with torch.no_grad():
        for n, prm in m.named_parameters():
            prm.copy_(prm.to(dt).float())
            getattr(ref, n).copy_(prm)
    return m.to("cuda", dt), ref


@pytest.mark.parametrize("kw", [dict(bias=False), dict(batch_first=True), dict(bidirectional=True),
                                dict(bias=False, batch_first=True, bidirectional=True)])
def test_option_surface_vs_nn_lstm(kw):
    T, B, I, H, layers = 12, 5, 9, 20, 2
    m, ref = _option_pair(I, H, layers, torch.float32, 31, **kw)
    D = 2 if kw.get("bidirectional") else 1
    g = torch.Generator().manual_seed(2)
    x = torch.randn((B, T, I) if kw.get("batch_first") else (T, B, I), generator=g)
    h0, c0 = torch.randn(layers * D, B, H, generator=g) * 0.3, torch.randn(layers * D, B, H, generator=g) * 0.3
    w = torch.randn(x.shape[0], x.shape[1], D * H, generator=g)
    xg, xr = x.cuda().requires_grad_(True), x.clone().requires_grad_(True)
    y, (hn, cn) = m(xg, (h0.cuda(), c0.cuda()))
    yr, (hr, cr) = ref(xr, (h0, c0))
    assert y.shape == yr.shape and hn.shape == hr.shape
    assert_close32(y, yr); assert_close32(hn, hr); assert_close32(cn, cr)
    (y * w.cuda()).sum().backward(); (yr * w).sum().backward()
    assert_close32(xg.grad, xr.grad)
    assert [n for n, _ in m.named_parameters()] == [n for n, _ in ref.named_parameters()]
    for n, prm in m.named_parameters():
        rg = getattr(ref, n).grad
        assert_close32(prm.grad, rg)


@pytest.mark.parametrize("kw,lengths", [(dict(), [5, 9, 1, 9, 3, 7]),
                                        (dict(bidirectional=True), [4, 4, 12, 1, 7]),
                                        (dict(bidirectional=True, bias=False), [6])])
def test_packed_sequence_vs_nn_lstm(kw, lengths):
    """PackedSequence in, PackedSequence out (unsorted lengths with ties): packed data, the states at each
    row's own last step and every gradient against nn.LSTM; the loss also reads h_n."""
    from torch.nn.utils.rnn import pack_sequence
    I, H, layers = 7, 24, 2
    m, ref = _option_pair(I, H, layers, torch.float32, 41, **kw)
    D = 2 if kw.get("bidirectional") else 1
    g = torch.Generator().manual_seed(9)
    seqs = [torch.randn(n, I, generator=g) for n in lengths]
    B = len(lengths)
    h0, c0 = torch.randn(layers * D, B, H, generator=g) * 0.3, torch.randn(layers * D, B, H, generator=g) * 0.3
    w, wh = torch.randn(sum(lengths), D * H, generator=g), torch.randn(layers * D, B, H, generator=g)
    xr = pack_sequence(seqs, enforce_sorted=False)
    xg = pack_sequence([t.cuda() for t in seqs], enforce_sorted=False)
    y, (hn, cn) = m(xg, (h0.cuda(), c0.cuda()))
    yr, (hr, cr) = ref(xr, (h0, c0))
    assert torch.equal(y.batch_sizes, yr.batch_sizes) and torch.equal(y.sorted_indices.cpu(), yr.sorted_indices)
    assert torch.equal(y.unsorted_indices.cpu(), yr.unsorted_indices)
    assert_close32(y.data, yr.data); assert_close32(hn, hr); assert_close32(cn, cr)
    ((y.data * w.cuda()).sum() + (hn * wh.cuda()).sum()).backward()
    ((yr.data * w).sum() + (hr * wh).sum()).backward()
    for n, prm in m.named_parameters():
        rg = getattr(ref, n).grad
        assert_close32(prm.grad, rg)


@pytest.mark.parametrize("kw,T,B,I,H,Hp,Ip,dt", [(dict(bidirectional=True), 32, 24, 50, 100, 112, 50, torch.float32),
                                                 (dict(), 64, 16, 70, 650, 704, 128, torch.float16),   # (stacked layers: a multiple of 64)
                                                 (dict(bidirectional=True), 64, 16, 300, 256, 256, 320, torch.float16),
                                                 (dict(bias=False, batch_first=True), 32, 8, 33, 1150, 1280, 33, torch.bfloat16),
                                                 (dict(), 16, 128, 64, 1150, 1280, 64, torch.bfloat16),   # few steps, many rows
                                                 (dict(), 64, 16, 70, 576, 640, 70, torch.float32),    # for the reverse pass's sake
                                                 (dict(), 64, 40, 20, 32, 64, 64, torch.float16),      # narrow layers: as 64 units
                                                 (dict(bidirectional=True), 40, 30, 16, 16, 64, 16, torch.bfloat16)])   # (an input size the streaming products take)
def test_hidden_and_input_sizes_off_the_fast_kernels_run_zero_padded(kw, T, B, I, H, Hp, Ip, dt):
    """The module pads a hidden size that only the general kernels take to the next one the XCD-local /
    register-resident kernels take (zero weights, biases and initial states for the added units), and a 16-bit
    input size to a multiple of 64 (zero columns of x and W_x): outputs, final states and every gradient against
    nn.LSTM in fp32 on the CPU, two layers, initial states given, a loss on out, h_n and c_n."""
    layers = 2
    D = 2 if kw.get("bidirectional") else 1
    m, ref = _option_pair(I, H, layers, dt, 47, state_grads=True, **kw)
    g = torch.Generator().manual_seed(12)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(dt).float()
    x = rnd(B, T, I) if kw.get("batch_first") else rnd(T, B, I)
    h0, c0 = rnd(layers * D, B, H) * 0.3, rnd(layers * D, B, H) * 0.3
    wy, wh, wc = rnd(*x.shape[:2], D * H), rnd(layers * D, B, H), rnd(layers * D, B, H)
    leaves = [t.cuda().to(dt).requires_grad_(True) for t in (x, h0, c0)]
    leaves_r = [t.clone().requires_grad_(True) for t in (x, h0, c0)]
    assert m._operand_padding(leaves[0]) == (Hp, Ip)
    # sizes the fast kernels take run as they are, H = 64 (the one-tile form of the general kernels) among them;
    # narrower 16-bit layers run as 64 units
    for i_, h_ in ((64, 64), (256, 512), (1024, 2048)):
        assert FastLSTM(i_, h_).to("cuda", torch.float16)._operand_padding(torch.empty(32, 256, i_, device="cuda", dtype=torch.float16)) is None
    assert FastLSTM(128, 32).to("cuda", torch.float16)._operand_padding(torch.empty(32, 256, 128, device="cuda", dtype=torch.float16)) == (64, 128)
    # ... and a few timesteps do not repay the padding (unless rows x units are many: the last case)
    assert m._operand_padding(leaves[0][:, :4] if kw.get("batch_first") else leaves[0][:4]) is None
    y, (hn, cn) = m(leaves[0], (leaves[1], leaves[2]))
    yr, (hr, cr) = ref(leaves_r[0], (leaves_r[1], leaves_r[2]))
    assert y.shape == yr.shape and hn.shape == hr.shape and y.is_contiguous() and hn.is_contiguous()
    ((y.float() * wy.cuda()).sum() + (hn.float() * wh.cuda()).sum() + (cn.float() * wc.cuda()).sum()).backward()
    ((yr * wy).sum() + (hr * wh).sum() + (cr * wc).sum()).backward()
    pairs = [(a.grad, b.grad, n) for a, b, n in zip(leaves, leaves_r, ("x", "h0", "c0"))]
    pairs += [(prm.grad, getattr(ref, n).grad, n) for n, prm in m.named_parameters()]
    for got, want, name in [(y, yr, "y"), (hn, hr, "hn"), (cn, cr, "cn")] + pairs:
        assert got.shape == want.shape, name
        if dt == torch.float32:
            assert_close32(got, want)
        else:
            assert rel_err(got, want) < HALF_TOL, name


@pytest.mark.parametrize("kw,B,H,dt", [(dict(), 400, 1024, torch.float16), (dict(bidirectional=True), 200, 1536, torch.bfloat16)])
def test_packed_batch_larger_than_one_launch_is_cut_at_its_row_ranges(kw, B, H, dt, monkeypatch):
    """A packed batch that the library runs as several launches over ranges of rows is cut at those ranges in
    the packed order, and every range stops at its own longest sequence: same contract, against nn.LSTM in
    fp32 on the CPU (packed data, final states, every gradient; unsorted lengths, initial states given)."""
    from torch.nn.utils.rnn import pack_sequence
    import fastlstm_amd.lstm as L
    I, layers, Tmax = 24, 2, 22
    D = 2 if kw.get("bidirectional") else 1
    m, ref = _option_pair(I, H, layers, dt, 43, **kw)
    g = torch.Generator().manual_seed(10)
    lengths = [int(v) for v in torch.randint(3, Tmax + 1, (B,), generator=g)]
    lengths[5] = Tmax
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(dt).float()
    seqs = [rnd(n, I) for n in lengths]
    h0, c0 = rnd(layers * D, B, H) * 0.3, rnd(layers * D, B, H) * 0.3
    w, wh = rnd(sum(lengths), D * H), rnd(layers * D, B, H)
    xr = pack_sequence(seqs, enforce_sorted=False)
    xg = pack_sequence([t.cuda().to(dt) for t in seqs], enforce_sorted=False)
    cuts = []
    run_padded = L.FastLSTM._run_padded
    for cls in (L.FastLSTM, L._OperandsPadded):   # (the module itself, and its view with zero-padded sizes)
        monkeypatch.setattr(cls, "_run_padded", lambda self, x, *a: (cuts.append(tuple(x.shape[:2])), run_padded(self, x, *a))[1])
    y, (hn, cn) = m(xg, (h0.cuda().to(dt), c0.cuda().to(dt)))
    # several ranges, the later ones shorter than the first
    assert len(cuts) > 1 and sum(b for _, b in cuts) == B and cuts[0][0] == Tmax and cuts[-1][0] < Tmax, cuts
    yr, (hr, cr) = ref(xr, (h0, c0))
    assert torch.equal(y.batch_sizes, yr.batch_sizes) and torch.equal(y.unsorted_indices.cpu(), yr.unsorted_indices)
    for got, want, name in ((y.data, yr.data, "y"), (hn, hr, "hn"), (cn, cr, "cn")):
        assert rel_err(got, want) < HALF_TOL, name
    ((y.data.float() * w.cuda()).sum() + (hn.float() * wh.cuda()).sum()).backward()
    ((yr.data * w).sum() + (hr * wh).sum()).backward()
    for n, prm in m.named_parameters():
        assert rel_err(prm.grad, getattr(ref, n).grad) < HALF_TOL, n


@pytest.mark.parametrize("T,B,I,H,layers,dt", [(9, 7, 11, 33, 1, torch.float32), (14, 5, 6, 65, 3, torch.float32),
                                               (70, 32, 256, 1024, 2, torch.float16)])   # one launch per pair
def test_state_gradients_vs_nn_lstm(T, B, I, H, layers, dt):
    """state_grads=True: a loss on out, h_n and c_n together, with h_0 and c_0 as leaves; every
    gradient against nn.LSTM in fp32 on the CPU.  (The reference's nested tuple carries no gradient to
    h_n / c_n and its backward raises for one, fastlstm/lstm.py:522-531.)"""
    m, ref = _option_pair(I, H, layers, dt, 77, state_grads=True)
    g = torch.Generator().manual_seed(3)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(dt).float()
    x, h0, c0 = rnd(T, B, I), rnd(layers, B, H) * 0.3, rnd(layers, B, H) * 0.3
    wy, wh, wc = rnd(T, B, H), rnd(layers, B, H), rnd(layers, B, H)
    leaves = [t.cuda().to(dt).requires_grad_(True) for t in (x, h0, c0)]
    leaves_r = [t.clone().requires_grad_(True) for t in (x, h0, c0)]
    y, (hn, cn) = m(leaves[0], (leaves[1], leaves[2]))
    yr, (hr, cr) = ref(leaves_r[0], (leaves_r[1], leaves_r[2]))
    assert hn.requires_grad and cn.requires_grad
    ((y.float() * wy.cuda()).sum() + (hn.float() * wh.cuda()).sum() + (cn.float() * wc.cuda()).sum()).backward()
    ((yr * wy).sum() + (hr * wh).sum() + (cr * wc).sum()).backward()
    pairs = [(a.grad, b.grad, n) for a, b, n in zip(leaves, leaves_r, ("x", "h0", "c0"))]
    pairs += [(prm.grad, getattr(ref, n).grad, n) for n, prm in m.named_parameters()]
    for got, want, name in [(y, yr, "y"), (hn, hr, "hn"), (cn, cr, "cn")] + pairs:
        if dt == torch.float32:
            assert_close32(got, want)
        else:
            assert rel_err(got, want) < HALF_TOL, name


def test_state_carried_across_segments_trains_like_the_whole_sequence():
    """Two segments with the state handed over (not detached) give the gradients of the whole sequence:
    the reverse kernel's dh_n / dc_n operands carry the second segment's gradient into the first."""
    T, B, I, H = 24, 6, 10, 48
    torch.manual_seed(5)
    m = FastLSTM(I, H, num_layers=2, state_grads=True).cuda()
    x = torch.randn(T, B, I, device="cuda")
    w = torch.randn(T, B, H, device="cuda")
    y, _ = m(x)
    (y * w).sum().backward()
    whole = {n: p.grad.clone() for n, p in m.named_parameters()}
    m.zero_grad()
    y1, state = m(x[:10])
    y2, _ = m(x[10:], state)
    assert torch.equal(torch.cat((y1, y2)), y)
    (torch.cat((y1, y2)) * w).sum().backward()
    for n, p in m.named_parameters():
        assert_close32(p.grad, whole[n].cpu())


def _mixed_shape(rng):
    if rng.random() < 0.5:
        return rng.randint(20, 90), rng.choice([16, 32, 48, 64]), rng.choice([64, 256, 100]), rng.choice([256, 512, 1024])
    return rng.randint(1, 30), rng.randint(1, 70), rng.randint(1, 100), rng.randint(1, 300)


def _narrow_shape(rng):
    """H <= 64: one hidden tile per workgroup; with 16-bit elements and T*B >= 256 also the one-pass reverse
    products and, for I no multiple of 64, the streaming input projection."""
    return (rng.choice([1, 2, 3, 5, 8, 17, 33, 64, 100, 129, 200]),
            rng.choice([1, 3, 15, 16, 17, 31, 32, 48, 64, 65, 100, 128, 200, 256, 300]),
            rng.choice([16, 32, 48, 64, 64, 20, 80, 128]), rng.choice([16, 32, 48, 64, 64, 64, 24]))


@pytest.mark.parametrize("seed,shape,max_layers,ref64", [(21, _mixed_shape, 4, False), (22, _mixed_shape, 4, False),
                                                         (31, _narrow_shape, 3, True)])
def test_random_modules_vs_nn_lstm(seed, shape, max_layers, ref64):
    """30 seeded random modules per seed (1-4 layers, every option, with and without an initial state,
    ragged shapes and shapes whose layer pairs run as one launch; one seed of narrow layers): outputs, states and
    every gradient against nn.LSTM on the CPU, in fp32.  The narrow shapes have up to 60000 rows, where nn.LSTM's
    own fp32 bias sums are off by more than the element-wise fp32 bar (measured against fp64: 1.4 x the bar, this
    library 0.06 x), so that seed's reference computes in fp64."""
    import random
    rng = random.Random(seed)
    old, L.CHECK_STATUS = L.CHECK_STATUS, True
    try:
        for case in range(30):
            dt = rng.choice([torch.float32, torch.float16, torch.bfloat16])
            layers = rng.randint(1, max_layers)
            kw = dict(bias=rng.random() < 0.8, batch_first=rng.random() < 0.3, bidirectional=rng.random() < 0.3,
                      state_grads=rng.random() < 0.5)
            T, B, I, H = shape(rng)
            with_state = rng.random() < 0.5
            tag = f"seed {seed} case {case}: T={T} B={B} I={I} H={H} L={layers} {dt} {kw} state={with_state}"
            print(tag, flush=True)
            m, ref = _option_pair(I, H, layers, dt, seed * 1000 + case, **dict(kw))
            rdt = torch.float64 if ref64 else torch.float32
            ref = ref.to(rdt)
            D = 2 if kw["bidirectional"] else 1
            g = torch.Generator().manual_seed(case)
            rnd = lambda *shape: torch.randn(*shape, generator=g).to(dt).to(rdt)
            x = rnd(B, T, I) if kw["batch_first"] else rnd(T, B, I)
            h0, c0 = rnd(layers * D, B, H) * 0.3, rnd(layers * D, B, H) * 0.3
            wy, wh, wc = rnd(*x.shape[:2], D * H), rnd(layers * D, B, H), rnd(layers * D, B, H)
            leaves = [t.cuda().to(dt).requires_grad_(True) for t in (x, h0, c0)]
            leaves_r = [t.clone().requires_grad_(True) for t in (x, h0, c0)]
            if with_state:
                y, (hn, cn) = m(leaves[0], (leaves[1], leaves[2]))
                yr, (hr, cr) = ref(leaves_r[0], (leaves_r[1], leaves_r[2]))
            else:
                y, (hn, cn) = m(leaves[0])
                yr, (hr, cr) = ref(leaves_r[0])
            loss, loss_r = (y.float() * wy.cuda().float()).sum(), (yr * wy).sum()
            if kw["state_grads"]:
                loss = loss + (hn.float() * wh.cuda().float()).sum() + (cn.float() * wc.cuda().float()).sum()
                loss_r = loss_r + (hr * wh).sum() + (cr * wc).sum()
            loss.backward(); loss_r.backward()
            pairs = [("y", y, yr), ("hn", hn, hr), ("cn", cn, cr)]
            pairs += [(n, a.grad, b.grad) for n, a, b in zip(("dx", "dh0", "dc0"), leaves, leaves_r)][:3 if with_state else 1]
            pairs += [(n, prm.grad, getattr(ref, n).grad) for n, prm in m.named_parameters()]
            tol = FP32_TOL if dt == torch.float32 else HALF_TOL   # max-norm relative error
            for name, got, want in pairs:
                within(got, want, tol, (tag, name))
    finally:
        L.CHECK_STATUS = old


@pytest.mark.parametrize("T,B,I,H,dt", [(6, 20, 64, 64, torch.float16),       # single-tile kernel
                                        (5, 33, 70, 300, torch.float32),      # general kernel, element-wise stores
                                        (7, 40, 64, 512, torch.float32),      # general kernel, tile stores
                                        (40, 64, 256, 1024, torch.float16),   # XCD-local, projection inside the launch
                                        (3, 128, 128, 2048, torch.bfloat16),  # register-resident H = 2048
                                        (3, 300, 64, 1024, torch.float16)])   # several launches over the batch
def test_inference_forward_is_the_training_forward_without_the_stores(T, B, I, H, dt):
    """keep_activations=False (fastlstm_fwd_layer_infer): out and the final cell state bit for bit, the
    gate buffer left as the input projection, cell[1:-1] untouched."""
    p = make_problem(T, B, I, H, seed=T + H)
    g = {k: dev(v, dt) for k, v in p.items()}
    args = (g["x"], g["h0"], g["c0"], g["Wx"], g["bx"], g["Wh"], g["bh"])
    out, cell, ifgo = L.lstm_persistent_fwd(*args)
    out_i, cell_i, ifgo_i = L.lstm_persistent_fwd(*args, keep_activations=False)
    assert torch.equal(out_i, out)
    assert torch.equal(cell_i[-1], cell[-1]) and torch.equal(cell_i[0], cell[0])
    proj = torch.empty_like(ifgo)
    lib = _lib.load()
    _lib.check(lib.fastlstm_gemm_ifgo(g["x"].data_ptr(), g["Wx"].data_ptr(), g["bx"].data_ptr(), g["bh"].data_ptr(),
                                      proj.data_ptr(), T, B, I, H, L._code(g["x"]), L._stream()), "gemm_ifgo")
    assert torch.equal(ifgo_i, proj) and not torch.equal(ifgo_i, ifgo)


@pytest.mark.parametrize("kw,T,B,I,H", [(dict(num_layers=2), 70, 32, 256, 1024),          # layer pair in one launch
                                        (dict(num_layers=3, bidirectional=True), 9, 5, 12, 40)])
def test_module_without_grad_takes_the_inference_path_same_bits(kw, T, B, I, H, monkeypatch):
    torch.manual_seed(3)
    m = FastLSTM(I, H, **kw).to("cuda", torch.float16)
    x = torch.randn(T, B, I, device="cuda").half()
    calls = []
    for name in ("lstm_persistent_fwd", "lstm_persistent_fwd_stack2", "lstm_persistent_fwd_pair"):
        orig = getattr(L, name)
        monkeypatch.setattr(L, name, lambda *a, _o=orig, **k: (calls.append(k.get("keep_activations", True)), _o(*a, **k))[1])
    y, (hn, cn) = m(x)
    assert calls and all(calls)
    calls.clear()
    with torch.no_grad():
        y2, (hn2, cn2) = m(x)
    assert calls and not any(calls)
    assert torch.equal(y2, y) and torch.equal(hn2, hn) and torch.equal(cn2, cn)
    calls.clear()
    m.requires_grad_(False)
    y3, _ = m(x)                                   # nothing that enters requires a gradient
    assert calls and not any(calls) and torch.equal(y3, y)
    calls.clear()
    y4, _ = m(x.clone().requires_grad_(True))      # ... unless the input does
    assert calls and all(calls) and y4.requires_grad


@pytest.mark.parametrize("T,B,I,H,layers,dt", [(32, 64, 256, 1024, 1, torch.float16),   # XCD-local, projection in the launch
                                               (40, 32, 128, 1024, 2, torch.float16),   # two layers in one launch
                                               (16, 20, 24, 64, 1, torch.float16),      # one hidden tile per workgroup
                                               (8, 16, 32, 256, 1, torch.float32)])
def test_forward_replays_from_a_captured_graph(T, B, I, H, layers, dt):
    """The module's forward captured into a HIP graph (the reference builds its version="graph" on
    torch.cuda.graph too, fastlstm/lstm.py:149-233, one kernel node per timestep): every replay, with new input contents and other work on the device in
    between, gives the eager result bit for bit.  The launches clear their workspaces with fill
    kernels, never with memset nodes."""
    torch.manual_seed(0)
    m = FastLSTM(I, H, num_layers=layers).to("cuda", dt)
    xs = [torch.randn(T, B, I, device="cuda").to(dt) for _ in range(3)]
    static_x = xs[0].clone()
    with torch.no_grad():
        eager = [m(x)[0].clone() for x in xs]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                m(static_x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y, _ = m(static_x)
        for rep in range(2):
            for i, x in enumerate(xs):
                static_x.copy_(x)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(y, eager[i]), (rep, i)
                (torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")).sum().item()


@pytest.mark.parametrize("T,B,I,H,layers,dt", [(16, 20, 24, 64, 1, torch.float16),      # one hidden tile per workgroup
                                               (32, 64, 256, 1024, 1, torch.float16),   # XCD-local, GEMMs inside both launches
                                               (40, 32, 128, 1024, 2, torch.float16)])  # two layers per launch, both directions
def test_training_step_replays_from_a_captured_graph(T, B, I, H, layers, dt):
    """Forward AND backward of the module captured into one HIP graph, the whole-network recipe of
    PyTorch's CUDA-graph notes: warm-up on a side stream, gradients set to None, and no tensor of an earlier
    autograd graph alive when the capture starts (an AccumulateGrad node kept alive from a step on another
    stream makes the autograd engine add cross-stream event waits to the capture, which ends it with a
    host crash inside hipStreamEndCapture -- a property of the capture, not of these kernels).  Every replay,
    with new input contents, gives the eager step's output and parameter gradients bit for bit."""
    import gc
    torch.manual_seed(0)
    m = FastLSTM(I, H, num_layers=layers).to("cuda", dt)
    xs = [torch.randn(T, B, I, device="cuda").to(dt) for _ in range(3)]
    ws = [torch.randn(T, B, H, device="cuda").to(dt) for _ in range(3)]
    sx, sw = xs[0].clone(), ws[0].clone()

    def step():
        y, _ = m(sx)
        (y * sw).sum().backward()
        return y.detach()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            m.zero_grad(set_to_none=True)
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    m.zero_grad(set_to_none=True)
    gc.collect()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sy = step()
    replayed = []
    for rep in range(2):
        for i in range(3):
            sx.copy_(xs[i]); sw.copy_(ws[i])
            graph.replay()
            torch.cuda.synchronize()
            replayed.append((sy.clone(), [prm.grad.clone() for prm in m.parameters()]))
            (torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")).sum().item()
    for rep in range(2):
        for i in range(3):
            sx.copy_(xs[i]); sw.copy_(ws[i])
            m.zero_grad(set_to_none=True)
            y = step()
            torch.cuda.synchronize()
            gy, gp = replayed[rep * 3 + i]
            assert torch.equal(gy, y), (rep, i)
            for prm, gr in zip(m.parameters(), gp):
                assert torch.equal(prm.grad, gr), (rep, i)


# --------------------------------------------------------------------------------------
# 4. BASELINE.json configurations at their real shapes
# --------------------------------------------------------------------------------------
def _module_pair(I, H, layers, dt, seed):
    torch.manual_seed(seed)
    m = FastLSTM(I, H, num_layers=layers)
    ref = torch.nn.LSTM(I, H, num_layers=layers)
    with torch.no_grad():
        for n, prm in m.named_parameters():
            prm.copy_(prm.to(dt).float())        # weights representable in dt
            getattr(ref, n).copy_(prm)
    return m.to("cuda", dt), ref


def test_config_A_fp32_fwd_bwd_full_size():
    T, B, I, H = 128, 16, 256, 256
    m, ref = _module_pair(I, H, 1, torch.float32, 1234)
    x = torch.randn(T, B, I, generator=torch.Generator().manual_seed(1))
    xg = x.cuda().requires_grad_(True)
    xr = x.clone().requires_grad_(True)
    y, (hn, cn) = m(xg)
    yr, (hr, cr) = ref(xr)
    assert_close32(y, yr); assert_close32(hn, hr); assert_close32(cn, cr)
    y.sum().backward(); yr.sum().backward()
    rows = [("out", y, yr), ("h_n", hn, hr), ("c_n", cn, cr), ("dx", xg.grad, xr.grad)]
    rows += [(n + ".grad", prm.grad, getattr(ref, n).grad) for n, prm in m.named_parameters()]
    assert_elementwise32(rows, "config A")


def test_config_B_fp16_forward_full_size():
    T, B, I, H = 512, 64, 1024, 1024
    m, ref = _module_pair(I, H, 1, torch.float16, 1235)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, B, I, generator=g).half().float()
    h0 = (torch.randn(1, B, H, generator=g) * 0.1).half().float()
    c0 = (torch.randn(1, B, H, generator=g) * 0.1).half().float()
    with torch.no_grad():
        y, (hn, cn) = m(x.cuda().half(), (h0.cuda().half(), c0.cuda().half()))
        yr, (hr, cr) = ref(x, (h0, c0))
    assert rel_err(y, yr) < HALF_TOL
    assert rel_err(hn, hr) < HALF_TOL
    assert rel_err(cn, cr) < HALF_TOL


def test_config_C_bf16_tiles_fwd_bwd():
    """Config C's tiling (B=128, I=H=2048, bf16) with T cut to 24 so the CPU reference
    finishes in seconds; the per-step work and every kernel shape are the real ones."""
    T, B, I, H = 24, 128, 2048, 2048
    m, ref = _module_pair(I, H, 1, torch.bfloat16, 1236)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, B, I, generator=g).bfloat16().float()
    dout = torch.randn(T, B, H, generator=g).bfloat16().float()
    h0 = torch.zeros(1, B, H); c0 = torch.zeros(1, B, H)
    xg = x.cuda().bfloat16().requires_grad_(True)
    h0g, c0g = h0.cuda().bfloat16().requires_grad_(True), c0.cuda().bfloat16().requires_grad_(True)
    y, _ = m(xg, (h0g, c0g))
    (y.float() * dout.cuda()).sum().backward()
    xr = x.clone().requires_grad_(True)
    h0r, c0r = h0.clone().requires_grad_(True), c0.clone().requires_grad_(True)
    yr, _ = ref(xr, (h0r, c0r))
    (yr * dout).sum().backward()
    assert rel_err(y, yr) < HALF_TOL
    assert rel_err(xg.grad, xr.grad) < HALF_TOL
    assert rel_err(h0g.grad, h0r.grad) < HALF_TOL
    assert rel_err(c0g.grad, c0r.grad) < HALF_TOL
    for n, prm in m.named_parameters():
        assert rel_err(prm.grad, getattr(ref, n).grad) < HALF_TOL, n
    assert torch.equal(m.bias_ih_l0.grad, m.bias_hh_l0.grad)


def test_config_D_small_hidden_fp16_full_size():
    """loss = mean(out^2) over 16.7 M elements: the upstream gradient 2*out/N is ~1e-7 and
    underflows fp16 (any fp16 backward would lose it), so the loss is scaled by 2^20 the
    way AMP loss scaling does and the fp32 reference's gradients are scaled alike."""
    T, B, I, H = 1024, 256, 64, 64
    scale = 2.0 ** 20
    m, ref = _module_pair(I, H, 1, torch.float16, 1237)
    x = (torch.rand(T, B, I, generator=torch.Generator().manual_seed(4)) * 2 - 1).half().float()
    y, _ = m(x.cuda().half())
    ((y.float() ** 2).mean() * scale).backward()
    yr, _ = ref(x)
    ((yr ** 2).mean() * scale).backward()
    assert rel_err(y, yr) < HALF_TOL
    for n, prm in m.named_parameters():
        assert rel_err(prm.grad, getattr(ref, n).grad) < HALF_TOL, n


def test_config_E_two_layers_fp16():
    """Config E (2 stacked layers, B=32, I=H=1024) with T = 256 of its 2048 steps for the
    CPU reference's sake; 16-bit error growth over the full length is covered by config D."""
    T, B, I, H = 256, 32, 1024, 1024
    m, ref = _module_pair(I, H, 2, torch.float16, 1238)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, B, I, generator=g).half().float()
    dout = torch.randn(T, B, H, generator=g).half().float()
    y, (hn, cn) = m(x.cuda().half())
    (y.float() * dout.cuda()).sum().backward()
    yr, (hr, cr) = ref(x)
    (yr * dout).sum().backward()
    assert hn.shape == (2, B, H)
    assert rel_err(y, yr) < HALF_TOL
    assert rel_err(cn, cr) < HALF_TOL
    for n, prm in m.named_parameters():
        assert rel_err(prm.grad, getattr(ref, n).grad) < HALF_TOL, n

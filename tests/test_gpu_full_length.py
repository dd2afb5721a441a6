"""BASELINE.json's long configurations at their FULL sequence length against the fp32 CPU oracle
(run with -m gpu on an MI355X).

Config B (fp16, B=64, T=512, I=H=1024: forward and backward) is the headline configuration.  Config C
(bf16, B=128, T=256, I=H=2048) and config E (fp16, two stacked layers, B=32, T=2048,
I=H=1024) are the two configurations whose time-dependent host code (exchange ring sizes, chunk
hand-over between the stacked layers, which kernel a workspace size selects) only shows at the real
T.  The 16-bit GPU results are compared with the oracle evaluated in fp32 WITHOUT any 16-bit
rounding on the same (16-bit representable) inputs and weights: the tolerance therefore bounds the
error growth of the 16-bit path over all T steps, 2e-2 of the reference's largest magnitude for
every output and gradient (north star: <= 2e-2 relative in fp16/bf16 with fp32 accumulation).
The oracle needs about half a minute per configuration on the box's 16 host cores.
"""
import numpy as np
import pytest
import torch

import fastlstm_amd.lstm as L
from fastlstm_amd import FastLSTM, _lib
from helpers import rel_err

pytestmark = pytest.mark.gpu
HALF_TOL = 2e-2


@pytest.fixture(scope="module", autouse=True)
def _gpu_setup():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    old = L.CHECK_STATUS
    L.CHECK_STATUS = True
    yield
    L.CHECK_STATUS = old


def _kind(T, B, H, dt, backward):
    """fastlstm_recurrent_kernel_kind for the workspace lstm.py allocates for this shape."""
    lib = _lib.load()
    code = L._DTYPE_CODE[dt]
    plan = L._plan(torch.device("cuda:0"), B, H, code, backward)
    ws = L._workspace(plan, T, H, code, backward, torch.device("cuda:0"))
    return lib.fastlstm_recurrent_kernel_kind(T, B, H, code, int(backward), ws.numel())


def _weights(I, H, layers, dt, seed):
    """FastLSTM on the GPU in dt and its weights (dt-representable) as fp32 numpy arrays."""
    torch.manual_seed(seed)
    m = FastLSTM(I, H, num_layers=layers)
    with torch.no_grad():
        for prm in m.parameters():
            prm.copy_(prm.to(dt).float())
    w = {n: prm.detach().numpy().copy() for n, prm in m.named_parameters()}
    return m.to("cuda", dt), w


def _report(rows):
    for name, e in rows:
        print("    %-12s max|err|/max|ref| = %.3e" % (name, e))
    worst = max(rows, key=lambda r: r[1])
    assert worst[1] < HALF_TOL, worst


def test_config_C_bf16_full_length_vs_fp32_oracle(oracle):
    T, B, I, H = 256, 128, 2048, 2048
    dt = torch.bfloat16
    assert _kind(T, B, H, dt, False) == 2 and _kind(T, B, H, dt, True) == 2   # register-resident kernels, no fall-back
    m, w = _weights(I, H, 1, dt, 1236)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, B, I, generator=g).to(dt).float()
    dout = torch.randn(T, B, H, generator=g).to(dt).float()
    xg = x.cuda().to(dt).requires_grad_(True)
    h0g = torch.zeros(1, B, H, device="cuda", dtype=dt, requires_grad=True)
    c0g = torch.zeros(1, B, H, device="cuda", dtype=dt, requires_grad=True)
    y, (hn, cn) = m(xg, (h0g, c0g))
    (y.float() * dout.cuda()).sum().backward()
    torch.cuda.synchronize()
    z = np.zeros((B, H), np.float32)
    o_out, o_cell, o_ifgo = oracle.forward(x.numpy(), z, z, w["weight_ih_l0"], w["bias_ih_l0"], w["weight_hh_l0"],
                                           w["bias_hh_l0"], dtype=np.float32)
    r = oracle.backward(dout.numpy(), None, None, x.numpy(), o_out, o_cell, o_ifgo, w["weight_ih_l0"],
                        w["weight_hh_l0"], dtype=np.float32)
    _report([("out", rel_err(y, o_out[1:])), ("h_n", rel_err(hn[0], o_out[-1])), ("c_n", rel_err(cn[0], o_cell[-1])),
             ("dx", rel_err(xg.grad, r["dx"])), ("dh0", rel_err(h0g.grad[0], r["dh0"])),
             ("dc0", rel_err(c0g.grad[0], r["dc0"])), ("dW_x", rel_err(m.weight_ih_l0.grad, r["dWx"])),
             ("dW_h", rel_err(m.weight_hh_l0.grad, r["dWh"])), ("db_x", rel_err(m.bias_ih_l0.grad, r["db"])),
             ("db_h", rel_err(m.bias_hh_l0.grad, r["db"]))])


def test_config_B_fp16_fwd_bwd_full_size_vs_fp32_oracle(oracle):
    """The headline configuration, forward AND backward at full size (the GEMMs run inside both recurrent
    launches), with a non-zero initial state and a random upstream gradient."""
    T, B, I, H = 512, 64, 1024, 1024
    dt = torch.float16
    assert _kind(T, B, H, dt, False) == 1 and _kind(T, B, H, dt, True) == 1   # XCD-local kernels
    m, w = _weights(I, H, 1, dt, 1235)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, B, I, generator=g).to(dt).float()
    dout = torch.randn(T, B, H, generator=g).to(dt).float()
    h0 = (torch.randn(1, B, H, generator=g) * 0.1).to(dt).float()
    c0 = (torch.randn(1, B, H, generator=g) * 0.1).to(dt).float()
    xg = x.cuda().to(dt).requires_grad_(True)
    h0g, c0g = h0.cuda().to(dt).requires_grad_(True), c0.cuda().to(dt).requires_grad_(True)
    y, (hn, cn) = m(xg, (h0g, c0g))
    (y.float() * dout.cuda()).sum().backward()
    torch.cuda.synchronize()
    o_out, o_cell, o_ifgo = oracle.forward(x.numpy(), h0[0].numpy(), c0[0].numpy(), w["weight_ih_l0"], w["bias_ih_l0"],
                                           w["weight_hh_l0"], w["bias_hh_l0"], dtype=np.float32)
    r = oracle.backward(dout.numpy(), None, None, x.numpy(), o_out, o_cell, o_ifgo, w["weight_ih_l0"],
                        w["weight_hh_l0"], dtype=np.float32)
    _report([("out", rel_err(y, o_out[1:])), ("h_n", rel_err(hn[0], o_out[-1])), ("c_n", rel_err(cn[0], o_cell[-1])),
             ("dx", rel_err(xg.grad, r["dx"])), ("dh0", rel_err(h0g.grad[0], r["dh0"])),
             ("dc0", rel_err(c0g.grad[0], r["dc0"])), ("dW_x", rel_err(m.weight_ih_l0.grad, r["dWx"])),
             ("dW_h", rel_err(m.weight_hh_l0.grad, r["dWh"])), ("db_x", rel_err(m.bias_ih_l0.grad, r["db"])),
             ("db_h", rel_err(m.bias_hh_l0.grad, r["db"]))])


def test_config_E_fp16_two_layers_full_length_vs_fp32_oracle(oracle):
    T, B, I, H = 2048, 32, 1024, 1024
    dt = torch.float16
    assert _kind(T, B, H, dt, False) == 1 and _kind(T, B, H, dt, True) == 1   # XCD-local kernels at the real T
    assert L.stack2_runs_in_one_launch(T, B, I, H, dt, "cuda:0")              # both layers, one launch per direction
    m, w = _weights(I, H, 2, dt, 1238)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, B, I, generator=g).to(dt).float()
    dout = torch.randn(T, B, H, generator=g).to(dt).float()
    xg = x.cuda().to(dt).requires_grad_(True)
    y, (hn, cn) = m(xg)
    (y.float() * dout.cuda()).sum().backward()
    torch.cuda.synchronize()
    # the oracle, layer by layer: forward up, backward down (the upper layer's dx is the lower one's dout)
    fwd = []
    inp = x.numpy()
    for l in range(2):
        fwd.append(oracle.forward(inp, None, None, w["weight_ih_l%d" % l], w["bias_ih_l%d" % l],
                                  w["weight_hh_l%d" % l], w["bias_hh_l%d" % l], dtype=np.float32))
        inp = fwd[-1][0][1:]
    r1 = oracle.backward(dout.numpy(), None, None, fwd[0][0][1:], *fwd[1], w["weight_ih_l1"], w["weight_hh_l1"],
                         dtype=np.float32)
    r0 = oracle.backward(r1["dx"], None, None, x.numpy(), *fwd[0], w["weight_ih_l0"], w["weight_hh_l0"],
                         dtype=np.float32)
    rows = [("out", rel_err(y, fwd[1][0][1:])), ("dx", rel_err(xg.grad, r0["dx"]))]
    for l, r in ((0, r0), (1, r1)):
        rows += [("h_n[%d]" % l, rel_err(hn[l], fwd[l][0][-1])), ("c_n[%d]" % l, rel_err(cn[l], fwd[l][1][-1])),
                 ("dW_x[%d]" % l, rel_err(getattr(m, "weight_ih_l%d" % l).grad, r["dWx"])),
                 ("dW_h[%d]" % l, rel_err(getattr(m, "weight_hh_l%d" % l).grad, r["dWh"])),
                 ("db[%d]" % l, rel_err(getattr(m, "bias_ih_l%d" % l).grad, r["db"]))]
    _report(rows)


def test_stack2_at_2048_steps_is_bit_identical_to_layer_by_layer():
    """32 chunks of 64 timesteps through the chunk hand-over of both stacked launches, against the two
    layers called one after the other (GPU only: no CPU reference involved)."""
    T, B, I, H = 2048, 32, 1024, 1024
    dt = torch.float16
    assert _kind(T, B, H, dt, False) == 1 and _kind(T, B, H, dt, True) == 1
    assert L.stack2_runs_in_one_launch(T, B, I, H, dt, "cuda:0")
    g = torch.Generator().manual_seed(77)
    k = 1.0 / H ** 0.5
    u = lambda *s: ((torch.rand(*s, generator=g) * 2 - 1) * k).to(dt).cuda()
    x = torch.randn(T, B, I, generator=g).to(dt).cuda()
    dout = torch.randn(T, B, H, generator=g).to(dt).cuda()
    Wx0, bx0, Wh0, bh0 = u(4 * H, I), u(4 * H), u(4 * H, H), u(4 * H)
    Wx1, bx1, Wh1, bh1 = u(4 * H, H), u(4 * H), u(4 * H, H), u(4 * H)
    out0, cell0, ifgo0, out1, cell1, ifgo1 = L.lstm_persistent_fwd_stack2(x, None, None, Wx0, bx0, Wh0, bh0, None, None,
                                                                          Wx1, bx1, Wh1, bh1)
    a0, c0_, i0 = L.lstm_persistent_fwd(x, None, None, Wx0, bx0, Wh0, bh0)
    a1, c1_, i1 = L.lstm_persistent_fwd(a0[1:].contiguous(), None, None, Wx1, bx1, Wh1, bh1)
    for got, want in ((out0, a0), (cell0, c0_), (ifgo0, i0), (out1, a1), (cell1, c1_), (ifgo1, i1)):
        assert torch.equal(got, want)
    lo, up = L.lstm_persistent_bwd_stack2(dout, x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1)
    z = lambda: torch.zeros(B, H, device="cuda", dtype=dt)
    up_ref = L.lstm_persistent_bwd(dout, z(), z(), a0[1:].contiguous(), a1, c1_, i1, Wx1, Wh1)
    lo_ref = L.lstm_persistent_bwd(up_ref[0], z(), z(), x, a0, c0_, i0, Wx0, Wh0)
    for got, want, names in ((up, up_ref, "upper"), (lo, lo_ref, "lower")):
        for idx, name in ((0, "dx"), (1, "dh0"), (2, "dc0"), (4, "db")):
            assert torch.equal(got[idx], want[idx]), (names, name)
        for idx, name in ((3, "dWx"), (5, "dWh")):   # a different summation order over T*B
            assert rel_err(got[idx], want[idx]) < 2e-3, (names, name)

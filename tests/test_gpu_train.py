"""Training-loop check (run with -m gpu on an MI355X): the loop of the reference's scripts/overfit.py:10-43
-- a Linear head on top of the LSTM, Adam with lr 1e-3, mean squared error against fixed random targets,
under torch.autocast -- run with FastLSTM and with torch.nn.LSTM (MIOpen) from the same seed, so both start
from identical parameters (same RNG consumption, fastlstm/lstm.py:604-662), and compared step by step.

What is asserted, every 50th step and at the last one:
  * the two loss curves stay within BAND (relative, plus an absolute FLOOR) of each other -- they are two
    different 16-bit evaluations of the same optimisation, so they drift apart slowly, not bit for bit;
  * both stay within FP32_BAND of the same loop run in plain fp32 with nn.LSTM (no autocast);
  * the loss goes down by at least a third (the reference's script is an over-fitting smoke test);
  * parameters and their gradients stay fp32 (autocast casts inside the Function, lstm.py:509-515, the
    autograd engine casts the 16-bit gradients back), and no gradient is ever non-finite.
fp16 runs with a GradScaler (the reference's script does not scale; with the scaler the comparison also
covers scaled upstream gradients going through the reverse kernels).
"""
import pytest
import torch
import torch.nn as nn

import fastlstm_amd.lstm as L
from fastlstm_amd import FastLSTM

pytestmark = pytest.mark.gpu

STEPS = 250
BAND = 0.05        # FastLSTM vs nn.LSTM under the same autocast dtype, relative to the larger loss
FP32_BAND = 0.10   # either of them vs the fp32 loop
FLOOR = 1e-4       # absolute: the loop over-fits to a loss of ~1e-11 in fp32, far below what a 16-bit forward resolves


def _run(kind, precision, seq_len=128, batch_size=16, hidden_size=256, steps=STEPS):
    g = torch.Generator(device="cuda").manual_seed(7)
    y = torch.randn((seq_len, batch_size, 1), device="cuda", generator=g)
    x = torch.randn((seq_len, batch_size, hidden_size), device="cuda", generator=g)
    torch.manual_seed(123)
    onet = nn.Linear(in_features=hidden_size, out_features=1, device="cuda")
    if kind == "lstm":
        snet = nn.LSTM(hidden_size, hidden_size, device="cuda")
    else:
        snet = FastLSTM(hidden_size, hidden_size, version="persistent", device="cuda")
    params = list(onet.parameters()) + list(snet.parameters())
    opt = torch.optim.Adam(params, lr=1e-3)
    amp = precision in (torch.float16, torch.bfloat16)
    scaler = torch.amp.GradScaler("cuda", enabled=precision == torch.float16)
    losses = []
    for it in range(steps):
        opt.zero_grad()
        with torch.autocast("cuda", dtype=precision if amp else torch.bfloat16, enabled=amp):
            out = snet(x)[0]
            if amp and it == 0 and kind != "lstm":   # (nn.LSTM on MIOpen answers bf16 autocast in fp16)
                assert out.dtype == precision
            yhat = onet(out)
            loss = ((yhat.float() - y) ** 2).mean()
        scaler.scale(loss).backward()
        if it % 50 == 0 or it == steps - 1:
            for p in params:
                assert p.dtype == torch.float32 and p.grad.dtype == torch.float32
                assert torch.isfinite(p.grad).all()
            losses.append(loss.item())
        scaler.step(opt)
        scaler.update()
    return losses, [p.detach().clone() for p in snet.parameters()]


@pytest.fixture(scope="module")
def fp32_curve():
    return _run("lstm", None)[0]


@pytest.mark.parametrize("precision", [torch.float16, torch.bfloat16])
def test_overfit_loop_tracks_nn_lstm(precision, fp32_curve):
    old = L.CHECK_STATUS
    L.CHECK_STATUS = False   # the loop runs as a user's would: asynchronous, failures reported by the next call
    try:
        fast, fast_params = _run("persistent", precision)
    finally:
        L.CHECK_STATUS = old
    ref, ref_params = _run("lstm", precision)
    print("\n    step      FastLSTM      nn.LSTM   nn.LSTM fp32   (%s autocast)" % str(precision).replace("torch.", ""))
    marks = list(range(0, STEPS, 50)) + [STEPS - 1]
    for s, a, b, c in zip(marks, fast, ref, fp32_curve):
        print("    %4d  %12.4e %12.4e %12.4e" % (s, a, b, c))
    assert fast[0] == pytest.approx(ref[0], rel=2e-3)            # identical parameters at step 0
    assert fast[-1] < fast[0] * 2 / 3 and ref[-1] < ref[0] * 2 / 3
    for s, a, b, c in zip(marks, fast, ref, fp32_curve):
        assert abs(a - b) <= BAND * max(a, b) + FLOOR, (s, a, b)
        assert abs(a - c) <= FP32_BAND * max(a, c) + FLOOR, (s, a, c)
        assert abs(b - c) <= FP32_BAND * max(b, c) + FLOOR, (s, b, c)
    # after 250 Adam steps of 1e-3 the parameters have moved by up to ~0.25: the two runs end close to each other
    for p, q in zip(fast_params, ref_params):
        assert (p - q).abs().max().item() < 0.05

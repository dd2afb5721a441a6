"""Seeded sweep of the module's option surface against torch.nn.LSTM (fp32, CPU, same weights).

Every case draws its shape and options from its seed: sequence length, batch, input and hidden size
(multiples of the MFMA k-step and odd sizes alike, so the padded and the unpadded dispatch both occur),
1-4 layers, bidirectional, bias, batch_first, initial states given or not, dense or PackedSequence input,
state_grads, dtype.  The module chooses among its forms by shape (general / XCD-local / register-resident
kernels, pairs of layers in one launch, wavefronts of chunked launches, both directions side by side,
zero-padded sizes, packed batches cut at row ranges); whichever it takes, outputs, final states and every
gradient have to match nn.LSTM: fp32 rtol = atol = 1e-4 element by element, 16-bit <= 2e-2 of the reference's max-norm (reference evaluated with the rounded weights
and inputs)."""
import random

import pytest
import torch
from torch.nn.utils.rnn import pack_sequence

import fastlstm_amd.lstm as L
from fastlstm_amd import FastLSTM
from helpers import rel_err

pytestmark = pytest.mark.gpu

FP32_TOL, HALF_TOL = 1e-4, 2e-2


@pytest.fixture(scope="module", autouse=True)
def _check_every_launch():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    old = L.CHECK_STATUS
    L.CHECK_STATUS = True
    yield
    L.CHECK_STATUS = old


def draw(seed):
    r = random.Random(1000 + seed)
    dt = r.choice([torch.float32, torch.float16, torch.bfloat16])
    kw = dict(bidirectional=r.random() < 0.4, bias=r.random() < 0.8, batch_first=r.random() < 0.3)
    layers = r.choice([1, 1, 2, 2, 3, 4])
    T = r.choice([1, 3, 17, 33, 64, 70, 130, 260])
    B = r.choice([1, 2, 5, 16, 24, 33, 64, 70])
    I = r.choice([1, 7, 32, 50, 64, 100, 128, 200, 300])
    H = r.choice([8, 20, 32, 48, 64, 65, 96, 100, 128, 200, 256, 300, 384, 512, 650])
    if T * B * H * layers > 260 * 33 * 512 * 2:   # keep the CPU reference to seconds
        T = min(T, 70)
    return dict(dt=dt, kw=kw, layers=layers, T=T, B=B, I=I, H=H, states=r.random() < 0.5, packed=r.random() < 0.3,
                state_grads=r.random() < 0.5)


# Shapes at which the dispatch changes form: both directions side by side with a larger unit tile; two stacked
# layers in one launch at a small batch (chunks of 64 timesteps); reverse launches that keep all, only dx, or none
# of their GEMMs inside; row ranges of 32-row groups; a remainder of rows behind full fp32 register-resident
# launches; small hidden sizes that run as 64 units.
FORMS = [
    dict(dt=torch.float16, kw=dict(bidirectional=True, bias=True, batch_first=False), layers=1, T=64, B=128, I=256, H=256),
    dict(dt=torch.float16, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=2, T=256, B=16, I=1024, H=1024),
    dict(dt=torch.float16, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=1, T=64, B=128, I=768, H=768),
    dict(dt=torch.bfloat16, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=1, T=64, B=256, I=384, H=384),
    dict(dt=torch.bfloat16, kw=dict(bidirectional=False, bias=False, batch_first=True), layers=1, T=40, B=1024, I=512, H=512),
    dict(dt=torch.float32, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=1, T=20, B=144, I=64, H=1024),
    dict(dt=torch.float16, kw=dict(bidirectional=True, bias=True, batch_first=False), layers=2, T=40, B=24, I=48, H=48),
    dict(dt=torch.float32, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=2, T=40, B=24, I=48, H=48),
    # two stacked layers whose reverse launch takes both dx on its few idle workgroups and leaves the weight gradients
    # to launches of their own; three layers whose reverse pass goes pair by pair; an fp32 hidden size padded for the
    # reverse pass's sake
    dict(dt=torch.bfloat16, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=2, T=64, B=64, I=128, H=768),
    dict(dt=torch.bfloat16, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=3, T=130, B=48, I=64, H=576),
    dict(dt=torch.float32, kw=dict(bidirectional=False, bias=True, batch_first=False), layers=1, T=40, B=8, I=64, H=576),
]


@pytest.mark.parametrize("form", range(len(FORMS)))
def test_module_against_nn_lstm_where_the_dispatch_changes_form(form):
    c = dict(FORMS[form], states=form % 2 == 0, packed=False, state_grads=form % 3 == 0)
    _check(c, 100 + form)


@pytest.mark.parametrize("seed", range(48))
def test_module_against_nn_lstm(seed):
    _check(draw(seed), seed)


def _check(c, seed):
    dt, kw, layers, T, B, I, H = c["dt"], c["kw"], c["layers"], c["T"], c["B"], c["I"], c["H"]
    D = 2 if kw["bidirectional"] else 1
    torch.manual_seed(seed)
    m = FastLSTM(I, H, num_layers=layers, state_grads=c["state_grads"], **kw)
    # reference: nn.LSTM on the CPU; for the fp32 cases in float64, so that the element-wise 1e-4 bound measures this
    # build's error alone (a bias gradient is a sum over T*B terms of mixed sign: two fp32 evaluations of an element
    # near zero can differ by more than 1e-4 of it while each is well inside 1e-4 of the exact value)
    rdt = torch.float64 if dt == torch.float32 else torch.float32
    ref = torch.nn.LSTM(I, H, num_layers=layers, **kw).to(rdt)
    with torch.no_grad():
        for n, prm in m.named_parameters():
            prm.copy_(prm.to(dt).float())
            getattr(ref, n).copy_(prm)
    m = m.to("cuda", dt)
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(dt).float()
    h0, c0 = rnd(layers * D, B, H) * 0.3, rnd(layers * D, B, H) * 0.3
    wh, wc = rnd(layers * D, B, H), rnd(layers * D, B, H)
    state = (lambda *ts: tuple(ts)) if c["states"] else (lambda *ts: None)
    leaves = [t.cuda().to(dt).requires_grad_(True) for t in (h0, c0)]
    leaves_r = [t.clone().to(rdt).requires_grad_(True) for t in (h0, c0)]
    if c["packed"]:
        lengths = [int(v) for v in torch.randint(1, T + 1, (B,), generator=g)]
        seqs = [rnd(n, I) for n in lengths]
        xs = [s.cuda().to(dt).requires_grad_(True) for s in seqs]
        xr = [s.clone().to(rdt).requires_grad_(True) for s in seqs]
        y, (hn, cn) = m(pack_sequence(xs, enforce_sorted=False), state(*leaves))
        yr, (hr, cr) = ref(pack_sequence(xr, enforce_sorted=False), state(*leaves_r))
        assert torch.equal(y.batch_sizes, yr.batch_sizes)
        y, yr = y.data, yr.data
    else:
        x = rnd(B, T, I) if kw["batch_first"] else rnd(T, B, I)
        xs, xr = [x.cuda().to(dt).requires_grad_(True)], [x.clone().to(rdt).requires_grad_(True)]
        y, (hn, cn) = m(xs[0], state(*leaves))
        yr, (hr, cr) = ref(xr[0], state(*leaves_r))
    assert y.shape == yr.shape and hn.shape == hr.shape and cn.shape == cr.shape, c
    wy = rnd(*yr.shape)
    loss, loss_r = (y.float() * wy.cuda()).sum(), (yr * wy.to(rdt)).sum()
    if c["state_grads"] or c["packed"]:   # final states that carry a gradient
        loss, loss_r = loss + (hn.float() * wh.cuda()).sum(), loss_r + (hr * wh.to(rdt)).sum()
    if c["state_grads"] and not c["packed"]:
        loss, loss_r = loss + (cn.float() * wc.cuda()).sum(), loss_r + (cr * wc.to(rdt)).sum()
    loss.backward()
    loss_r.backward()
    rows = [(y, yr, "y"), (hn, hr, "hn"), (cn, cr, "cn")]
    # (the sequences of a packed batch as one tensor: the max-norm of a one-element gradient is no yardstick)
    rows += [(torch.cat([a.grad for a in xs]), torch.cat([b.grad for b in xr]), "dx")]
    if c["states"]:
        rows += [(a.grad, b.grad, n) for a, b, n in zip(leaves, leaves_r, ("dh0", "dc0"))]
    rows += [(prm.grad, getattr(ref, n).grad, n) for n, prm in m.named_parameters()]
    for got, want, name in rows:
        assert got is not None and got.shape == want.shape, (name, c)
        if dt == torch.float32:
            torch.testing.assert_close(got.detach().cpu().double(), want.detach().double(), rtol=FP32_TOL,
                                       atol=FP32_TOL, msg=lambda s: "%s %s: %s" % (name, c, s))
        else:
            assert rel_err(got, want) < HALF_TOL, (name, c, rel_err(got, want))


@pytest.mark.parametrize("dt,H,scale_x,scale_w", [
    (torch.float16, 64, 50.0, 1.0), (torch.float16, 1024, 100.0, 1.0), (torch.bfloat16, 2048, 20.0, 2.0),
    (torch.bfloat16, 300, 60.0, 2.0), (torch.float32, 256, 30.0, 3.0), (torch.float32, 1024, 100.0, 1.0)])
def test_saturated_gates_stay_finite_and_match_nn_lstm(dt, H, scale_x, scale_w):
    """Pre-activations of a few hundred: exp() of either sign overflows in the gate formulas, the gates have to
    come out as exactly 0 / 1 / +-1 all the same, with finite gradients (one kernel family per hidden size)."""
    torch.manual_seed(0)
    T, B, I = 40, 16, 64
    m = FastLSTM(I, H).to("cuda", dt)
    with torch.no_grad():
        for prm in m.parameters():
            prm.mul_(scale_w)
    ref = torch.nn.LSTM(I, H)
    ref.load_state_dict({k: v.float().cpu() for k, v in m.state_dict().items()})
    x = (torch.randn(T, B, I) * scale_x).to(dt)
    xg, xr = x.cuda().requires_grad_(True), x.float().requires_grad_(True)
    y, (hn, cn) = m(xg)
    y.float().sum().backward()
    yr, (hr, cr) = ref(xr)
    yr.sum().backward()
    rows = [(y, yr, "y"), (hn, hr, "hn"), (cn, cr, "cn"), (xg.grad, xr.grad, "dx")]
    rows += [(prm.grad, getattr(ref, n).grad, n) for n, prm in m.named_parameters()]
    for got, want, name in rows:
        assert torch.isfinite(got.float()).all(), name
        assert rel_err(got, want) < (FP32_TOL if dt == torch.float32 else HALF_TOL), (name, rel_err(got, want))

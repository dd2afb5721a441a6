"""Shared helpers for the parity tests: seeded problem generation and the
torch.nn.LSTM float64 reference (a library routine, used to pin the oracle)."""
import numpy as np
import torch


def make_problem(T, B, I, H, seed=0, h0=True, scale=None, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    k = (1.0 / H ** 0.5) if scale is None else scale
    u = lambda *s: (torch.rand(*s, generator=g, dtype=torch.float64) * 2 - 1) * k
    p = dict(
        x=torch.randn(T, B, I, generator=g, dtype=torch.float64),
        Wx=u(4 * H, I), Wh=u(4 * H, H), bx=u(4 * H), bh=u(4 * H),
        h0=torch.randn(B, H, generator=g, dtype=torch.float64) * 0.5 if h0 else None,
        c0=torch.randn(B, H, generator=g, dtype=torch.float64) * 0.5 if h0 else None,
        dout=torch.randn(T, B, H, generator=g, dtype=torch.float64),
        dh_n=torch.randn(B, H, generator=g, dtype=torch.float64),
        dc_n=torch.randn(B, H, generator=g, dtype=torch.float64),
    )
    return {k_: (v.to(dtype) if v is not None else None) for k_, v in p.items()}


def nn_lstm_reference(p, with_state_grads=True, dtype=torch.float64):
    """torch.nn.LSTM forward+autograd on the CPU with the problem's weights.
    loss = sum(out*dout) [+ sum(h_n*dh_n) + sum(c_n*dc_n)]."""
    T, B, I = p["x"].shape
    H = p["Wh"].shape[1]
    m = torch.nn.LSTM(I, H).to(dtype)
    with torch.no_grad():
        m.weight_ih_l0.copy_(p["Wx"]); m.weight_hh_l0.copy_(p["Wh"])
        m.bias_ih_l0.copy_(p["bx"]); m.bias_hh_l0.copy_(p["bh"])
    x = p["x"].to(dtype).clone().requires_grad_(True)
    if p["h0"] is not None:
        h0 = p["h0"].to(dtype).clone().requires_grad_(True)
        c0 = p["c0"].to(dtype).clone().requires_grad_(True)
        out, (hn, cn) = m(x, (h0[None], c0[None]))
    else:
        h0 = c0 = None
        out, (hn, cn) = m(x)
    loss = (out * p["dout"].to(dtype)).sum()
    if with_state_grads:
        loss = loss + (hn[0] * p["dh_n"].to(dtype)).sum() + (cn[0] * p["dc_n"].to(dtype)).sum()
    loss.backward()
    r = dict(out=out.detach(), h_n=hn[0].detach(), c_n=cn[0].detach(), dx=x.grad,
             dWx=m.weight_ih_l0.grad, dWh=m.weight_hh_l0.grad, dbx=m.bias_ih_l0.grad,
             dbh=m.bias_hh_l0.grad, dh0=None if h0 is None else h0.grad,
             dc0=None if c0 is None else c0.grad)
    return r


def to_np(p, keys):
    return [None if p[k] is None else p[k].detach().cpu().double().numpy() for k in keys]


def _np64(a):
    if torch.is_tensor(a):
        a = a.detach().double().cpu().numpy()
    return np.asarray(a, np.float64)


def rel_err(a, b):
    """max |a - b| / max |b| (error max-norm relative to the reference's max-norm)"""
    a = _np64(a); b = _np64(b)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def elementwise_ratio(got, want, rtol=1e-4, atol=1e-4):
    """max over elements of |got - want| / (atol + rtol * |want|): <= 1 means every element is within
    the allclose bound at these tolerances, with no scaling by the tensor's magnitude."""
    a = _np64(got); b = _np64(want)
    return float((np.abs(a - b) / (atol + rtol * np.abs(b))).max())

"""Pins the CPU oracle (oracle/lstm_oracle.c) before anything is compared with
it.  The reference's own tests hold no golden files -- every one of them is a
live comparison with torch.nn.LSTM / nn.LSTMCell (tests/test_lstm.py:21-220 in
the reference) -- so the oracle is pinned the same way, in float64, plus by
finite differences and closed-form special cases."""
import numpy as np
import pytest
import torch

from helpers import make_problem, nn_lstm_reference, to_np

FWD_KEYS = ["x", "h0", "c0", "Wx", "bx", "Wh", "bh"]
# shapes of the reference's tests: (63,12,128,213) test_lstm.py:46-69; ragged
# H/B of test_fastlstm (test_lstm.py:160-220) scaled to CPU time
SHAPES = [(7, 5, 11, 13), (63, 12, 128, 213), (10, 4, 123, 16), (10, 44, 123, 65), (1, 3, 4, 2)]


@pytest.mark.parametrize("T,B,I,H", SHAPES)
@pytest.mark.parametrize("h0", [True, False])
def test_forward_matches_nn_lstm(oracle, T, B, I, H, h0):
    p = make_problem(T, B, I, H, seed=T + B, h0=h0)
    ref = nn_lstm_reference(p)
    out, cell, ifgo = oracle.forward(*to_np(p, FWD_KEYS))
    assert out.shape == (T + 1, B, H) and cell.shape == (T + 1, B, H) and ifgo.shape == (T, B, 4 * H)
    np.testing.assert_allclose(out[1:], ref["out"].numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(out[-1], ref["h_n"].numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(cell[-1], ref["c_n"].numpy(), rtol=1e-11, atol=1e-12)
    if h0:
        np.testing.assert_array_equal(out[0], p["h0"].numpy())
        np.testing.assert_array_equal(cell[0], p["c0"].numpy())
    else:
        assert not out[0].any() and not cell[0].any()


def test_cell_trajectory_matches_lstmcell(oracle):
    T, B, I, H = 9, 6, 10, 7
    p = make_problem(T, B, I, H, seed=3)
    cellm = torch.nn.LSTMCell(I, H).double()
    with torch.no_grad():
        cellm.weight_ih.copy_(p["Wx"]); cellm.weight_hh.copy_(p["Wh"])
        cellm.bias_ih.copy_(p["bx"]); cellm.bias_hh.copy_(p["bh"])
        h, c = p["h0"], p["c0"]
        hs, cs = [h], [c]
        for t in range(T):
            h, c = cellm(p["x"][t], (h, c))
            hs.append(h); cs.append(c)
    out, cell, _ = oracle.forward(*to_np(p, FWD_KEYS))
    np.testing.assert_allclose(out, torch.stack(hs).numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(cell, torch.stack(cs).numpy(), rtol=1e-11, atol=1e-12)


def test_ifgo_is_the_preactivation(oracle):
    """ifgo[t] = x_t Wx^T + bx + bh + h_{t-1} Wh^T with library GEMMs, using
    nn.LSTM's own hidden states; gate order pinned by re-deriving c and h from
    the chunks with torch.sigmoid/tanh."""
    T, B, I, H = 6, 4, 9, 5
    p = make_problem(T, B, I, H, seed=5)
    ref = nn_lstm_reference(p)
    out, cell, ifgo = oracle.forward(*to_np(p, FWD_KEYS))
    hprev = torch.cat([p["h0"][None], ref["out"][:-1]])
    want = torch.nn.functional.linear(p["x"], p["Wx"], p["bx"] + p["bh"]) + \
        torch.nn.functional.linear(hprev, p["Wh"])
    np.testing.assert_allclose(ifgo, want.numpy(), rtol=1e-11, atol=1e-12)
    i, f, g, o = torch.from_numpy(ifgo).chunk(4, dim=-1)
    c_prev = torch.from_numpy(cell[:-1])
    c = torch.sigmoid(f) * c_prev + torch.sigmoid(i) * torch.tanh(g)
    np.testing.assert_allclose(cell[1:], c.numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(out[1:], (torch.sigmoid(o) * torch.tanh(c)).numpy(), rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("T,B,I,H", SHAPES)
@pytest.mark.parametrize("h0", [True, False])
def test_backward_matches_nn_lstm_autograd(oracle, T, B, I, H, h0):
    p = make_problem(T, B, I, H, seed=11 + T, h0=h0)
    ref = nn_lstm_reference(p, with_state_grads=True)
    out, cell, ifgo = oracle.forward(*to_np(p, FWD_KEYS))
    dout, dh_n, dc_n, x, Wx, Wh = to_np(p, ["dout", "dh_n", "dc_n", "x", "Wx", "Wh"])
    r = oracle.backward(dout, dh_n, dc_n, x, out, cell, ifgo, Wx, Wh)
    tol = dict(rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(r["dx"], ref["dx"].numpy(), **tol)
    np.testing.assert_allclose(r["dWx"], ref["dWx"].numpy(), **tol)
    np.testing.assert_allclose(r["dWh"], ref["dWh"].numpy(), **tol)
    np.testing.assert_allclose(r["db"], ref["dbx"].numpy(), **tol)
    np.testing.assert_allclose(r["db"], ref["dbh"].numpy(), **tol)
    if h0:
        np.testing.assert_allclose(r["dh0"], ref["dh0"].numpy(), **tol)
        np.testing.assert_allclose(r["dc0"], ref["dc0"].numpy(), **tol)


def test_backward_without_state_grads_equals_zero_state_grads(oracle):
    T, B, I, H = 5, 3, 4, 6
    p = make_problem(T, B, I, H, seed=2)
    out, cell, ifgo = oracle.forward(*to_np(p, FWD_KEYS))
    dout, x, Wx, Wh = to_np(p, ["dout", "x", "Wx", "Wh"])
    a = oracle.backward(dout, None, None, x, out, cell, ifgo, Wx, Wh)
    z = np.zeros((B, H))
    b = oracle.backward(dout, z, z, x, out, cell, ifgo, Wx, Wh)
    for k in a:
        np.testing.assert_array_equal(a[k], b[k])
    ref = nn_lstm_reference(p, with_state_grads=False)
    np.testing.assert_allclose(a["dWh"], ref["dWh"].numpy(), rtol=1e-9, atol=1e-10)


def test_d_ifgo_via_identity_input_projection(oracle):
    """With I = 4H, Wx = identity and bx = 0 the input adds straight onto the
    pre-activations, so nn.LSTM's autograd x.grad IS d_ifgo."""
    T, B, H = 6, 3, 4
    I = 4 * H
    p = make_problem(T, B, I, H, seed=9)
    p["Wx"] = torch.eye(I, dtype=torch.float64)
    p["bx"] = torch.zeros(I, dtype=torch.float64)
    ref = nn_lstm_reference(p)
    out, cell, ifgo = oracle.forward(*to_np(p, FWD_KEYS))
    dout, dh_n, dc_n, x, Wx, Wh = to_np(p, ["dout", "dh_n", "dc_n", "x", "Wx", "Wh"])
    r = oracle.backward(dout, dh_n, dc_n, x, out, cell, ifgo, Wx, Wh)
    np.testing.assert_allclose(r["d_ifgo"], ref["dx"].numpy(), rtol=1e-9, atol=1e-10)


def test_finite_differences_tiny(oracle):
    T, B, I, H = 3, 2, 2, 3
    p = make_problem(T, B, I, H, seed=1)
    args = to_np(p, FWD_KEYS)
    dout, dh_n, dc_n = to_np(p, ["dout", "dh_n", "dc_n"])

    def loss(a):
        out, cell, _ = oracle.forward(*a)
        return (out[1:] * dout).sum() + (out[-1] * dh_n).sum() + (cell[-1] * dc_n).sum()

    out, cell, ifgo = oracle.forward(*args)
    r = oracle.backward(dout, dh_n, dc_n, args[0], out, cell, ifgo, args[3], args[5])
    grads = {0: r["dx"], 1: r["dh0"], 2: r["dc0"], 3: r["dWx"], 4: r["db"], 5: r["dWh"], 6: r["db"]}
    eps = 1e-6
    for idx, g in grads.items():
        flat = args[idx].reshape(-1)
        for j in range(0, flat.size, max(1, flat.size // 7)):
            old = flat[j]
            flat[j] = old + eps; lp = loss(args)
            flat[j] = old - eps; lm = loss(args)
            flat[j] = old
            assert abs((lp - lm) / (2 * eps) - g.reshape(-1)[j]) < 1e-7, (idx, j)


def test_special_cases(oracle):
    T, B, I, H = 4, 3, 5, 6
    p = make_problem(T, B, I, H, seed=4, h0=False)
    # Wh = 0: every step is a point-wise function of x_t W^T + b and c_{t-1}
    p["Wh"] = torch.zeros_like(p["Wh"])
    out, cell, ifgo = oracle.forward(*to_np(p, FWD_KEYS))
    pre = torch.nn.functional.linear(p["x"], p["Wx"], p["bx"] + p["bh"])
    np.testing.assert_allclose(ifgo, pre.numpy(), rtol=1e-12, atol=1e-13)
    # 2-D x is one timestep (fastlstm/lstm.py:33-34)
    a = to_np(p, FWD_KEYS)
    o2, c2, _ = oracle.forward(a[0][0], *a[1:])
    np.testing.assert_allclose(o2[1], out[1], rtol=1e-12)
    np.testing.assert_allclose(c2[1], cell[1], rtol=1e-12)


def test_f32_variant_tracks_f64(oracle):
    T, B, I, H = 20, 6, 17, 19
    p = make_problem(T, B, I, H, seed=6)
    a = to_np(p, FWD_KEYS)
    o64, c64, p64 = oracle.forward(*a)
    o32, c32, p32 = oracle.forward(*a, dtype=np.float32)
    assert o32.dtype == np.float32
    np.testing.assert_allclose(o32, o64, atol=5e-6)
    np.testing.assert_allclose(p32, p64, atol=2e-5)
    dout, dh_n, dc_n = to_np(p, ["dout", "dh_n", "dc_n"])
    r64 = oracle.backward(dout, dh_n, dc_n, a[0], o64, c64, p64, a[3], a[5])
    r32 = oracle.backward(dout, dh_n, dc_n, a[0], o32, c32, p32, a[3], a[5], dtype=np.float32)
    for k in r64:
        np.testing.assert_allclose(r32[k], r64[k], atol=2e-4 * max(1.0, np.abs(r64[k]).max()))


def test_rounding_helpers_match_numpy_and_torch(oracle):
    rng = np.random.default_rng(0)
    v = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 5, 4000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, 6e-8, 5.96e-8, 2.98e-8, 2.99e-8,
                  6.1e-5, 6.2e-5, 1.0009765625, 1.00048828125, 1.00146484375], np.float32)])
    v = np.concatenate([v, -v]).astype(np.float32)
    want16 = v.astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(oracle.round_fp16(v), want16)
    wantbf = torch.from_numpy(v).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(oracle.round_bf16(v), wantbf)


@pytest.mark.parametrize("mode,tdt", [(1, torch.float16), (2, torch.bfloat16)])
def test_round_mode_stores_representable_values(oracle, mode, tdt):
    T, B, I, H = 12, 4, 8, 8
    p = make_problem(T, B, I, H, seed=8)
    a = to_np(p, FWD_KEYS)
    o, c, g = oracle.forward(*a, dtype=np.float32, round_mode=mode)
    for arr in (o[1:], c[1:], g):
        t = torch.from_numpy(arr)
        assert torch.equal(t.to(tdt).float(), t)
    o0, c0, g0 = oracle.forward(*a, dtype=np.float32)
    eps = 2.0 ** -10 if mode == 1 else 2.0 ** -7
    np.testing.assert_allclose(o, o0, atol=T * eps)


@pytest.mark.parametrize("mode,tdt", [(1, torch.float16), (2, torch.bfloat16)])
def test_backward_round_mode_rounds_d_ifgo_and_everything_downstream_uses_it(oracle, mode, tdt):
    """The 16-bit mode of the backward: the returned d_ifgo is representable in the 16-bit type, it is the
    unrounded one to within half a unit in the last place per step, and dx, dW_x, dW_h, db are exactly
    the matrix products / column sums of THAT rounded d_ifgo (a textbook matmul in float64)."""
    T, B, I, H = 9, 5, 7, 12
    p = make_problem(T, B, I, H, seed=21)
    a = to_np(p, FWD_KEYS)
    o, c, g = oracle.forward(*a, round_mode=mode)
    dout, dh_n, dc_n = to_np(p, ["dout", "dh_n", "dc_n"])
    r = oracle.backward(dout, dh_n, dc_n, a[0], o, c, g, a[3], a[5], round_mode=mode)
    r0 = oracle.backward(dout, dh_n, dc_n, a[0], o, c, g, a[3], a[5])
    d = torch.from_numpy(r["d_ifgo"])
    assert torch.equal(d.to(tdt).double(), d)
    eps = 2.0 ** -10 if mode == 1 else 2.0 ** -7
    np.testing.assert_allclose(r["d_ifgo"], r0["d_ifgo"], atol=T * eps * np.abs(r0["d_ifgo"]).max())
    assert np.abs(r["d_ifgo"] - r0["d_ifgo"]).max() > 0          # the mode does something
    d2 = r["d_ifgo"].reshape(T * B, 4 * H)
    np.testing.assert_allclose(r["dx"].reshape(T * B, I), d2 @ a[3], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(r["dWx"], d2.T @ a[0].reshape(T * B, I), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(r["dWh"], d2.T @ o[:-1].reshape(T * B, H), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(r["db"], d2.sum(0), rtol=1e-12, atol=1e-12)
    # the state gradients are the recurrent product of the rounded d_ifgo of step 0 / the carried dc
    np.testing.assert_allclose(r["dh0"], r["d_ifgo"][0] @ a[5], rtol=1e-12, atol=1e-12)

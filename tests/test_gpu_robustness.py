"""Robustness of the boundary (run with -m gpu): gradients that autograd does not ask for are not computed,
recurrent calls from several streams are ordered by the library, a failed launch shows in its own results,
and the host-side dispatch caches follow the kernel-family switch."""
import pytest
import torch

import fastlstm_amd
import fastlstm_amd.lstm as L
from fastlstm_amd import _lib

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _clean_state():
    yield
    lib = _lib.load()
    lib.fastlstm_set_spin_limit(400000000)
    lib.fastlstm_set_kernel_families(7)
    torch.cuda.synchronize()
    lib.fastlstm_device_status(0, 1)


def _module(I, H, layers, dt, seed, **kw):
    torch.manual_seed(seed)
    return fastlstm_amd.FastLSTM(I, H, num_layers=layers, dtype=dt, **kw).cuda()


# T, B, I, H, layers, dtype, keyword arguments:
#   the dx / dW products inside the reverse launch (idle CUs), as launches behind it, fp32 general kernels,
#   two layers in one launch each way, a wavefront of three layers, both directions side by side
PRUNE_CASES = [(96, 64, 1024, 1024, 1, torch.float16, {}),
               (64, 128, 512, 512, 1, torch.bfloat16, {}),
               (20, 16, 48, 160, 1, torch.float32, {}),
               (128, 32, 256, 1024, 2, torch.float16, {}),
               (128, 16, 96, 256, 3, torch.float16, {}),
               (64, 32, 128, 256, 1, torch.float16, {"bidirectional": True})]


@pytest.mark.parametrize("T,B,I,H,layers,dt,kw", PRUNE_CASES)
def test_gradient_of_the_input_is_computed_only_when_asked_for(T, B, I, H, layers, dt, kw):
    """x.requires_grad = False: autograd's needs_input_grad reaches the library as a null dx, the product
    d_ifgo . Wx of the lowest layer is skipped (inside the fused launch and outside it), x.grad stays None and
    every parameter gradient is the same bits as with the product computed."""
    m = _module(I, H, layers, dt, 3, **kw)
    g = torch.Generator().manual_seed(5)
    x0 = torch.randn(T, B, I, generator=g).to(dt).cuda()
    dout = torch.randn(T, B, H * (2 if kw.get("bidirectional") else 1), generator=g).to(dt).cuda()
    grads = []
    for want_dx in (True, False):
        m.zero_grad(set_to_none=True)
        x = x0.clone().requires_grad_(want_dx)
        y, _ = m(x)
        (y * dout).sum().backward()
        torch.cuda.synchronize()
        assert (x.grad is not None) == want_dx
        if want_dx:
            assert torch.isfinite(x.grad.float()).all() and x.grad.abs().max() > 0
        grads.append({n: p.grad.clone() for n, p in m.named_parameters()})
    assert fastlstm_amd.pending_status() == _lib.OK
    for n in grads[0]:
        assert torch.equal(grads[0][n], grads[1][n]), n


def test_null_dx_and_null_weight_gradients_through_the_c_abi():
    """fastlstm_bwd_layer with dx = NULL / with dWx = dWh = db = NULL: the other results are the bits of the full call."""
    T, B, I, H, dt = 96, 64, 1024, 1024, torch.float16
    g = torch.Generator().manual_seed(11)
    k = 1.0 / H ** 0.5
    u = lambda *s: ((torch.rand(*s, generator=g) * 2 - 1) * k).to(dt).cuda()
    x = torch.randn(T, B, I, generator=g).to(dt).cuda()
    Wx, bx, Wh, bh = u(4 * H, I), u(4 * H), u(4 * H, H), u(4 * H)
    dout = torch.randn(T, B, H, generator=g).to(dt).cuda()
    out, cell, ifgo = L.lstm_persistent_fwd(x, None, None, Wx, bx, Wh, bh)
    z = lambda: torch.zeros(B, H, device="cuda", dtype=dt)
    full = L.lstm_persistent_bwd(dout, z(), z(), x, out, cell, ifgo, Wx, Wh)
    no_dx = L.lstm_persistent_bwd(dout, z(), z(), x, out, cell, ifgo, Wx, Wh, need_dx=False)
    no_dw = L.lstm_persistent_bwd(dout, z(), z(), x, out, cell, ifgo, Wx, Wh, need_dw=False)
    torch.cuda.synchronize()
    assert no_dx[0] is None and all(t is None for t in no_dw[3:])
    for k_ in (1, 2, 3, 4, 5):
        assert torch.equal(full[k_], no_dx[k_]), k_
    for k_ in (0, 1, 2):
        assert torch.equal(full[k_], no_dw[k_]), k_
    # a null weight gradient next to the others is an argument error, not a silent skip
    lib = _lib.load()
    t = torch.zeros(64, device="cuda", dtype=dt)
    p = t.data_ptr()
    rc = lib.fastlstm_bwd_layer(p, p, p, p, p, p, p, p, p, p, p, p, None, p, p, 1 << 20, p, 1 << 20, 4, 16, 64, 64, 1,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.ERR_NULL


def test_recurrent_calls_from_two_streams_are_ordered_by_the_library():
    """Two forward + backward passes of a shape whose time loop holds half the device, issued from two streams
    with nothing between them: the library makes each recurrent call wait for the one before it on the other
    stream (an event per device), so neither starves the other until the time-out, and the results are the bits
    of the same passes run one after the other."""
    T, B, I, H, dt = 128, 64, 512, 1024, torch.float16
    mods = [_module(I, H, 1, dt, 20 + i) for i in range(2)]
    g = torch.Generator().manual_seed(9)
    xs = [torch.randn(T, B, I, generator=g).to(dt).cuda() for _ in range(2)]
    douts = [torch.randn(T, B, H, generator=g).to(dt).cuda() for _ in range(2)]

    def one(i):
        mods[i].zero_grad(set_to_none=True)
        x = xs[i].clone().requires_grad_(True)
        y, (hn, cn) = mods[i](x)
        (y * douts[i]).sum().backward()
        return [y.detach(), hn, cn, x.grad] + [p.grad for p in mods[i].parameters()]

    serial = [[t.clone() for t in one(i)] for i in range(2)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
    got = [None, None]
    for rep in range(3):   # several rounds: the passes of the two streams interleave differently each time
        for i, s in enumerate(streams):
            with torch.cuda.stream(s):
                got[i] = one(i)
    for s in streams:
        s.synchronize()
    torch.cuda.synchronize()
    assert fastlstm_amd.pending_status() == _lib.OK
    for i in range(2):
        for a, b in zip(serial[i], got[i]):
            assert torch.equal(a, b), i


def test_a_failed_launch_shows_in_its_own_results_and_in_pending_status():
    """Failure path forced from the host (a spin limit of one tick; every kernel still exits normally): the
    failing calls return success, their results hold NaN, pending_status reports the failure without a
    synchronisation of its own, and the module raises before it enqueues new work behind it."""
    lib = _lib.load()
    T, B, I, H, dt = 64, 16, 128, 512, torch.float16
    m = _module(I, H, 1, dt, 1)
    x = torch.randn(T, B, I, device="cuda").to(dt).requires_grad_(True)
    y, _ = m(x)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all() and fastlstm_amd.pending_status() == _lib.OK
    try:
        lib.fastlstm_set_spin_limit(1)
        y, (hn, cn) = m(x)           # returns normally: nothing synchronises
        torch.cuda.synchronize()
    finally:
        lib.fastlstm_set_spin_limit(400000000)
    assert torch.isnan(y[-1].float()).all() and torch.isnan(hn.float()).all() and torch.isnan(cn.float()).all()
    assert not torch.isfinite(y.float().sum())          # any loss over the output trips
    assert fastlstm_amd.pending_status() == _lib.ERR_TIMEOUT      # (reading does not clear)
    with pytest.raises(RuntimeError):
        m(x)                          # reported before new work is enqueued; the report is cleared
    assert fastlstm_amd.pending_status() == _lib.OK
    y, _ = m(x)                       # healthy again
    y.float().sum().backward()
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all() and torch.isfinite(x.grad.float()).all()
    # the reverse pass: a failed launch poisons dh_0, dc_0, db and the first timestep of dx
    out, cell, ifgo = L.lstm_persistent_fwd(x.detach(), None, None, m.weight_ih_l0.detach(), m.bias_ih_l0.detach(),
                                            m.weight_hh_l0.detach(), m.bias_hh_l0.detach())
    torch.cuda.synchronize()
    z = lambda: torch.zeros(B, H, device="cuda", dtype=dt)
    try:
        lib.fastlstm_set_spin_limit(1)
        r = L.lstm_persistent_bwd(torch.randn(T, B, H, device="cuda").to(dt), z(), z(), x.detach(), out, cell, ifgo,
                                  m.weight_ih_l0.detach(), m.weight_hh_l0.detach())
        torch.cuda.synchronize()
    finally:
        lib.fastlstm_set_spin_limit(400000000)
    assert torch.isnan(r[0][0].float()).all() and torch.isnan(r[1].float()).all() and torch.isnan(r[4].float()).all()
    assert fastlstm_amd.pending_status(clear=True) == _lib.ERR_TIMEOUT
    assert fastlstm_amd.pending_status() == _lib.OK


def test_dispatch_caches_follow_the_kernel_family_switch():
    """The host caches of which kernel a shape gets (and with them the padding and wavefront decisions) are keyed
    on the family mask: a switch changes the answer at once, and switching back restores it."""
    lib = _lib.load()
    code = L._DTYPE_CODE[torch.float16]
    assert lib.fastlstm_get_kernel_families() == 7
    assert L._recurrent_kind(64, 16, 512, code, 0) == 1
    chunks = L.stack_wavefront_chunks(2, 256, 16, 512, torch.float16, "cuda:0")
    assert chunks > 0
    lib.fastlstm_set_kernel_families(0)
    assert L._recurrent_kind(64, 16, 512, code, 0) == 0
    assert L.stack_wavefront_chunks(2, 256, 16, 512, torch.float16, "cuda:0") == 0
    lib.fastlstm_set_kernel_families(7)
    assert L._recurrent_kind(64, 16, 512, code, 0) == 1
    assert L.stack_wavefront_chunks(2, 256, 16, 512, torch.float16, "cuda:0") == chunks


def test_padded_operand_cache_is_opt_in_and_follows_the_version_counters():
    """Inference with a hidden size that runs zero-padded: with cache_padded_operands the padded weights are kept
    across calls and refreshed when a parameter's version counter moves (an optimizer-style in-place update)."""
    T, B, I, H, dt = 40, 16, 300, 300, torch.float16
    m = _module(I, H, 1, dt, 7)
    x = torch.randn(T, B, I, device="cuda").to(dt)
    with torch.no_grad():
        assert m._operand_padding(x) is not None        # this shape is padded
        y0 = m(x)[0].clone()
        assert not m.__dict__.get("_padded_operand_cache")    # off by default: nothing kept
        m.cache_padded_operands = True
        y1 = m(x)[0].clone()
        kept = m._padded_operand_cache
        assert len(kept) == 1 and torch.equal(y0, y1)
        first = next(iter(kept.values()))[1][0]
        y2 = m(x)[0].clone()
        assert next(iter(kept.values()))[1][0] is first and torch.equal(y1, y2)    # reused
        m.weight_hh_l0.mul_(0.5)                          # bumps the version counter
        y3 = m(x)[0].clone()
        assert next(iter(kept.values()))[1][0] is not first
        m.cache_padded_operands = False
        assert torch.equal(y3, m(x)[0]) and not torch.equal(y3, y2)

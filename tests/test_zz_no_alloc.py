"""The entry point that allocates nothing (fastlstm_fwd_layer_noalloc) against fastlstm_fwd_layer,
through the C ABI, two calls in a row on the same GPU, the second with a smaller input (run with -m gpu)."""
import pytest
import torch

import fastlstm_amd.lstm as L
from fastlstm_amd import _lib

pytestmark = pytest.mark.gpu


def _problem(T, B, I, H, dt, seed):
    g = torch.Generator().manual_seed(seed)
    k = 1.0 / H ** 0.5
    u = lambda *s: ((torch.rand(*s, generator=g) * 2 - 1) * k).to(dt).cuda()
    x = torch.randn(T, B, I, generator=g).to(dt).cuda()
    h0 = (torch.randn(B, H, generator=g) * 0.3).to(dt).cuda()
    c0 = (torch.randn(B, H, generator=g) * 0.3).to(dt).cuda()
    return x, h0, c0, u(4 * H, I), u(4 * H), u(4 * H), u(4 * H, H)


def _buffers(T, B, H, dt, h0, c0):
    ifgo = torch.empty(T, B, 4 * H, device="cuda", dtype=dt)
    out = torch.empty(T + 1, B, H, device="cuda", dtype=dt)
    cell = torch.empty(T + 1, B, H, device="cuda", dtype=dt)
    out[0], cell[0] = h0, c0
    return ifgo, out, cell


# first a shape whose ring fits the static array (XCD-local kernel, projection inside the launch, 5.3 MiB of
# the array written), then a smaller, ragged one (general kernel, its exchange blocks have padding that must
# read as zero: the array still holds the first call's data), then the first again
# ... and a batch of 300 rows at H = 1024, which runs as several launches over ranges of rows that share the array
# (the barrier counters are cleared in between)
CASES = [(40, 64, 256, 1024, torch.float16, 1), (12, 20, 48, 160, torch.float16, 2), (9, 33, 70, 300, torch.float32, 3),
         (40, 64, 256, 1024, torch.float16, 4), (24, 300, 128, 1024, torch.float16, 5)]


def test_noalloc_forward_equals_forward_with_a_workspace():
    assert torch.cuda.is_available()
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    cap = lib.fastlstm_noalloc_scratch_bytes()   # (also the set-up call: address of the array, status word, event)
    assert cap == 16 << 20
    for T, B, I, H, dt, seed in CASES:
        code = L._DTYPE_CODE[dt]
        x, h0, c0, Wx, bx, bh, Wh = _problem(T, B, I, H, dt, seed)
        plan = L._plan(torch.device("cuda:0"), B, H, code, False)
        nbytes = min(cap, max(lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 0), plan.ws_bytes))
        if H == 1024:   # the ring fits: the array serves the XCD-local kernel, not only the two-slot fall-back
            assert lib.fastlstm_recurrent_kernel_kind(T, B, H, code, 0, nbytes) == 1
        ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        ifgo_a, out_a, cell_a = _buffers(T, B, H, dt, h0, c0)
        _lib.check(lib.fastlstm_fwd_layer(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), Wh.data_ptr(),
                                          ifgo_a.data_ptr(), out_a.data_ptr(), cell_a.data_ptr(), ws.data_ptr(), ws.numel(),
                                          T, B, I, H, code, st), "fastlstm_fwd_layer")
        ifgo_b, out_b, cell_b = _buffers(T, B, H, dt, h0, c0)
        if B == 300:
            assert lib.fastlstm_recurrent_rows_per_launch(T, B, H, code, 0, nbytes) > 0   # several launches
        # the device's own count of free bytes (hipMemGetInfo): it would show a hipMalloc inside the library,
        # which torch's allocator statistics cannot
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        _lib.check(lib.fastlstm_fwd_layer_noalloc(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), Wh.data_ptr(),
                                                  ifgo_b.data_ptr(), out_b.data_ptr(), cell_b.data_ptr(), T, B, I, H, code,
                                                  st), "fastlstm_fwd_layer_noalloc")
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] == free_before
        torch.cuda.synchronize()
        assert lib.fastlstm_device_status(0, 0) == _lib.OK
        assert torch.equal(out_a, out_b), (T, B, I, H)
        assert torch.equal(cell_a, cell_b), (T, B, I, H)
        assert torch.equal(ifgo_a, ifgo_b), (T, B, I, H)
        assert torch.isfinite(out_b.float()).all()


def test_noalloc_rejects_a_shape_beyond_the_array():
    lib = _lib.load()
    # B = 4096 rows at H = 1024: the smallest workspace (flags + two exchange slots per batch chunk) is past 16 MiB
    T, B, I, H, code = 2, 4096, 16, 1024, 1
    plan = L._plan(torch.device("cuda:0"), B, H, code, False)
    if plan.ws_bytes <= lib.fastlstm_noalloc_scratch_bytes():
        pytest.skip("plan fits the array on this device: %d bytes" % plan.ws_bytes)
    t = torch.zeros(64, device="cuda", dtype=torch.float16)
    p = t.data_ptr()
    rc = lib.fastlstm_fwd_layer_noalloc(p, p, p, p, p, p, p, p, T, B, I, H, code, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.ERR_WORKSPACE

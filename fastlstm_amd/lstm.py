"""PyTorch-facing LSTM for AMD Instinct MI355X -- drop-in for fastlstm/lstm.py.

Mirrors the persistent path of the reference (names, argument meaning, return
layout, error behaviour):

    FastLSTM              fastlstm/lstm.py:586-698
    PersistentLSTMfn      fastlstm/lstm.py:504-538
    lstm_persistent_fwd   fastlstm/lstm.py:31-146
    lstm_persistent_bwd   fastlstm/lstm.py:236-334
    Wgrad                 fastlstm/lstm.py:494-501

Everything below the Python signatures is different: the host functions only
allocate torch tensors and call the C ABI of libfastlstm_hip.so (hand-written
gfx950 kernels) on the current HIP stream.  There is one code path, no Triton,
no autotune warm-up run and no CPU fallback: tensors must live on the GPU and
the library must be built, otherwise the calls raise.
"""
import ctypes
import functools
import os
import threading

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.amp import custom_bwd, custom_fwd

from . import _lib

dtype_str = {  # fastlstm/lstm.py:24-28
    torch.float32: "fp32",
    torch.float16: "fp16",
    torch.bfloat16: "bf16",
}
_DTYPE_CODE = {torch.float32: _lib.FP32, torch.float16: _lib.FP16, torch.bfloat16: _lib.BF16}

# When set, every recurrent launch is followed by a device sync and a check of the
# workspace status word (barrier time-out detection at the failing call itself).  Off by
# default: the calls are fully asynchronous, as in the reference, and a failed launch is
# reported by the NEXT library call on the device (fastlstm_device_status, no sync).
CHECK_STATUS = os.environ.get("FASTLSTM_CHECK_STATUS", "0") == "1"


# Host-phase profiler ranges (the reference brackets its host phases with torch.cuda.nvtx ranges,
# fastlstm/lstm.py:32-144, 237-292, 508-516; on ROCm they reach rocprofv3 --marker-trace as roctx ranges).
# Off unless FASTLSTM_PROFILE_RANGES=1: a range costs a microsecond or two of host time per phase.
PROFILE_RANGES = os.environ.get("FASTLSTM_PROFILE_RANGES", "0") == "1"


class _Range:
    __slots__ = ("name",)

    def __init__(self, name):
        self.name = name

    def __enter__(self):
        if PROFILE_RANGES:
            torch.cuda.nvtx.range_push(self.name)

    def __exit__(self, *exc):
        if PROFILE_RANGES:
            torch.cuda.nvtx.range_pop()
        return False


def pending_status(device=None, clear=False):
    """Status of the recurrent launches enqueued on `device` so far that have already run: 0, or the error code of a
    launch that ended in a barrier time-out or on the wrong XCD (fastlstm_device_status).  Reads one pinned host
    word: no synchronisation.  A launch that has not finished yet cannot be reported -- synchronise first to learn
    about the last call of a program.  clear=True resets the word."""
    if device is None:
        idx = torch.cuda.current_device()
    else:
        device = torch.device(device)
        idx = device.index if device.index is not None else torch.cuda.current_device()
    return _lib.load().fastlstm_device_status(idx, 1 if clear else 0)


def _raise_pending(device):
    """Raises for a failed earlier launch on `device` (and clears the report), before new work is enqueued behind
    it.  The results of the failed call itself hold NaN (the library poisons them), so a loss computed from them
    is not finite either."""
    status = pending_status(device, clear=True)
    if status != _lib.OK:
        _lib.check(status, "an earlier fastlstm launch on %s" % (device,))


def _raise_pending_before_backward(grad):
    if grad is not None and grad.is_cuda and not torch.cuda.is_current_stream_capturing():
        _raise_pending(grad.device)


def _code(t):
    if t.dtype not in _DTYPE_CODE:
        raise TypeError("fastlstm_amd supports float32, float16 and bfloat16, got %s" % t.dtype)
    return _DTYPE_CODE[t.dtype]


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "fastlstm_amd runs on the GPU only (tensor on %s); there is no CPU fallback" % t.device)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """Handle of the current stream of the current device (the raw accessor where this torch has it:
    torch.cuda.current_stream() costs ~25 us of host time per call, a third of a short forward call)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _plan(device, B, H, code, backward):
    idx = device.index if device.index is not None else torch.cuda.current_device()
    return _plan_cached(idx, B, H, code, int(backward))


@functools.lru_cache(maxsize=4096)
def _plan_cached(idx, B, H, code, backward):
    """The tiling of a (device, B, H, dtype, direction): a pure function of its arguments (the first call per device
    also probes the device), kept across calls -- callers only read the struct."""
    plan = _lib.Plan()
    _lib.check(_lib.load().fastlstm_plan_device(idx, B, H, code, backward, plan), "fastlstm_plan_device")
    return plan


def _workspace(plan, T, H, code, backward, device):
    """Recurrence workspace, with the part the kernels need zeroed (header, counters, flags; everything
    when the exchange blocks have padding).  Its size does not depend on T: every kernel exchanges
    h_t / d_ifgo[t] through two slots (a few hundred KiB; plans that stream W_h add one packed copy of it,
    which the call itself writes)."""
    n = _lib.load().fastlstm_recurrent_workspace_bytes(plan, T, H, code, 1 if backward else 0)
    ws = torch.empty(n, dtype=torch.uint8, device=device)
    ws[:(n if plan.ring_needs_zero else min(n, plan.ws_zero_bytes))].zero_()
    return ws


def _prepared_forward_workspace(plan, T, H, code, out, cell, h0, c0, stream):
    """The workspace of a forward call, cleared where the kernels need zeros, and out[0] / cell[0] set to the
    initial state (fastlstm/lstm.py:84-90) -- one launch (fastlstm_prepare_forward) instead of three."""
    lib = _lib.load()
    n = lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 0)
    ws = torch.empty(n, dtype=torch.uint8, device=out.device)
    zero = n if plan.ring_needs_zero else min(n, plan.ws_zero_bytes)
    direct = h0 is None or all(s_.dtype == out.dtype and s_.shape == out[0].shape and s_.is_contiguous() for s_ in (h0, c0))
    hp, cp = (h0.data_ptr(), c0.data_ptr()) if (direct and h0 is not None) else (None, None)
    _lib.check(lib.fastlstm_prepare_forward(ws.data_ptr(), zero, out.data_ptr(), cell.data_ptr(), hp, cp,
                                            out.shape[1], out.shape[2], code, stream), "fastlstm_prepare_forward")
    if not direct:   # another dtype, a broadcast or a strided state: torch converts (the slots hold zeros)
        out[0] = h0
        cell[0] = c0
    return ws


def _check_ws(ws, what):
    # (reading the status word synchronises: not while the stream is being captured into a graph)
    if CHECK_STATUS and not torch.cuda.is_current_stream_capturing():
        head = ws[:64].cpu().numpy().tobytes()  # synchronises
        status = _lib.load().fastlstm_ws_status(head)
        if status != _lib.OK:
            # reported here: the device's sticky status word need not report it again at the next call
            _lib.load().fastlstm_device_status(ws.device.index, 1)
        _lib.check(status, what)


def lstm_persistent_fwd(x, h0, c0, Wx, bx, Wh, bh, version=None, keep_activations=True):
    """x[T,B,I] (or [B,I]) -> (out[T+1,B,H], cell[T+1,B,H], ifgo[T,B,4H]).

    out[0]/cell[0] hold the initial state (zeros when h0 is None); ifgo holds
    the full gate pre-activations of every step (kept for the backward pass).
    `version` is accepted for signature compatibility; there is one path.
    keep_activations=False is the forward pass no backward pass follows: out and
    cell[-1] are the same bits, cell[1:-1] is uninitialised and ifgo holds the input
    projection only (the reference stores everything regardless, fastlstm/lstm.py:507-522).
    """
    if x.dim() == 2:  # fastlstm/lstm.py:33-34
        x = x[None]
    _require_gpu(x, Wx, bx, Wh, bh, h0, c0)
    code = _code(x)
    seq_len, batch_size, input_size = x.shape
    hidden_size = Wh.shape[1]
    assert x.is_contiguous()  # fastlstm/lstm.py:49-50
    assert Wh.is_contiguous()
    assert Wx.shape == (4 * hidden_size, input_size) and Wh.shape == (4 * hidden_size, hidden_size)
    for w in (Wx, bx, Wh, bh):
        if w.dtype != x.dtype:
            raise TypeError("weights must have the dtype of x (%s), got %s" % (x.dtype, w.dtype))
    Wx, bx, bh = Wx.contiguous(), bx.contiguous(), bh.contiguous()
    x = _aligned(x)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        ifgo = torch.empty((seq_len, batch_size, 4 * hidden_size), device=x.device, dtype=x.dtype)
        # two allocations (the reference slices one, lstm.py:84-86): each base pointer must
        # be 16-byte aligned for the vector loads of the weight-gradient GEMM
        out = torch.empty((seq_len + 1, batch_size, hidden_size), device=x.device, dtype=x.dtype)
        cell = torch.empty_like(out)
        with _Range("fastlstm: prepare forward"):
            plan = _plan(x.device, batch_size, hidden_size, code, False)
            stream = _stream()
            ws = _prepared_forward_workspace(plan, seq_len, hidden_size, code, out, cell, h0, c0, stream)
        # input projection + time loop in one call (the library fuses the two where CUs would idle)
        entry = lib.fastlstm_fwd_layer if keep_activations else lib.fastlstm_fwd_layer_infer
        with _Range("fastlstm: forward layer launch"):
            _lib.check(entry(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), Wh.data_ptr(),
                             ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), ws.data_ptr(),
                             ws.numel(), seq_len, batch_size, input_size, hidden_size, code, stream),
                       "fastlstm_fwd_layer")
        with _Range("fastlstm: status"):
            _check_ws(ws, "fastlstm_fwd_layer")
    return out, cell, ifgo


def _stack2_workspace(plan, T, H, code, device):
    """Workspace for fastlstm_fwd_stack2 (exchange slots for both layers); the part the kernels need
    zeroed is zeroed."""
    n = _lib.load().fastlstm_stack2_workspace_bytes(plan, T, H, code)
    ws = torch.empty(n, dtype=torch.uint8, device=device)
    ws[:(n if plan.ring_needs_zero else min(n, plan.ws_zero_bytes))].zero_()
    return ws


def stack2_runs_in_one_launch(T, B, I, H, dtype, device):
    """True if two stacked layers of this shape run as one launch (fastlstm_fwd_stack2_fused)."""
    if dtype not in _DTYPE_CODE or torch.device(device).type != "cuda":
        return False
    lib = _lib.load()
    code = _DTYPE_CODE[dtype]
    with torch.cuda.device(device):
        plan = _plan(torch.device(device), B, H, code, False)
        n = lib.fastlstm_stack2_workspace_bytes(plan, T, H, code)
        return lib.fastlstm_fwd_stack2_fused(T, B, I, H, code, n) == 1


def _aligned(t):
    """t itself, or a copy when its first byte is not 16-byte aligned (a slice such as out[1:] with
    an odd B*H): the library takes base pointers on 16-byte boundaries only."""
    return t if t.data_ptr() % 16 == 0 else t.clone()


def multi_runs_in_one_launch(n, T, B, H, dtype, device, backward=False):
    """True if n independent recurrences of this shape run as one launch (fastlstm_multi_fused)."""
    if dtype not in _DTYPE_CODE or torch.device(device).type != "cuda":
        return False
    lib = _lib.load()
    code = _DTYPE_CODE[dtype]
    with torch.cuda.device(device):
        plan = _plan(torch.device(device), B, H, code, backward)
        nb = lib.fastlstm_multi_workspace_bytes(plan, n, T, H, code, int(backward))
        return lib.fastlstm_multi_fused(n, T, B, H, code, int(backward), nb) == 1


def _families():
    """The kernel families the library may dispatch to (fastlstm_set_kernel_families; all of them unless a test or
    an experiment switched some off).  Part of every cache key below: their answers depend on it."""
    return _lib.load().fastlstm_get_kernel_families()


def _wavefront_chunks(L, T, B, H, dtype, device, backward):
    return _wavefront_chunks_cached(L, T, B, H, dtype, device, backward, _families())


@functools.lru_cache(maxsize=512)
def _wavefront_chunks_cached(L, T, B, H, dtype, device, backward, families):
    # chunks of at least 64 timesteps: every launch costs about 50 us besides its steps (launch gaps, the prologue,
    # the small GEMMs in between), which a chunk of 32 steps does not win back (measured: no gain at T = 256 with
    # 8 chunks); whole 16-byte units per timestep, so that every chunk's buffers start on a 16-byte boundary
    if T < 128 or (B * H * torch.empty((), dtype=dtype).element_size()) % 16:
        return 0
    for n in (8, 6, 5, 4, 3, 2):
        if T % n == 0 and T // n >= 64 and multi_runs_in_one_launch(L, T // n, B, H, dtype, device, backward):
            return n
    # no even cut: n equal chunks behind a prefix of T % n < n timesteps, which every layer runs on its own first
    for n in (8, 6, 5, 4, 3, 2):
        if T // n >= 64 and multi_runs_in_one_launch(L, T // n, B, H, dtype, device, backward):
            return n
    return 0


def stack_wavefront_chunks(L, T, B, H, dtype, device, backward=False):
    """Into how many chunks of timesteps L = 2 ... 4 stacked layers of this shape are cut so that layer l's chunk
    k - l runs beside the other layers' in launch k (0: they are not): the shapes whose L time loops fit the device
    side by side (multi_runs_in_one_launch)."""
    return _wavefront_chunks(int(L), int(T), int(B), int(H), dtype, str(torch.device(device)), bool(backward))


def stack2_wavefront_chunks(T, B, H, dtype, device, backward=False):
    """stack_wavefront_chunks for two layers."""
    return stack_wavefront_chunks(2, T, B, H, dtype, device, backward)


def _chunk_workspaces(n_bytes, zero_bytes, count, device):
    """`count` workspaces of n_bytes each, the first zero_bytes of every one cleared by ONE fill."""
    stride = (n_bytes + 255) // 256 * 256
    if zero_bytes >= n_bytes:
        buf = torch.zeros(count * stride, dtype=torch.uint8, device=device)
    else:
        buf = torch.empty(count * stride, dtype=torch.uint8, device=device)
        buf.view(count, stride)[:, :zero_bytes].zero_()
    return [buf[k * stride:k * stride + n_bytes] for k in range(count)]


def _ptr_array(ptrs):
    return (ctypes.c_void_p * len(ptrs))(*ptrs)


def _fwd_stack_wavefront(x, layers, n, keep_activations):
    """L = len(layers) stacked layers, layers[l] = (h0, c0, Wx, bx, Wh, bh), as n + L - 1 launches: launch k runs
    chunk k - l of layer l's time loop for every l side by side (fastlstm_fwd_persistent_multi on sub-ranges of the
    buffers: a time loop started at out[t0], cell[t0] continues the sequence); the input projection of an upper
    layer's chunk is a GEMM launch in between.  Returns [(out, cell, ifgo)] per layer.  (A chunk starts from the
    stored cell state, where the one-launch loop carries it in fp32: with 16-bit elements the results differ from
    the layer-by-layer path by that rounding, once per chunk.)"""
    lib = _lib.load()
    code = _code(x)
    T, B, I = x.shape
    H = layers[0][4].shape[1]
    L = len(layers)
    Tc = T // n
    dev_ = x.device
    stream = _stream()
    p = lambda t: t.data_ptr()
    bufs = []
    for h0, c0, *_ in layers:
        ifgo = torch.empty((T, B, 4 * H), device=dev_, dtype=x.dtype)
        out = torch.empty((T + 1, B, H), device=dev_, dtype=x.dtype)
        cell = torch.empty_like(out)
        if h0 is not None:
            out[0] = h0
            cell[0] = c0
        else:
            out[0].zero_()
            cell[0].zero_()
        bufs.append((out, cell, ifgo))
    Wx0, bx0, bh0 = layers[0][2], layers[0][3], layers[0][5]
    _lib.check(lib.fastlstm_gemm_ifgo(p(x), p(Wx0), p(bx0), p(bh0), p(bufs[0][2]), T, B, I, H, code, stream), "fastlstm_gemm_ifgo")
    plan = _plan(dev_, B, H, code, False)
    r = T - n * Tc   # timesteps in front of the n equal chunks (T not a multiple of n): layer by layer
    nb = lib.fastlstm_multi_workspace_bytes(plan, L, Tc, H, code, 0)
    wss = _chunk_workspaces(nb, nb if plan.ring_needs_zero else min(nb, plan.ws_zero_bytes), n + L - 1 + (L if r else 0), dev_)
    keep = int(keep_activations)
    # (addresses of the chunks by arithmetic: slicing tensors would cost the host more than a short chunk runs)
    row = B * H * x.element_size()
    po, pc, pg = [p(b[0]) for b in bufs], [p(b[1]) for b in bufs], [p(b[2]) for b in bufs]
    pw = [(p(l[2]), p(l[3]), p(l[4]), p(l[5])) for l in layers]   # Wx, bx, Wh, bh
    for l in range(L if r else 0):
        if l >= 1:
            _lib.check(lib.fastlstm_gemm_ifgo(po[l - 1] + row, pw[l][0], pw[l][1], pw[l][3], pg[l], r, B, H, H, code, stream),
                       "fastlstm_gemm_ifgo")
        ws = wss[n + L - 1 + l]
        _lib.check(lib.fastlstm_fwd_persistent_multi(1, _ptr_array([pg[l]]), _ptr_array([po[l]]), _ptr_array([pc[l]]),
                                                     _ptr_array([pw[l][2]]), p(ws), ws.numel(), r, B, H, code, keep, stream),
                   "fastlstm_fwd_persistent_multi")
    for k in range(n + L - 1):
        active = [l for l in range(L) if 0 <= k - l < n]
        for l in active:
            if l >= 1:   # this layer's projection of the chunk the layer below has just finished
                t = r + (k - l) * Tc
                _lib.check(lib.fastlstm_gemm_ifgo(po[l - 1] + (1 + t) * row, pw[l][0], pw[l][1], pw[l][3], pg[l] + t * 4 * row,
                                                  Tc, B, H, H, code, stream), "fastlstm_gemm_ifgo")
        t_of = [r + (k - l) * Tc for l in active]
        ws = wss[k]
        _lib.check(lib.fastlstm_fwd_persistent_multi(
            len(active), _ptr_array([pg[l] + t * 4 * row for l, t in zip(active, t_of)]),
            _ptr_array([po[l] + t * row for l, t in zip(active, t_of)]), _ptr_array([pc[l] + t * row for l, t in zip(active, t_of)]),
            _ptr_array([pw[l][2] for l in active]), p(ws), ws.numel(), Tc, B, H, code, keep, stream), "fastlstm_fwd_persistent_multi")
    for ws in wss:
        _check_ws(ws, "fastlstm_fwd_persistent_multi")
    return bufs


def _bwd_stack_wavefront(dh, x, acts, weights, d_states, n, need_dx=True):
    """Reverse pass of _fwd_stack_wavefront: acts[l] = (out, cell, ifgo), weights[l] = (Wx, Wh), d_states[l] = None or
    (dh_n, dc_n).  Launch k runs chunk n - 1 - (k - u) of layer L - 1 - u for every u side by side; a lower layer's
    dout of a chunk (the dx of the layer above) is a GEMM launch in between; the weight gradients and the lowest
    layer's dx follow over the whole sequence.  Returns [(d_x, dh_0, dc_0, dWx, dbx, dWh, dbh)] per layer."""
    lib = _lib.load()
    L = len(acts)
    code = _code(acts[0][2])
    T, B, H = dh.shape
    I = weights[0][0].shape[1]
    Tc = T // n
    dev_ = x.device
    dt = acts[0][2].dtype
    stream = _stream()
    p = lambda t: t.data_ptr()
    dh = dh.contiguous()
    if dh.dtype != dt:
        dh = dh.to(dt)
    dh, x = _aligned(dh), _aligned(x.contiguous())
    state = lambda d, k: (torch.zeros((B, H), device=dev_, dtype=dt) if d is None else d[k].to(dt).reshape(B, H).clone())
    dhs, dcs = [state(d, 0) for d in d_states], [state(d, 1) for d in d_states]
    d_ifgo = [torch.empty_like(a[2]) for a in acts]
    # douts[l]: gradient of layer l's out[1:]: dh for the top layer, the dx of layer l + 1 below it
    douts = [torch.empty((T, B, H), device=dev_, dtype=dt) for _ in range(L - 1)] + [dh]
    plan = _plan(dev_, B, H, code, True)
    r = T - n * Tc   # the prefix of the forward pass: here behind the chunks, layer by layer from the top
    nb = lib.fastlstm_multi_workspace_bytes(plan, L, Tc, H, code, 1)
    wss = _chunk_workspaces(nb, nb if plan.ring_needs_zero else min(nb, plan.ws_zero_bytes), n + L - 1 + (L if r else 0), dev_)
    row = B * H * dh.element_size()
    pdo, pdg = [p(t) for t in douts], [p(t) for t in d_ifgo]
    pg, pc = [p(a[2]) for a in acts], [p(a[1]) for a in acts]
    Wxc = [w[0].contiguous() for w in weights]
    pWx, pWh = [p(w) for w in Wxc], [p(w[1]) for w in weights]
    pdh, pdc = [p(t) for t in dhs], [p(t) for t in dcs]
    for k in range(n + L - 1):
        active = [L - 1 - u for u in range(L) if 0 <= k - u < n]          # layers, top first
        t_of = [r + (n - 1 - (k - (L - 1 - l))) * Tc for l in active]
        for l, t in zip(active, t_of):
            if l < L - 1:   # this layer's dout of the chunk the layer above has just finished
                _lib.check(lib.fastlstm_gemm_dx(pdg[l + 1] + t * 4 * row, pWx[l + 1], pdo[l] + t * row, Tc, B, H, H, code, stream),
                           "fastlstm_gemm_dx")
        ws = wss[k]
        _lib.check(lib.fastlstm_bwd_persistent_multi(
            len(active), _ptr_array([pdo[l] + t * row for l, t in zip(active, t_of)]), _ptr_array([pdh[l] for l in active]),
            _ptr_array([pdc[l] for l in active]), _ptr_array([pg[l] + t * 4 * row for l, t in zip(active, t_of)]),
            _ptr_array([pc[l] + t * row for l, t in zip(active, t_of)]), _ptr_array([pdg[l] + t * 4 * row for l, t in zip(active, t_of)]),
            _ptr_array([pWh[l] for l in active]), p(ws), ws.numel(), Tc, B, H, code, stream), "fastlstm_bwd_persistent_multi")
    for l in range(L - 1, -1, -1) if r else ():
        if l < L - 1:
            _lib.check(lib.fastlstm_gemm_dx(pdg[l + 1], pWx[l + 1], pdo[l], r, B, H, H, code, stream), "fastlstm_gemm_dx")
        ws = wss[n + L - 1 + l]
        _lib.check(lib.fastlstm_bwd_persistent_multi(
            1, _ptr_array([pdo[l]]), _ptr_array([pdh[l]]), _ptr_array([pdc[l]]), _ptr_array([pg[l]]), _ptr_array([pc[l]]),
            _ptr_array([pdg[l]]), _ptr_array([pWh[l]]), p(ws), ws.numel(), r, B, H, code, stream), "fastlstm_bwd_persistent_multi")
    for ws in wss:
        _check_ws(ws, "fastlstm_bwd_persistent_multi")
    res = []
    for l in range(L):
        if l == 0:   # (need_dx false: no gradient of the stack's input is asked for)
            dx0, db, _, dWx, dWh = DxWgrad(d_ifgo[0], Wxc[0], x, acts[0][0], need_dx)
        else:
            db, _, dWx, dWh = Wgrad(d_ifgo[l], acts[l - 1][0][1:], acts[l][0])
        res.append((dx0 if l == 0 else douts[l - 1], dhs[l], dcs[l], dWx, db, dWh, db))
    return res


def _fwd_stack2_wavefront(x, h0a, c0a, Wx0, bx0, Wh0, bh0, h0b, c0b, Wx1, bx1, Wh1, bh1, n, keep_activations):
    (out0, cell0, ifgo0), (out1, cell1, ifgo1) = _fwd_stack_wavefront(
        x, [(h0a, c0a, Wx0, bx0, Wh0, bh0), (h0b, c0b, Wx1, bx1, Wh1, bh1)], n, keep_activations)
    return out0, cell0, ifgo0, out1, cell1, ifgo1


def _bwd_stack2_wavefront(dh, x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1, d_state0, d_state1, n,
                          need_dx=True):
    r0, r1 = _bwd_stack_wavefront(dh, x, [(out0, cell0, ifgo0), (out1, cell1, ifgo1)], [(Wx0, Wh0), (Wx1, Wh1)],
                                  [d_state0, d_state1], n, need_dx)
    return r0, r1


def lstm_persistent_fwd_stack(x, layers, keep_activations=True):
    """L = 2 ... 4 stacked layers, layers[l] = (h0 | None, c0 | None, Wx, bx, Wh, bh): [(out, cell, ifgo)] per layer,
    the results of L calls of lstm_persistent_fwd in a row (16-bit elements: up to the rounding of the cell state at
    chunk boundaries, see _fwd_stack_wavefront).  Needs stack_wavefront_chunks(L, ...) > 0."""
    if x.dim() == 2:
        x = x[None]
    _require_gpu(x, *(t for l in layers for t in l))
    T, B, I = x.shape
    H = layers[0][4].shape[1]
    assert x.is_contiguous()
    for l, (_, _, Wx, bx, Wh, bh) in enumerate(layers):
        assert Wx.shape == (4 * H, I if l == 0 else H) and Wh.shape == (4 * H, H) and Wh.is_contiguous()
        for w in (Wx, bx, Wh, bh):
            if w.dtype != x.dtype:
                raise TypeError("weights must have the dtype of x (%s), got %s" % (x.dtype, w.dtype))
    layers = [(h0, c0, Wx.contiguous(), bx.contiguous(), Wh, bh.contiguous()) for h0, c0, Wx, bx, Wh, bh in layers]
    with torch.cuda.device(x.device):
        n = stack_wavefront_chunks(len(layers), T, B, H, x.dtype, x.device)
        if not n:
            raise ValueError("no wavefront for %d layers of this shape" % len(layers))
        return _fwd_stack_wavefront(_aligned(x), layers, n, keep_activations)


def _pairs_min_hidden(B):
    """Hidden size from which the reverse pass of three or more stacked layers goes pair by pair (see
    lstm_persistent_bwd_stack)."""
    return 576 if B > 32 else 704


def lstm_persistent_bwd_stack(dh, x, acts, weights, d_states=None, need_dx=True):
    """Reverse pass of lstm_persistent_fwd_stack: acts[l] = (out, cell, ifgo), weights[l] = (Wx, Wh), d_states[l] = None
    or (dh_n, dc_n).  [(d_x, dh_0, dc_0, dWx, dbx, dWh, dbh)] per layer; falls back to one layer after the other where
    the reverse time loops do not fit side by side.  need_dx=False: the lowest layer's d_x is not computed (None)."""
    L = len(acts)
    d_states = list(d_states) if d_states is not None else [None] * L
    T, B, H = dh.shape
    with torch.cuda.device(x.device):
        lib = _lib.load()
        code = _code(acts[0][2])
        res = [None] * L
        # From H = 704 on (576 with more than 32 rows), the reverse pass is faster as the library's two-layer launches
        # from the top down (the GEMMs inside them) than as one wavefront with the GEMMs in the open, whichever way the
        # forward pass went (4 x (T = 512, I = H): forward + backward H = 1024, B = 16 6.60 against 7.59 ms, H = 768,
        # B = 16 6.16 / 6.82, H = 1024, B = 8 6.52 / 7.21; level at H = 512; H = 384 7.68 / 6.90; 4 x (T = 512, I = 256,
        # H = 576): B = 48 6.66 / 9.13, B = 64 7.69 / 9.71, B = 32 6.34 / 6.49).
        plan = _plan(x.device, B, H, code, True)
        # (the pairs from the top down: the lowest pair reads the stack's input, whose size need not be H)
        lowest_I = x.shape[-1] if L % 2 == 0 else H
        pair_fused = lambda I_: lib.fastlstm_bwd_stack2_fused(
            T, B, I_, H, code, lib.fastlstm_stack2_bwd_workspace_bytes(plan, T, H, code)) == 1
        if L >= 3 and H >= _pairs_min_hidden(B) and pair_fused(H) and (lowest_I == H or pair_fused(lowest_I)):
            l = L - 1
            while l >= 1:
                xin = x if l == 1 else acts[l - 2][0][1:]
                res[l - 1], res[l] = lstm_persistent_bwd_stack2(dh, xin, *acts[l - 1], weights[l - 1][0], weights[l - 1][1],
                                                                *acts[l], weights[l][0], weights[l][1],
                                                                d_state0=d_states[l - 1], d_state1=d_states[l],
                                                                need_dx=need_dx or l > 1)
                dh = res[l - 1][0]
                l -= 2
            L = l + 1   # a lowest layer without a partner follows below
        else:
            n = stack_wavefront_chunks(L, T, B, H, acts[0][2].dtype, x.device, backward=True)
            if n:
                return _bwd_stack_wavefront(dh, x, acts, weights, d_states, n, need_dx)
        for l in range(L - 1, -1, -1):
            out, cell, ifgo = acts[l]
            dt = ifgo.dtype
            zeros = lambda: torch.zeros((B, H), device=x.device, dtype=dt)
            dhn, dcn = (zeros(), zeros()) if d_states[l] is None else tuple(d.to(dt).reshape(B, H).clone() for d in d_states[l])
            xin = x if l == 0 else acts[l - 1][0][1:]
            res[l] = lstm_persistent_bwd(dh, dcn, dhn, xin, out, cell, ifgo, weights[l][0], weights[l][1],
                                         need_dx=need_dx or l > 0)
            dh = res[l][0]
        return res


def lstm_persistent_fwd_stack2(x, h0a, c0a, Wx0, bx0, Wh0, bh0, h0b, c0b, Wx1, bx1, Wh1, bh1, keep_activations=True):
    """Two stacked layers (the second reads the first one's h): returns
    (out0, cell0, ifgo0, out1, cell1, ifgo1) with the layouts of lstm_persistent_fwd.  The same
    results as two calls of lstm_persistent_fwd (two iterations of the layer loop at
    fastlstm/lstm.py:685-696); one launch where the library can run both recurrences side by side."""
    if x.dim() == 2:
        x = x[None]
    _require_gpu(x, Wx0, bx0, Wh0, bh0, Wx1, bx1, Wh1, bh1, h0a, c0a, h0b, c0b)
    code = _code(x)
    T, B, I = x.shape
    H = Wh0.shape[1]
    assert x.is_contiguous() and Wh0.is_contiguous() and Wh1.is_contiguous()
    assert Wx0.shape == (4 * H, I) and Wh0.shape == (4 * H, H) and Wx1.shape == (4 * H, H) and Wh1.shape == (4 * H, H)
    for w in (Wx0, bx0, Wh0, bh0, Wx1, bx1, Wh1, bh1):
        if w.dtype != x.dtype:
            raise TypeError("weights must have the dtype of x (%s), got %s" % (x.dtype, w.dtype))
    Wx0, bx0, bh0, Wx1, bx1, bh1 = (t.contiguous() for t in (Wx0, bx0, bh0, Wx1, bx1, bh1))
    x = _aligned(x)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        n = stack2_wavefront_chunks(T, B, H, x.dtype, x.device)
        # (the library's own two-layer launch, with the GEMMs inside, wins wherever it applies)
        if n and not stack2_runs_in_one_launch(T, B, I, H, x.dtype, x.device):
            return _fwd_stack2_wavefront(x, h0a, c0a, Wx0, bx0, Wh0, bh0, h0b, c0b, Wx1, bx1, Wh1, bh1, n, keep_activations)
        bufs = []
        for h0, c0 in ((h0a, c0a), (h0b, c0b)):
            ifgo = torch.empty((T, B, 4 * H), device=x.device, dtype=x.dtype)
            out = torch.empty((T + 1, B, H), device=x.device, dtype=x.dtype)
            cell = torch.empty_like(out)
            if h0 is not None:
                out[0] = h0
                cell[0] = c0
            else:
                out[0].zero_()
                cell[0].zero_()
            bufs.append((out, cell, ifgo))
        (out0, cell0, ifgo0), (out1, cell1, ifgo1) = bufs
        plan = _plan(x.device, B, H, code, False)
        ws = _stack2_workspace(plan, T, H, code, x.device)
        entry = lib.fastlstm_fwd_stack2 if keep_activations else lib.fastlstm_fwd_stack2_infer
        _lib.check(entry(x.data_ptr(), Wx0.data_ptr(), bx0.data_ptr(), bh0.data_ptr(), Wh0.data_ptr(),
                         ifgo0.data_ptr(), out0.data_ptr(), cell0.data_ptr(), Wx1.data_ptr(),
                         bx1.data_ptr(), bh1.data_ptr(), Wh1.data_ptr(), ifgo1.data_ptr(),
                         out1.data_ptr(), cell1.data_ptr(), ws.data_ptr(), ws.numel(), T, B, I, H,
                         code, _stream()), "fastlstm_fwd_stack2")
        _check_ws(ws, "fastlstm_fwd_stack2")
    return out0, cell0, ifgo0, out1, cell1, ifgo1


def Wgrad(d_ifgo, x, h):
    """(dbx, dbh, dWx, dWh) from d_ifgo[T,B,4H], x[T,B,I], h[T+1,B,H]
    (fastlstm/lstm.py:494-501; the same db tensor is returned twice)."""
    _require_gpu(d_ifgo, x, h)
    code = _code(d_ifgo)
    T, B, G = d_ifgo.shape
    H, I = G // 4, x.shape[-1]
    lib = _lib.load()
    with torch.cuda.device(x.device):
        d_ifgo, x, h = _aligned(d_ifgo.contiguous()), _aligned(x.contiguous()), _aligned(h.contiguous())
        dWx = torch.empty((G, I), device=x.device, dtype=x.dtype)
        dWh = torch.empty((G, H), device=x.device, dtype=x.dtype)
        db = torch.empty((G,), device=x.device, dtype=x.dtype)
        nbytes = lib.fastlstm_wgrad_workspace_bytes(T, B, I, H, code)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        _lib.check(lib.fastlstm_gemm_wgrad(d_ifgo.data_ptr(), x.data_ptr(), h.data_ptr(), dWx.data_ptr(),
                                           dWh.data_ptr(), db.data_ptr(), ws.data_ptr(), ws.numel(), T, B, I,
                                           H, code, _stream()), "fastlstm_gemm_wgrad")
    return db, db, dWx, dWh


def DxWgrad(d_ifgo, Wx, x, h, need_dx=True):
    """(d_x | None, dbx, dbh, dWx, dWh): the input gradient d_ifgo . Wx (fastlstm/lstm.py:294) and Wgrad
    (fastlstm/lstm.py:494-501) in one library call -- one pass over d_ifgo for a narrow layer, the two stages
    otherwise."""
    _require_gpu(d_ifgo, x, h, Wx)
    code = _code(d_ifgo)
    T, B, G = d_ifgo.shape
    H, I = G // 4, x.shape[-1]
    lib = _lib.load()
    with torch.cuda.device(x.device):
        d_ifgo, x, h, Wx = _aligned(d_ifgo.contiguous()), _aligned(x.contiguous()), _aligned(h.contiguous()), _aligned(Wx.contiguous())
        d_x = torch.empty_like(x) if need_dx else None
        dWx = torch.empty((G, I), device=x.device, dtype=x.dtype)
        dWh = torch.empty((G, H), device=x.device, dtype=x.dtype)
        db = torch.empty((G,), device=x.device, dtype=x.dtype)
        nbytes = lib.fastlstm_wgrad_workspace_bytes(T, B, I, H, code)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        _lib.check(lib.fastlstm_gemm_dx_wgrad(d_ifgo.data_ptr(), Wx.data_ptr(), x.data_ptr(), h.data_ptr(),
                                              d_x.data_ptr() if need_dx else None, dWx.data_ptr(), dWh.data_ptr(),
                                              db.data_ptr(), ws.data_ptr(), ws.numel(), T, B, I, H, code, _stream()),
                   "fastlstm_gemm_dx_wgrad")
    return d_x, db, db, dWx, dWh


def lstm_persistent_bwd(dh, dc_n, dh_n, x, h, cell, ifgo, Wx, Wh, need_dx=True, need_dw=True):
    """Reverse pass.  dh[T,B,H]: gradient of out[1:]; dc_n, dh_n [B,H]: gradients
    flowing into the last cell / hidden state, overwritten with the gradients of
    the initial state and returned (fastlstm/lstm.py:236-334).  dc_n = dh_n = None: no gradient flows
    into the final state (the buffers are made here and zeroed by the launch that clears the workspace).
    Returns (d_x, dh_0, dc_0, dWx, dbx, dWh, dbh).  need_dx=False: the product d_ifgo . Wx is
    skipped and d_x is None (no gradient of the layer's input is asked for: the first layer of most
    models); need_dw=False: the weight and bias gradients are skipped and None (frozen weights).
    The reference computes all of them whatever autograd asks for (fastlstm/lstm.py:524-538)."""
    no_state_grad = dc_n is None and dh_n is None
    _require_gpu(dh, x, h, cell, ifgo, Wx, Wh, *(() if no_state_grad else (dc_n, dh_n)))
    code = _code(ifgo)
    seq_len, batch_size, hidden_size = dh.shape
    input_size = Wx.shape[1]
    lib = _lib.load()
    with torch.cuda.device(x.device):
        dh = dh.contiguous()
        if dh.dtype != ifgo.dtype:
            dh = dh.to(ifgo.dtype)
        dh = _aligned(dh)
        if PROFILE_RANGES:
            torch.cuda.nvtx.range_push("fastlstm: prepare backward")
        d_ifgo = torch.empty_like(ifgo)
        plan = _plan(x.device, batch_size, hidden_size, code, True)
        stream = _stream()
        if no_state_grad:   # one launch: workspace cleared, both state gradients zero
            dc_n, dh_n = torch.empty_like(cell[0]), torch.empty_like(cell[0])
            n = lib.fastlstm_recurrent_workspace_bytes(plan, seq_len, hidden_size, code, 1)
            ws = torch.empty(n, dtype=torch.uint8, device=x.device)
            _lib.check(lib.fastlstm_prepare_forward(ws.data_ptr(), n if plan.ring_needs_zero else min(n, plan.ws_zero_bytes),
                                                    dh_n.data_ptr(), dc_n.data_ptr(), None, None, batch_size, hidden_size,
                                                    code, stream), "fastlstm_prepare_forward")
        else:
            assert dc_n.is_contiguous() and dh_n.is_contiguous()
            ws = _workspace(plan, seq_len, hidden_size, code, True, x.device)
        x, h = _aligned(x.contiguous()), h.contiguous()
        d_x = torch.empty_like(x) if need_dx else None
        G = 4 * hidden_size
        dWx = dWh = db = None
        if need_dw:
            dWx = torch.empty((G, input_size), device=x.device, dtype=x.dtype)
            dWh = torch.empty((G, hidden_size), device=x.device, dtype=x.dtype)
            db = torch.empty((G,), device=x.device, dtype=x.dtype)
        wws = torch.empty(lib.fastlstm_wgrad_workspace_bytes(seq_len, batch_size, input_size, hidden_size, code),
                          dtype=torch.uint8, device=x.device)
        ptr = lambda t: None if t is None else t.data_ptr()   # (a null pointer: that result is not wanted)
        if PROFILE_RANGES:
            torch.cuda.nvtx.range_pop()
        # reverse time loop + dx + weight gradients in one call (the library fuses them where CUs would idle)
        if PROFILE_RANGES:
            torch.cuda.nvtx.range_push("fastlstm: backward layer launch")
        _lib.check(lib.fastlstm_bwd_layer(dh.data_ptr(), dh_n.data_ptr(), dc_n.data_ptr(), ifgo.data_ptr(),
                                          cell.data_ptr(), d_ifgo.data_ptr(), Wh.data_ptr(), Wx.data_ptr(),
                                          x.data_ptr(), h.data_ptr(), ptr(d_x), ptr(dWx),
                                          ptr(dWh), ptr(db), ws.data_ptr(), ws.numel(),
                                          wws.data_ptr(), wws.numel(), seq_len, batch_size, input_size,
                                          hidden_size, code, stream),
                   "fastlstm_bwd_layer")
        if PROFILE_RANGES:
            torch.cuda.nvtx.range_pop()
        with _Range("fastlstm: status"):
            _check_ws(ws, "fastlstm_bwd_layer")
        dbx = dbh = db   # the same tensor twice, as Wgrad returns it (fastlstm/lstm.py:501)
    return d_x, dh_n, dc_n, dWx, dbx, dWh, dbh


def lstm_persistent_bwd_stack2(dh, x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1,
                               d_state0=None, d_state1=None, need_dx=True):
    """Reverse pass of two stacked layers (suffix 1: upper, 0: lower); dh[T,B,H] is the gradient of
    out1[1:]; d_state0 / d_state1 are optional (dh_n, dc_n) pairs, the gradients flowing into the
    final states of the lower / upper layer (zero when None).  The same results as lstm_persistent_bwd for
    the upper layer followed by lstm_persistent_bwd for the lower layer on the upper layer's d_x;
    one launch for both recurrences where the library can run them side by side.
    Returns ((d_x, dh_0, dc_0, dWx, dbx, dWh, dbh) of the lower layer, the same of the upper layer);
    need_dx=False: the lower layer's d_x is not computed and None."""
    _require_gpu(dh, x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1)
    code = _code(ifgo1)
    T, B, H = dh.shape
    I = Wx0.shape[1]
    lib = _lib.load()
    with torch.cuda.device(x.device):
        plan = _plan(x.device, B, H, code, True)
        n = stack2_wavefront_chunks(T, B, H, ifgo1.dtype, x.device, backward=True)
        if n and lib.fastlstm_bwd_stack2_fused(T, B, I, H, code, lib.fastlstm_stack2_bwd_workspace_bytes(plan, T, H, code)) != 1:
            return _bwd_stack2_wavefront(dh, x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1,
                                         d_state0, d_state1, n, need_dx)
        dh = dh.contiguous()
        if dh.dtype != ifgo1.dtype:
            dh = dh.to(ifgo1.dtype)
        dh, x = _aligned(dh), _aligned(x.contiguous())
        new = lambda *shape: torch.empty(shape, device=x.device, dtype=x.dtype)
        zeros = lambda: torch.zeros((B, H), device=x.device, dtype=x.dtype)
        G = 4 * H
        d_ifgo1, d_ifgo0 = torch.empty_like(ifgo1), torch.empty_like(ifgo0)
        state = lambda d, k: zeros() if d is None else d[k].to(x.dtype).reshape(B, H).clone()
        dh1, dc1, dh0, dc0 = state(d_state1, 0), state(d_state1, 1), state(d_state0, 0), state(d_state0, 1)
        dx1, dx0 = new(T, B, H), (torch.empty_like(x) if need_dx else None)
        dWx1, dWh1, db1 = new(G, H), new(G, H), new(G)
        dWx0, dWh0, db0 = new(G, I), new(G, H), new(G)
        plan = _plan(x.device, B, H, code, True)
        n = lib.fastlstm_stack2_bwd_workspace_bytes(plan, T, H, code)
        ws = torch.empty(n, dtype=torch.uint8, device=x.device)
        ws[:(n if plan.ring_needs_zero else min(n, plan.ws_zero_bytes))].zero_()
        # (large enough for the one launch to take the lower layer's weight gradients too)
        wws = torch.empty(lib.fastlstm_stack2_bwd_wgrad_workspace_bytes(T, B, I, H, code), dtype=torch.uint8, device=x.device)
        p = lambda t: None if t is None else t.data_ptr()
        _lib.check(lib.fastlstm_bwd_stack2(
            p(dh), p(dh1), p(dc1), p(ifgo1), p(cell1), p(d_ifgo1), p(Wh1), p(Wx1), p(out1), p(dWx1), p(dWh1), p(db1), p(dx1),
            p(dh0), p(dc0), p(ifgo0), p(cell0), p(d_ifgo0), p(Wh0), p(Wx0), p(x), p(out0), p(dx0), p(dWx0), p(dWh0), p(db0),
            p(ws), ws.numel(), p(wws), wws.numel(), T, B, I, H, code, _stream()), "fastlstm_bwd_stack2")
        _check_ws(ws, "fastlstm_bwd_stack2")
    return (dx0, dh0, dc0, dWx0, db0, dWh0, db0), (dx1, dh1, dc1, dWx1, db1, dWh1, db1)


def pair_runs_in_one_launch(T, B, H, dtype, device, backward=False):
    """True if two independent recurrences of this shape (the two directions of a bidirectional layer) run as
    one launch (fastlstm_pair_fused)."""
    if dtype not in _DTYPE_CODE or torch.device(device).type != "cuda":
        return False
    lib = _lib.load()
    code = _DTYPE_CODE[dtype]
    with torch.cuda.device(device):
        plan = _plan(torch.device(device), B, H, code, backward)
        n = (lib.fastlstm_stack2_bwd_workspace_bytes if backward else lib.fastlstm_stack2_workspace_bytes)(plan, T, H, code)
        return lib.fastlstm_pair_fused(T, B, H, code, int(backward), n) == 1


def lstm_persistent_fwd_pair(xa, h0a, c0a, Wxa, bxa, Wha, bha, xb, h0b, c0b, Wxb, bxb, Whb, bhb, keep_activations=True):
    """Two independent layers of one shape on their own inputs xa, xb [T,B,I] -- the two directions of a
    bidirectional layer, xb being the time-reversed sequence: returns (out_a, cell_a, ifgo_a, out_b, cell_b,
    ifgo_b) with the layouts and the results of two calls of lstm_persistent_fwd.  The two input projections are
    two GEMM launches; the two time loops are one launch where the library can run them side by side."""
    _require_gpu(xa, xb, Wxa, bxa, Wha, bha, Wxb, bxb, Whb, bhb, h0a, c0a, h0b, c0b)
    code = _code(xa)
    T, B, I = xa.shape
    H = Wha.shape[1]
    assert xb.shape == xa.shape and xb.dtype == xa.dtype and xa.is_contiguous() and xb.is_contiguous()
    assert Wha.is_contiguous() and Whb.is_contiguous()
    assert Wxa.shape == (4 * H, I) and Wxb.shape == (4 * H, I) and Wha.shape == (4 * H, H) and Whb.shape == (4 * H, H)
    for w in (Wxa, bxa, Wha, bha, Wxb, bxb, Whb, bhb):
        if w.dtype != xa.dtype:
            raise TypeError("weights must have the dtype of x (%s), got %s" % (xa.dtype, w.dtype))
    lib = _lib.load()
    with torch.cuda.device(xa.device):
        stream = _stream()
        bufs = []
        for x, h0, c0, Wx, bx, bh in ((xa, h0a, c0a, Wxa, bxa, bha), (xb, h0b, c0b, Wxb, bxb, bhb)):
            x, Wx, bx, bh = _aligned(x), Wx.contiguous(), bx.contiguous(), bh.contiguous()
            ifgo = torch.empty((T, B, 4 * H), device=x.device, dtype=x.dtype)
            out = torch.empty((T + 1, B, H), device=x.device, dtype=x.dtype)
            cell = torch.empty_like(out)
            if h0 is not None:
                out[0] = h0
                cell[0] = c0
            else:
                out[0].zero_()
                cell[0].zero_()
            _lib.check(lib.fastlstm_gemm_ifgo(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), ifgo.data_ptr(),
                                              T, B, I, H, code, stream), "fastlstm_gemm_ifgo")
            bufs.append((out, cell, ifgo))
        (out_a, cell_a, ifgo_a), (out_b, cell_b, ifgo_b) = bufs
        plan = _plan(xa.device, B, H, code, False)
        ws = _stack2_workspace(plan, T, H, code, xa.device)
        p = lambda t: t.data_ptr()
        _lib.check(lib.fastlstm_fwd_persistent_pair(p(ifgo_a), p(out_a), p(cell_a), p(Wha), p(ifgo_b), p(out_b), p(cell_b), p(Whb),
                                                    p(ws), ws.numel(), T, B, H, code, int(keep_activations), stream),
                   "fastlstm_fwd_persistent_pair")
        _check_ws(ws, "fastlstm_fwd_persistent_pair")
    return out_a, cell_a, ifgo_a, out_b, cell_b, ifgo_b


def lstm_persistent_bwd_pair(dh_a, d_state_a, xa, out_a, cell_a, ifgo_a, Wxa, Wha,
                             dh_b, d_state_b, xb, out_b, cell_b, ifgo_b, Wxb, Whb, need_dx=(True, True)):
    """Reverse pass of lstm_persistent_fwd_pair: dh_* [T,B,H] are the gradients of out_*[1:], d_state_* optional
    (dh_n, dc_n) pairs (zero when None).  The two reverse time loops are one launch where the library can run
    them side by side; dx and the weight gradients follow per layer.  The same results as two calls of
    lstm_persistent_bwd.  Returns two tuples (d_x, dh_0, dc_0, dWx, dbx, dWh, dbh); need_dx[k] False: that
    side's d_x is not computed (None)."""
    _require_gpu(dh_a, dh_b, xa, xb, out_a, cell_a, ifgo_a, Wxa, Wha, out_b, cell_b, ifgo_b, Wxb, Whb)
    code = _code(ifgo_a)
    T, B, H = dh_a.shape
    I = Wxa.shape[1]
    lib = _lib.load()
    with torch.cuda.device(xa.device):
        stream = _stream()
        p = lambda t: t.data_ptr()
        sides = []
        for dh, d_state, ifgo in ((dh_a, d_state_a, ifgo_a), (dh_b, d_state_b, ifgo_b)):
            dh = dh.contiguous()
            if dh.dtype != ifgo.dtype:
                dh = dh.to(ifgo.dtype)
            state = lambda k: (torch.zeros((B, H), device=ifgo.device, dtype=ifgo.dtype) if d_state is None
                               else d_state[k].to(ifgo.dtype).reshape(B, H).clone())
            sides.append((_aligned(dh), state(0), state(1), torch.empty_like(ifgo)))
        (dha, dhn_a, dcn_a, d_ifgo_a), (dhb, dhn_b, dcn_b, d_ifgo_b) = sides
        plan = _plan(xa.device, B, H, code, True)
        n = lib.fastlstm_stack2_bwd_workspace_bytes(plan, T, H, code)
        ws = torch.empty(n, dtype=torch.uint8, device=xa.device)
        ws[:(n if plan.ring_needs_zero else min(n, plan.ws_zero_bytes))].zero_()
        _lib.check(lib.fastlstm_bwd_persistent_pair(
            p(dha), p(dhn_a), p(dcn_a), p(ifgo_a), p(cell_a), p(d_ifgo_a), p(Wha),
            p(dhb), p(dhn_b), p(dcn_b), p(ifgo_b), p(cell_b), p(d_ifgo_b), p(Whb),
            p(ws), ws.numel(), T, B, H, code, stream), "fastlstm_bwd_persistent_pair")
        _check_ws(ws, "fastlstm_bwd_persistent_pair")
        res = []
        for x, out, d_ifgo, Wx, dhn, dcn, want in ((xa, out_a, d_ifgo_a, Wxa, dhn_a, dcn_a, need_dx[0]),
                                                   (xb, out_b, d_ifgo_b, Wxb, dhn_b, dcn_b, need_dx[1])):
            d_x, dbx, dbh, dWx, dWh = DxWgrad(d_ifgo, Wx, x, out, want)
            res.append((d_x, dhn, dcn, dWx, dbx, dWh, dbh))
    return res[0], res[1]


def _autocast_operands(*tensors):
    """x and the parameters in the autocast dtype when autocast is on (fastlstm/lstm.py:509-515;
    the initial states are not cast)."""
    if torch.is_autocast_enabled():
        target = torch.get_autocast_dtype("cuda")
        return tuple(t.to(target) for t in tensors)
    return tensors


class PersistentLSTMfn(torch.autograd.Function):
    """apply(x, h_0|None, c_0|None, Wx[4H,I], bx[4H], Wh[4H,H], bh[4H]) ->
    (out[T,B,H], (h_T[B,H], c_T[B,H])).  The nested tuple makes h_T/c_T
    non-differentiable, as in the reference (fastlstm/lstm.py:504-538)."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, x, h_0, c_0, Wx, bx, Wh, bh):
        x, Wx, bx, Wh, bh = _autocast_operands(x, Wx, bx, Wh, bh)
        out, cell, ifgo = lstm_persistent_fwd(x, h_0, c_0, Wx, bx, Wh, bh)
        ctx.h0_is_nan = h_0 is None
        if x.dim() == 2:
            x = x[None]
        ctx.save_for_backward(x, out, cell, ifgo, Wx, Wh)
        # first one is initial condition
        return out[1:], (out[-1], cell[-1])

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, dh, d_out_cell):
        _raise_pending_before_backward(dh)   # a failed forward launch is reported before its gradients are computed
        x, out, cell, ifgo, Wx, Wh = ctx.saved_tensors
        if d_out_cell is not None:
            raise ValueError("Not implemented")  # fastlstm/lstm.py:528-531
        need = ctx.needs_input_grad   # (x, h_0, c_0, Wx, bx, Wh, bh)
        # (no gradient into the final state: the reference passes two zeros_like, fastlstm/lstm.py:524-527)
        d_x, dh_0, dc_0, dWx, dbx, dWh, dbh = lstm_persistent_bwd(
            dh, None, None, x, out, cell, ifgo, Wx, Wh, need_dx=need[0], need_dw=any(need[3:7])
        )
        if ctx.h0_is_nan:
            dh_0 = None
            dc_0 = None
        return d_x, dh_0, dc_0, dWx, dbx, dWh, dbh


class PersistentLSTMStatefn(torch.autograd.Function):
    """PersistentLSTMfn with differentiable final states: apply(...) -> (out[T,B,H], h_T[B,H], c_T[B,H]),
    a flat tuple, so gradients with respect to h_T and c_T reach the reverse kernel as its dh_n / dc_n
    operands (the reference raises ValueError there, fastlstm/lstm.py:528-531, and its nested tuple
    never delivers them).  This is what carrying a state across segments and training through it needs."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, x, h_0, c_0, Wx, bx, Wh, bh):
        x, Wx, bx, Wh, bh = _autocast_operands(x, Wx, bx, Wh, bh)
        out, cell, ifgo = lstm_persistent_fwd(x, h_0, c_0, Wx, bx, Wh, bh)
        ctx.no_state = h_0 is None
        if x.dim() == 2:
            x = x[None]
        ctx.save_for_backward(x, out, cell, ifgo, Wx, Wh)
        return out[1:], out[-1].clone(), cell[-1].clone()

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, dh, dh_n, dc_n):
        _raise_pending_before_backward(dh)   # a failed forward launch is reported before its gradients are computed
        x, out, cell, ifgo, Wx, Wh = ctx.saved_tensors
        # the kernel overwrites its state operands with the gradients of the initial state
        dh_n = dh_n.to(cell.dtype).contiguous().clone()
        dc_n = dc_n.to(cell.dtype).contiguous().clone()
        need = ctx.needs_input_grad
        d_x, dh_0, dc_0, dWx, dbx, dWh, dbh = lstm_persistent_bwd(dh, dc_n, dh_n, x, out, cell, ifgo, Wx, Wh,
                                                                 need_dx=need[0], need_dw=any(need[3:7]))
        if ctx.no_state:
            dh_0 = dc_0 = None
        return d_x, dh_0, dc_0, dWx, dbx, dWh, dbh


class PersistentLSTMHistoryfn(torch.autograd.Function):
    """apply(...) -> (out[T,B,H], cell[T,B,H]): the layer with its whole cell-state history as a second,
    non-differentiable result.  Sequences of different lengths padded to one T read their final states
    out of the two histories (row b at step len_b - 1); a gradient reaches h_n through out."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, x, h_0, c_0, Wx, bx, Wh, bh):
        x, Wx, bx, Wh, bh = _autocast_operands(x, Wx, bx, Wh, bh)
        out, cell, ifgo = lstm_persistent_fwd(x, h_0, c_0, Wx, bx, Wh, bh)
        ctx.no_state = h_0 is None
        ctx.save_for_backward(x, out, cell, ifgo, Wx, Wh)
        history = cell[1:]
        ctx.mark_non_differentiable(history)
        return out[1:], history

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, dh, _):
        _raise_pending_before_backward(dh)   # a failed forward launch is reported before its gradients are computed
        x, out, cell, ifgo, Wx, Wh = ctx.saved_tensors
        need = ctx.needs_input_grad
        d_x, dh_0, dc_0, dWx, dbx, dWh, dbh = lstm_persistent_bwd(
            dh, torch.zeros_like(cell[0]), torch.zeros_like(cell[0]), x, out, cell, ifgo, Wx, Wh,
            need_dx=need[0], need_dw=any(need[3:7]))
        if ctx.no_state:
            dh_0 = dc_0 = None
        return d_x, dh_0, dc_0, dWx, dbx, dWh, dbh


class PersistentLSTMPairfn(torch.autograd.Function):
    """Two independent layers of one shape as one autograd node (the two directions of a bidirectional layer):
    forward through lstm_persistent_fwd_pair, backward through lstm_persistent_bwd_pair, one launch for both time
    loops each way where the shapes allow.  apply(xa, h0a, c0a, Wxa, bxa, Wha, bha, xb, h0b, c0b, Wxb, bxb, Whb,
    bhb, state_grads) -> (out_a, h_Ta, c_Ta, out_b, h_Tb, c_Tb, cells_a, cells_b); the final states carry a gradient
    only with state_grads (as PersistentLSTMStatefn), else none (as PersistentLSTMfn); cells_* [T,B,H] are the
    cell-state histories, non-differentiable (as PersistentLSTMHistoryfn's)."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, xa, h0a, c0a, Wxa, bxa, Wha, bha, xb, h0b, c0b, Wxb, bxb, Whb, bhb, state_grads):
        xa, Wxa, bxa, Wha, bha, xb, Wxb, bxb, Whb, bhb = _autocast_operands(xa, Wxa, bxa, Wha, bha, xb, Wxb, bxb, Whb, bhb)
        out_a, cell_a, ifgo_a, out_b, cell_b, ifgo_b = lstm_persistent_fwd_pair(xa, h0a, c0a, Wxa, bxa, Wha, bha,
                                                                                xb, h0b, c0b, Wxb, bxb, Whb, bhb)
        ctx.no_state = (h0a is None, h0b is None)
        ctx.save_for_backward(xa, out_a, cell_a, ifgo_a, Wxa, Wha, xb, out_b, cell_b, ifgo_b, Wxb, Whb)
        finals = (out_a[-1].clone(), cell_a[-1].clone(), out_b[-1].clone(), cell_b[-1].clone())
        histories = (cell_a[1:], cell_b[1:])
        ctx.mark_non_differentiable(*histories, *(() if state_grads else finals))
        return out_a[1:], finals[0], finals[1], out_b[1:], finals[2], finals[3], histories[0], histories[1]

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, dh_a, dhn_a, dcn_a, dh_b, dhn_b, dcn_b, _ha, _hb):
        _raise_pending_before_backward(dh_a)   # a failed forward launch is reported before its gradients are computed
        xa, out_a, cell_a, ifgo_a, Wxa, Wha, xb, out_b, cell_b, ifgo_b, Wxb, Whb = ctx.saved_tensors
        pair = lambda h, c: None if h is None and c is None else (
            torch.zeros_like(cell_a[0]) if h is None else h, torch.zeros_like(cell_a[0]) if c is None else c)
        ga, gb = lstm_persistent_bwd_pair(dh_a, pair(dhn_a, dcn_a), xa, out_a, cell_a, ifgo_a, Wxa, Wha,
                                          dh_b, pair(dhn_b, dcn_b), xb, out_b, cell_b, ifgo_b, Wxb, Whb,
                                          need_dx=(ctx.needs_input_grad[0], ctx.needs_input_grad[7]))
        ga, gb = list(ga), list(gb)
        if ctx.no_state[0]:
            ga[1] = ga[2] = None
        if ctx.no_state[1]:
            gb[1] = gb[2] = None
        return (*ga, *gb, None)


class PersistentLSTMStackfn(torch.autograd.Function):
    """L = 2 ... 4 stacked layers as one autograd node, run as a wavefront of chunked launches
    (lstm_persistent_fwd_stack / lstm_persistent_bwd_stack).  apply(x, state_grads, L, *flat) with flat = (h_0, c_0,
    Wx, bx, Wh, bh) per layer -> (out of the top layer, h_T, c_T of layer 0, h_T, c_T of layer 1, ...); the final
    states carry a gradient only with state_grads."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, x, state_grads, L, *flat):
        layers = []
        for l in range(L):
            h0, c0, Wx, bx, Wh, bh = flat[6 * l:6 * l + 6]
            layers.append((h0, c0) + tuple(_autocast_operands(Wx, bx, Wh, bh)))
        (x,) = _autocast_operands(x)
        if x.dim() == 2:
            x = x[None]
        acts = lstm_persistent_fwd_stack(x, layers)
        ctx.L = L
        ctx.no_state = [l[0] is None for l in layers]
        saved = [x]
        for (out, cell, ifgo), (_, _, Wx, _, Wh, _) in zip(acts, layers):
            saved += [out, cell, ifgo, Wx, Wh]
        ctx.save_for_backward(*saved)
        finals = []
        for out, cell, _ in acts:
            finals += [out[-1].clone(), cell[-1].clone()]
        if not state_grads:
            ctx.mark_non_differentiable(*finals)
        return (acts[-1][0][1:], *finals)

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, dh, *d_finals):
        _raise_pending_before_backward(dh)   # a failed forward launch is reported before its gradients are computed
        L = ctx.L
        x, rest = ctx.saved_tensors[0], ctx.saved_tensors[1:]
        acts = [tuple(rest[5 * l:5 * l + 3]) for l in range(L)]
        weights = [tuple(rest[5 * l + 3:5 * l + 5]) for l in range(L)]
        zero = lambda: torch.zeros_like(acts[0][1][0])
        d_states = []
        for l in range(L):
            h, c = d_finals[2 * l], d_finals[2 * l + 1]
            d_states.append(None if h is None and c is None else (zero() if h is None else h, zero() if c is None else c))
        res = lstm_persistent_bwd_stack(dh, x, acts, weights, d_states, need_dx=ctx.needs_input_grad[0])
        grads = [res[0][0], None, None]
        for l in range(L):
            _, dh0, dc0, dWx, dbx, dWh, dbh = res[l]
            if ctx.no_state[l]:
                dh0 = dc0 = None
            grads += [dh0, dc0, dWx, dbx, dWh, dbh]
        return tuple(grads)


class PersistentLSTMStack2fn(torch.autograd.Function):
    """Two stacked layers as one autograd node: forward through lstm_persistent_fwd_stack2, backward
    through lstm_persistent_bwd_stack2 (one launch each where the shapes allow).  Same
    results and the same contract as two PersistentLSTMfn nodes in a row (fastlstm/lstm.py:685-696):
    returns out[T,B,H] of the second layer and the (h_T, c_T) pairs of both layers, which carry no
    gradient; with state_grads=True the result is the flat tuple (out, h_T0, c_T0, h_T1, c_T1) and
    the final states are differentiable, as with PersistentLSTMStatefn."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, x, h0a, c0a, Wx0, bx0, Wh0, bh0, h0b, c0b, Wx1, bx1, Wh1, bh1, state_grads):
        x, Wx0, bx0, Wh0, bh0, Wx1, bx1, Wh1, bh1 = _autocast_operands(x, Wx0, bx0, Wh0, bh0, Wx1, bx1, Wh1, bh1)
        out0, cell0, ifgo0, out1, cell1, ifgo1 = lstm_persistent_fwd_stack2(x, h0a, c0a, Wx0, bx0, Wh0, bh0, h0b, c0b,
                                                                            Wx1, bx1, Wh1, bh1)
        ctx.no_state = (h0a is None, h0b is None)
        if x.dim() == 2:
            x = x[None]
        ctx.save_for_backward(x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1)
        if state_grads:
            return out1[1:], out0[-1].clone(), cell0[-1].clone(), out1[-1].clone(), cell1[-1].clone()
        return out1[1:], (out0[-1], cell0[-1]), (out1[-1], cell1[-1])

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, dh, *d_states):
        _raise_pending_before_backward(dh)   # a failed forward launch is reported before its gradients are computed
        x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1 = ctx.saved_tensors
        d_state0 = d_state1 = None
        if len(d_states) == 4:
            d_state0, d_state1 = d_states[:2], d_states[2:]
        elif any(d is not None for d in d_states):
            raise ValueError("Not implemented")  # fastlstm/lstm.py:528-531
        (d_x, dh0a, dc0a, dWx0, dbx0, dWh0, dbh0), (_, dh0b, dc0b, dWx1, dbx1, dWh1, dbh1) = lstm_persistent_bwd_stack2(
            dh, x, out0, cell0, ifgo0, Wx0, Wh0, out1, cell1, ifgo1, Wx1, Wh1, d_state0, d_state1,
            need_dx=ctx.needs_input_grad[0])
        if ctx.no_state[0]:
            dh0a = dc0a = None
        if ctx.no_state[1]:
            dh0b = dc0b = None
        return d_x, dh0a, dc0a, dWx0, dbx0, dWh0, dbh0, dh0b, dc0b, dWx1, dbx1, dWh1, dbh1, None


_staging = threading.local()


def _indices_to_device(dev, *tensors):
    """int64 CPU tensors -> `dev` in one asynchronous copy through a pinned staging buffer kept per thread and
    device (a pageable copy would stall the host until the stream has drained, and a fresh pinned allocation per
    call costs milliseconds).  The buffer is reused only after the previous call's copy has run."""
    if dev.type != "cuda":
        return tuple(t.to(dev) for t in tensors)
    n = sum(t.numel() for t in tensors)
    stages = _staging.__dict__.setdefault("by_device", {})
    with torch.cuda.device(dev):
        key = torch.cuda.current_device()
        stage = stages.get(key)
        if stage is not None:
            stage[1].synchronize()
        if stage is None or stage[0].numel() < n:
            stage = stages[key] = [torch.empty(max(n, 1 << 16), dtype=torch.int64).pin_memory(), None]
        torch.cat([t.flatten() for t in tensors], out=stage[0][:n])
        on_dev = stage[0][:n].to(dev, non_blocking=True)
        stage[1] = torch.cuda.Event()
        stage[1].record()
    return on_dev.split([t.numel() for t in tensors])


def _recurrent_kind(T, B, H, code, device_index, backward=False):
    """fastlstm_recurrent_kernel_kind of the forward (reverse) call for the workspace this module allocates."""
    return _recurrent_kind_cached(T, B, H, code, device_index, backward, _families())


@functools.lru_cache(maxsize=4096)
def _recurrent_kind_cached(T, B, H, code, device_index, backward, families):
    lib = _lib.load()
    device = torch.device("cuda", device_index)
    with torch.cuda.device(device):
        plan = _plan(device, B, H, code, backward)
        b = int(backward)
        return lib.fastlstm_recurrent_kernel_kind(T, B, H, code, b, lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, b))


def _padded_hidden_size(T, B, H, code, device_index, training=False):
    return _padded_hidden_size_cached(T, B, H, code, device_index, training, _families())


@functools.lru_cache(maxsize=4096)
def _padded_hidden_size_cached(T, B, H, code, device_index, training, families):
    """The next hidden size above H (within a quarter, in steps of the MFMA k-step) that the XCD-local or the
    register-resident kernels take, when H itself gets the general kernels; else 0.  `training`: a reverse pass
    follows, whose kernels count too."""
    fp32 = code == _DTYPE_CODE[torch.float32]
    kind = lambda h: _recurrent_kind(T, B, h, code, device_index)
    # fp32 with up to 32 rows keeps the general forward kernel at H = 640 ... 1024, but its reverse pass is twice as
    # fast on the register-resident kernel (T = 256, B = 8, I = 256, forward + backward: H = 576 3.8 ms, H = 640 2.9)
    fast = lambda h: kind(h) in (1, 2) or (training and fp32 and _recurrent_kind(T, B, h, code, device_index, True) in (1, 2))
    # The launches that pad and cut cost ~0.1 ms forward and ~0.2 ms forward + backward whatever the shape: a few steps
    # repay them only with many rows and units (T = 16, B = 128, H = 1150 bf16 forward + backward 0.82 ms as it is,
    # 0.59 ms as 1280; B = 64, H = 650 0.48 against 0.68).
    if T < 32 and (H <= 64 or T * B * H < (1_200_000 if fp32 else 2_000_000)):
        return 0
    if H <= 64:
        # The general kernels' one-tile form (no exchange between workgroups at all).  In 16 bits it is the fastest
        # there is at H = 64 (T = 1024, B = 256, I = H = 64 forward + backward 0.93 ms as it is, 3.4 ms as H = 96):
        # its 64-unit kernels spread the batch over tiles of 4 rows and move whole tiles in both directions, which the
        # narrower forms do not (T = 1024, B = 256, inference forward / forward + backward of a training step with its
        # loss: H = 32 as it is 0.50 / 3.20 ms, H = 16 0.42 / 2.12, H = 64 0.42 / 1.18).  The same holds in fp32 since
        # the 4-row tiles spread its true-fp32 MFMAs over four times the CUs (T = 256, B = 64: H = 64 as it is 0.36 /
        # 0.86 ms, as H = 80 on the XCD-local kernels 0.57 / 1.21; H = 48 as it is 0.74 / 2.40, as 64 0.45 / 0.98), except
        # that up to 16 units nothing gains (H = 16 0.18 / 1.03 as it is, 0.45 / 0.99 as 64) and up to 32 only a
        # training step does (H = 32 0.28 / 1.16 as it is, 0.45 / 0.98 as 64).
        if H == 64 or H <= (16 if fp32 or not training else 0):
            return 0
        if fp32 and H <= 32 and not training:
            return 0
        return 64
    if kind(H) != 0 or fast(H):
        return 0
    step = 16 if fp32 else 32
    for Hp in range((H // step + 1) * step, H + H // 4 + step + 1, step):
        if fast(Hp):
            return Hp
    return 0


class _GatherRows(torch.autograd.Function):
    """src[take]; the gradient of src is the rows `back` of the result's gradient -- for a gather in which every
    row of src has one slot that counts (back[p]) and the other slots' gradients are zero by construction."""

    @staticmethod
    def forward(ctx, src, take, back):
        ctx.save_for_backward(back)
        return src.index_select(0, take)

    @staticmethod
    def backward(ctx, g):
        back, = ctx.saved_tensors
        return g.index_select(0, back), None, None


class _TakeRows(torch.autograd.Function):
    """src[idx] for distinct idx; the gradient is scattered back without atomics."""

    @staticmethod
    def forward(ctx, src, idx):
        ctx.save_for_backward(idx)
        ctx.n = src.shape[0]
        return src.index_select(0, idx)

    @staticmethod
    def backward(ctx, g):
        idx, = ctx.saved_tensors
        return g.new_zeros(ctx.n, g.shape[1]).index_copy(0, idx, g), None


class FastLSTM(nn.Module):
    """nn.LSTM-compatible parameters (names, shapes, order, seeded values) and the
    reference's forward contract (fastlstm/lstm.py:586-698): sequence-first input
    x[T,B,I], optional (h_0[L,B,H], c_0[L,B,H]); returns out[T,B,H], (h_n, c_n).

    Keyword-only additions with nn.LSTM's meaning, all off by default so that the defaults are the
    reference's module (which lists them as unsupported, README.md:92-93): bias=False (no bias
    parameters), batch_first=True (x and out are [B,T,*]), bidirectional=True (a second set of
    `*_reverse` parameters runs the same kernels over the time-reversed sequence; out is [T,B,2H]
    and the states are [2L,B,H] in nn.LSTM's order).  state_grads=True makes h_n and c_n
    differentiable (PersistentLSTMStatefn).  A PackedSequence input gives a PackedSequence output and the
    states at each row's own last step, as nn.LSTM does."""

    def __init__(self, input_size, hidden_size, num_layers=1, version="persistent", device=None,
                 dtype=None, *, bias=True, batch_first=False, bidirectional=False, state_grads=False, dropout=0.0):
        super().__init__()
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.num_layers = num_layers
        self.version = version
        self.device = device
        self.dtype = dtype
        self.bias = bias
        self.batch_first = batch_first
        self.bidirectional = bidirectional
        self.state_grads = state_grads
        if not 0.0 <= dropout < 1.0:
            raise ValueError("dropout should be a number in [0, 1), got %r" % (dropout,))
        self.dropout = float(dropout)   # nn.LSTM's: on the outputs of every layer but the last, in training mode
        sqrt_k_inv = 1 / hidden_size**0.5
        directions = 2 if bidirectional else 1
        # same RNG consumption order as nn.LSTM: w_ih, w_hh, b_ih, b_hh per layer and direction
        for layer in range(num_layers):
            for suffix in ("", "_reverse")[:directions]:
                shapes = [
                    ("weight_ih_l%d%s" % (layer, suffix),
                     (4 * hidden_size, input_size if layer == 0 else hidden_size * directions)),
                    ("weight_hh_l%d%s" % (layer, suffix), (4 * hidden_size, hidden_size)),
                ]
                if bias:
                    shapes += [("bias_ih_l%d%s" % (layer, suffix), (4 * hidden_size,)),
                               ("bias_hh_l%d%s" % (layer, suffix), (4 * hidden_size,))]
                for name, shape in shapes:
                    value = torch.rand(*shape, device=device, dtype=dtype) * 2 * sqrt_k_inv - sqrt_k_inv
                    setattr(self, name, nn.Parameter(value))

    def _two_layers_at_once(self, x):
        """Two stacked layers of this input's shape run overlapped: as one launch of the library, or as a wavefront
        of chunked launches (stack2_wavefront_chunks)."""
        dt = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else x.dtype
        T, B, I = x.shape
        return (stack2_runs_in_one_launch(T, B, I, self.hidden_size, dt, x.device)
                or stack2_wavefront_chunks(T, B, self.hidden_size, dt, x.device) > 0)

    def _layer_operands(self, layer, suffix=""):
        """(Wx, bx, Wh, bh) of one layer and direction; zero biases when the module has none."""
        Wx = getattr(self, f"weight_ih_l{layer}{suffix}")
        Wh = getattr(self, f"weight_hh_l{layer}{suffix}")
        if self.bias:
            return Wx, getattr(self, f"bias_ih_l{layer}{suffix}"), Wh, getattr(self, f"bias_hh_l{layer}{suffix}")
        zero = torch.zeros(4 * self.hidden_size, device=Wx.device, dtype=Wx.dtype)
        return Wx, zero, Wh, zero

    def _forward_packed(self, packed, h_0, c_0):
        """PackedSequence input, nn.LSTM's contract: the sequences are padded to the longest, every layer
        runs over the padded batch (a row's steps behind its own end change nothing before it), the
        reverse direction runs over each row reversed within its own length, and the final states are
        row b's out / cell at step len_b - 1.  The result is packed like the input.

        The padded batch keeps the packed order (rows sorted by length, longest first) and is made with ONE
        gather, the packed result with one more (pad_packed_sequence / pack_padded_sequence copy timestep by
        timestep, T launches each); slots behind a row's end hold some other row's data instead of zeros --
        nothing reads what is computed from them, and their gradients are exactly zero.

        A batch that the library runs as several launches over ranges of rows (more batch tiles than one
        launch holds) is cut at those ranges here, and every range runs only to its own longest sequence: the
        steps and GEMM rows behind it are not computed."""
        from torch.nn.utils.rnn import PackedSequence
        data, sizes = packed.data, packed.batch_sizes            # sizes [T] on the CPU: rows alive at step t
        dev, N = data.device, data.shape[0]
        T, B = int(sizes.numel()), int(sizes[0])
        alive = sizes[:, None] > torch.arange(B)[None, :]        # [T,B]
        lengths = alive.sum(0)                                   # per row, descending
        offs = torch.cumsum(sizes, 0) - sizes                    # first packed row of step t
        rows = self._packed_range_rows(T, B, lengths, data)
        ranges = [(r0, min(B, r0 + rows), int(lengths[r0])) for r0 in range(0, B, rows)] if rows else [(0, B, T)]
        # slot (t, j) of range r = row base_r + t*n_r + j of the ranges' padded tensors laid end to end
        at = torch.zeros(T, B, dtype=torch.int64)
        takes, base = [], 0
        for r0, r1, Tr in ranges:
            j = torch.arange(r0, r1)[None, :]
            slot = base + torch.arange(Tr)[:, None] * (r1 - r0) + (j - r0)
            takes.append(torch.where(j < sizes[:Tr, None], offs[:Tr, None] + j, slot % N).flatten())
            at[:Tr, r0:r1] = slot
            base += Tr * (r1 - r0)
        take, at_packed, lengths_dev = _indices_to_device(dev, torch.cat(takes), at.flatten()[alive.flatten()], lengths)
        x_all = _GatherRows.apply(data, take, at_packed)         # [sum Tr*n_r, I]
        order = packed.sorted_indices
        if order is not None:   # the states come in the caller's batch order
            h_0 = [h if h is None else h.index_select(0, order) for h in h_0]
            c_0 = [c if c is None else c.index_select(0, order) for c in c_0]
        pieces, hs, cs, base = [], [], [], 0
        for r0, r1, Tr in ranges:
            n = Tr * (r1 - r0)
            y, h_r, c_r = self._run_padded(x_all[base:base + n].view(Tr, r1 - r0, -1), lengths_dev[r0:r1],
                                           [h if h is None else h[r0:r1] for h in h_0],
                                           [c if c is None else c[r0:r1] for c in c_0])
            pieces.append(y.reshape(n, -1))
            hs.append(torch.stack(h_r))
            cs.append(torch.stack(c_r))
            base += n
        y_all = pieces[0] if len(pieces) == 1 else torch.cat(pieces, dim=0)
        h_n, c_n = (hs[0], cs[0]) if len(hs) == 1 else (torch.cat(hs, dim=1), torch.cat(cs, dim=1))
        out = PackedSequence(_TakeRows.apply(y_all, at_packed), packed.batch_sizes, packed.sorted_indices,
                             packed.unsorted_indices)
        if packed.unsorted_indices is not None:
            h_n, c_n = h_n.index_select(1, packed.unsorted_indices), c_n.index_select(1, packed.unsorted_indices)
        return out, (h_n, c_n)

    def _packed_range_rows(self, T, B, lengths, data):
        """Rows per range for a packed batch of B rows sorted by length (descending, lengths on the CPU): the rows
        the library takes per launch where it runs this batch as several launches
        (fastlstm_recurrent_rows_per_launch) and cutting there saves at least an eighth of the steps; else 0."""
        dt = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else data.dtype
        if not data.is_cuda or dt not in _DTYPE_CODE or B < 32:
            return 0
        lib = _lib.load()
        code, H = _DTYPE_CODE[dt], self.hidden_size
        with torch.cuda.device(data.device):
            plan = _plan(data.device, B, H, code, False)
            rows = lib.fastlstm_recurrent_rows_per_launch(T, B, H, code, 0,
                                                          lib.fastlstm_recurrent_workspace_bytes(plan, T, H, code, 0))
        if rows <= 0 or rows >= B:
            return 0
        saved = sum((T - int(lengths[r0])) * (min(B, r0 + rows) - r0) for r0 in range(0, B, rows))
        return rows if saved * 8 >= T * B else 0

    def _run_padded(self, x, lengths_dev, h_0, c_0):
        """All layers over a padded batch x [T,B,I] with T = max(lengths); lengths_dev [B] on x's device; h_0, c_0:
        per layer and direction [B,H] or None.  Returns (y [T,B,D*H], [h_n per layer and direction], [c_n ...])
        with the final states taken at each row's own last step."""
        T, B = x.shape[0], x.shape[1]
        directions = 2 if self.bidirectional else 1
        steps = torch.arange(T, device=x.device)[:, None]
        last = (lengths_dev - 1)[None, :, None]                   # [1,B,1] index of a row's last step
        # time index that reverses row b within its length and leaves its padding in place
        flip = torch.where(steps < lengths_dev[None, :], lengths_dev[None, :] - 1 - steps, steps)[:, :, None]
        h_n, c_n = [], []
        H = self.hidden_size
        for layer in range(self.num_layers):
            ys = []
            xs = [x.contiguous()] + ([x.gather(0, flip.expand(T, B, x.shape[2]))] if directions == 2 else [])
            k = layer * directions
            if directions == 2 and pair_runs_in_one_launch(
                    T, B, H, torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else x.dtype, x.device):
                # both directions' time loops in one launch
                y_a, _, _, y_b, _, _, cells_a, cells_b = PersistentLSTMPairfn.apply(
                    xs[0], h_0[k], c_0[k], *self._layer_operands(layer),
                    xs[1], h_0[k + 1], c_0[k + 1], *self._layer_operands(layer, "_reverse"), False)
                results = [(y_a, cells_a), (y_b, cells_b)]
            else:
                results = [PersistentLSTMHistoryfn.apply(xs[d], h_0[k + d], c_0[k + d], *self._layer_operands(layer, suffix))
                           for d, suffix in enumerate(("", "_reverse")[:directions])]
            for d, (y, cells) in enumerate(results):
                h_n.append(y.gather(0, last.expand(1, B, H))[0])
                c_n.append(cells.gather(0, last.expand(1, B, H))[0])
                ys.append(y if d == 0 else y.gather(0, flip.expand(T, B, H)))
            x = ys[0] if directions == 1 else torch.cat(ys, dim=-1)
            if self.training and self.dropout > 0.0 and layer + 1 < self.num_layers:
                x = F.dropout(x, self.dropout, True)
        return x, h_n, c_n

    def forward(self, x, h_c_0=None):
        directions = 2 if self.bidirectional else 1
        if h_c_0 is None:
            h_0, c_0 = [None] * (self.num_layers * directions), [None] * (self.num_layers * directions)
        else:
            h_0, c_0 = h_c_0
        if self.version != "persistent":
            # the reference also offers "graph", "naive-pt" and "v1"; this build has one path
            raise ValueError(f"Not Implemnted: {self.version}")
        data = x.data if isinstance(x, nn.utils.rnn.PackedSequence) else x
        if data.is_cuda and not torch.cuda.is_current_stream_capturing():
            _raise_pending(data.device)   # a failed earlier launch is reported before new work goes behind it
        padding = self._operand_padding(x)
        if padding:
            return self._forward_operands_padded(x, h_c_0, *padding)
        if isinstance(x, nn.utils.rnn.PackedSequence):
            return self._forward_packed(x, h_0, c_0)
        if self.batch_first and x.dim() == 3:
            x = x.transpose(0, 1).contiguous()
        # no backward pass can follow (grad mode off, or nothing that enters requires a gradient): the
        # kernels skip the stores only the reverse pass reads; the outputs are the same bits
        tensors = [x] + [p for p in self.parameters()] + [t for t in list(h_0) + list(c_0) if t is not None]
        inference = not (torch.is_grad_enabled() and any(t.requires_grad for t in tensors))
        if inference:
            def fn(xi, h_i, c_i, Wx, bx, Wh, bh):
                xi, Wx, bx, Wh, bh = _autocast_operands(xi, Wx, bx, Wh, bh)
                out, cell, _ = lstm_persistent_fwd(xi, h_i, c_i, Wx, bx, Wh, bh, keep_activations=False)
                return out[1:], (out[-1], cell[-1])
        elif self.state_grads:
            def fn(*operands):
                out, h_i, c_i = PersistentLSTMStatefn.apply(*operands)
                return out, (h_i, c_i)
        else:
            fn = PersistentLSTMfn.apply
        h_n, c_n = [], []
        layer = 0
        drop = self.dropout if self.training else 0.0

        def between(y, done):   # dropout on what the next layer reads
            return F.dropout(y, drop, True) if drop > 0.0 and done < self.num_layers else y

        while layer < self.num_layers:
            # three or four layers at a time as a wavefront of chunked launches where their time loops fit the
            # device side by side
            width = min(self.num_layers - layer, 4)
            if directions == 1 and drop == 0.0 and width >= 3 and x.dim() == 3 and x.is_cuda:
                dt_ = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else x.dtype
                while width >= 3 and not stack_wavefront_chunks(width, x.shape[0], x.shape[1], self.hidden_size, dt_, x.device):
                    width -= 1
                # (the reverse pass of such a block chooses by itself between one wavefront and the library's two-layer
                # launches, lstm_persistent_bwd_stack)
                if width >= 3:
                    flat = []
                    for l in range(layer, layer + width):
                        flat += [h_0[l], c_0[l], *self._layer_operands(l)]
                    if inference:
                        xi, = _autocast_operands(x.contiguous())
                        ls = [(flat[6 * i], flat[6 * i + 1]) + tuple(_autocast_operands(*flat[6 * i + 2:6 * i + 6])) for i in range(width)]
                        acts = lstm_persistent_fwd_stack(xi, ls, keep_activations=False)
                        x = acts[-1][0][1:]
                        h_n += [a[0][-1] for a in acts]
                        c_n += [a[1][-1] for a in acts]
                    else:
                        x, *finals = PersistentLSTMStackfn.apply(x.contiguous(), self.state_grads, width, *flat)
                        h_n += finals[0::2]
                        c_n += finals[1::2]
                    layer += width
                    continue
            # two layers at a time where the library runs them as one launch (the second layer's
            # recurrence a chunk of timesteps behind the first); the results do not depend on it
            if (directions == 1 and drop == 0.0 and layer + 1 < self.num_layers and x.dim() == 3 and x.is_cuda
                    and self._two_layers_at_once(x)):
                w = self._layer_operands(layer) + self._layer_operands(layer + 1)
                if inference:
                    xi, *wc = _autocast_operands(x, *w)
                    out0, cell0, _, out1, cell1, _ = lstm_persistent_fwd_stack2(
                        xi, h_0[layer], c_0[layer], *wc[:4], h_0[layer + 1], c_0[layer + 1], *wc[4:],
                        keep_activations=False)
                    x = out1[1:]
                    h_n += [out0[-1], out1[-1]]
                    c_n += [cell0[-1], cell1[-1]]
                    layer += 2
                    continue
                res = PersistentLSTMStack2fn.apply(
                    x, h_0[layer], c_0[layer], *w[:4], h_0[layer + 1], c_0[layer + 1], *w[4:], self.state_grads)
                if self.state_grads:
                    x, h_a, c_a, h_b, c_b = res
                else:
                    x, (h_a, c_a), (h_b, c_b) = res
                h_n += [h_a, h_b]
                c_n += [c_a, c_b]
                layer += 2
                continue
            k = layer * directions
            if (directions == 2 and x.dim() == 3 and x.is_cuda and pair_runs_in_one_launch(
                    x.shape[0], x.shape[1], self.hidden_size,
                    torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else x.dtype, x.device)):
                # both directions' time loops in one launch (the reverse direction: the same kernels over the
                # time-reversed sequence; its final state belongs to t = 0)
                wa, wb = self._layer_operands(layer), self._layer_operands(layer, "_reverse")
                if inference:
                    xa, *wa = _autocast_operands(x.contiguous(), *wa)
                    xb, *wb = _autocast_operands(x.flip(0), *wb)
                    oa, ca, _, ob, cb, _ = lstm_persistent_fwd_pair(xa, h_0[k], c_0[k], *wa, xb, h_0[k + 1], c_0[k + 1], *wb,
                                                                    keep_activations=False)
                    y, h_i, c_i, y_r, h_r, c_r = oa[1:], oa[-1], ca[-1], ob[1:], ob[-1], cb[-1]
                else:
                    y, h_i, c_i, y_r, h_r, c_r, _, _ = PersistentLSTMPairfn.apply(
                        x.contiguous(), h_0[k], c_0[k], *wa, x.flip(0), h_0[k + 1], c_0[k + 1], *wb, self.state_grads)
                x = between(torch.cat((y, y_r.flip(0)), dim=-1), layer + 1)
                h_n += [h_i, h_r]
                c_n += [c_i, c_r]
                layer += 1
                continue
            y, (h_i, c_i) = fn(x, h_0[k], c_0[k], *self._layer_operands(layer))
            h_n += [h_i]
            c_n += [c_i]
            if directions == 2:
                # the same kernels over the time-reversed sequence; its final state belongs to t = 0
                y_r, (h_r, c_r) = fn(x.flip(0) if x.dim() == 3 else x, h_0[k + 1], c_0[k + 1],
                                     *self._layer_operands(layer, "_reverse"))
                y = torch.cat((y, y_r.flip(0)), dim=-1)
                h_n += [h_r]
                c_n += [c_r]
            x = between(y, layer + 1)
            layer += 1
        if self.batch_first:
            x = x.transpose(0, 1)
        if len(h_n) == 1:   # one layer, one direction: views of the layer's last slots, no copy
            return x, (h_n[0].unsqueeze(0), c_n[0].unsqueeze(0))
        return x, (torch.stack(h_n), torch.stack(c_n))

    # Opt-in (set on an instance or on the class): keep the zero-padded copies of the parameters across inference
    # calls (see _OperandsPadded._layer_operands for when they are refreshed, and for the case they miss).
    cache_padded_operands = False

    def _operand_padding(self, x):
        """(Hp, Ip): hidden and input size to zero-pad this call to, or None when it runs as it is.

        A hidden size that only the general recurrent kernels take (not a multiple of the MFMA k-step, or between
        the sizes the register-resident form covers) runs markedly faster as the next size that the XCD-local or
        register-resident kernels take (T = 256, B = 32, 2 layers, I = H = 650 as 672: forward 1.82 -> 1.15 ms), so
        the module pads W_x, W_h, the biases and the initial states with zeros up to it: the added units' states
        stay exactly zero, nothing of them reaches the others (their columns of W_h and of the next layer's W_x are
        zero), and their gradients are zero.  A 16-bit input size that is not a multiple of 64 keeps the first
        layer's products off the MFMA tile kernel (T = 256, B = 32, H = 1024: I = 650 forward + backward 2.71 ms,
        I = 704 1.64 ms): x and the columns of the first W_x get zero columns up to the next multiple."""
        packed = isinstance(x, nn.utils.rnn.PackedSequence)
        data = x.data if packed else x
        if not data.is_cuda or (not packed and data.dim() != 3):
            return None
        dt = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else data.dtype
        if dt not in _DTYPE_CODE:
            return None
        if packed:
            T, B = int(x.batch_sizes.numel()), int(x.batch_sizes[0])
        else:
            T, B = (data.shape[1], data.shape[0]) if self.batch_first else (data.shape[0], data.shape[1])
        idx = data.device.index if data.device.index is not None else torch.cuda.current_device()
        H, I = self.hidden_size, self.input_size
        training = torch.is_grad_enabled() and (data.requires_grad or any(p.requires_grad for p in self.parameters()))
        Hp = _padded_hidden_size(T, B, H, _DTYPE_CODE[dt], idx, training) or H
        # Where H is padded anyway and stacked layers read it as the K of their input projection: a multiple of 64, which
        # the MFMA tile kernel takes (2 x (T = 256, B = 32): H = 704 forward + backward 2.19 ms, H = 672 2.32).  (Two
        # directions make K = 2H; below 512 the projection is too small to matter.)
        if (Hp != H and self.num_layers > 1 and not self.bidirectional and dt != torch.float32 and Hp % 64 == 32
                and Hp >= 512 and _recurrent_kind(T, B, Hp + 32, _DTYPE_CODE[dt], idx) in (1, 2)):
            Hp += 32
        Ip = -(-I // 64) * 64 if dt != torch.float32 and T * B >= 1024 and data.shape[-1] == I else I
        if Hp <= 64 and I <= 64 and I % 16 == 0:   # a narrow layer's streaming products take any multiple of 16
            Ip = I
        return (Hp, Ip) if (Hp, Ip) != (H, I) else None

    def _forward_operands_padded(self, x, h_c_0, Hp, Ip):
        H, D = self.hidden_size, 2 if self.bidirectional else 1
        if h_c_0 is not None:
            h_c_0 = tuple(F.pad(t, (0, Hp - H)) for t in h_c_0)
        if isinstance(x, nn.utils.rnn.PackedSequence):
            x = nn.utils.rnn.PackedSequence(F.pad(x.data, (0, Ip - self.input_size)), x.batch_sizes, x.sorted_indices,
                                            x.unsorted_indices)
        else:
            x = F.pad(x, (0, Ip - self.input_size))
        y, (h_n, c_n) = _OperandsPadded(self, Hp, Ip).forward(x, h_c_0)

        def cut(t):   # [..., D*Hp] -> [..., D*H]
            if Hp == H:
                return t
            return t[..., :H].contiguous() if D == 1 else torch.cat((t[..., :H], t[..., Hp:Hp + H]), dim=-1)
        if isinstance(y, nn.utils.rnn.PackedSequence):
            y = nn.utils.rnn.PackedSequence(cut(y.data), y.batch_sizes, y.sorted_indices, y.unsorted_indices)
        else:
            y = cut(y)
        return y, (h_n[..., :H].contiguous(), c_n[..., :H].contiguous())

    def extra_repr(self):
        s = "%d, %d, num_layers=%d" % (self.input_size, self.hidden_size, self.num_layers)
        for name in ("bias", "batch_first", "bidirectional", "state_grads"):
            if getattr(self, name) != (name == "bias"):
                s += ", %s=%s" % (name, getattr(self, name))
        if self.dropout:
            s += ", dropout=%g" % self.dropout
        return s



class _OperandsPadded:
    """What FastLSTM.forward reads of a module, with the hidden size Hp, the input size Ip and the module's parameters
    zero-padded to them (FastLSTM._operand_padding): W [4H, K] is four gate blocks of H rows, each padded to Hp rows;
    the K = H columns of W_h, and the K = D*H columns of a deeper layer's W_x (D blocks of H, one per direction), are
    padded alike, the K = I columns of the first layer's W_x to Ip.  The pads are differentiable, so the gradients
    arrive at the module's own parameters."""

    forward = FastLSTM.forward
    _forward_packed = FastLSTM._forward_packed
    _packed_range_rows = FastLSTM._packed_range_rows
    _run_padded = FastLSTM._run_padded
    _two_layers_at_once = FastLSTM._two_layers_at_once

    def __init__(self, module, Hp, Ip):
        self._module, self.hidden_size, self.input_size, self._operands = module, Hp, Ip, {}
        for name in ("num_layers", "version", "bias", "batch_first", "bidirectional", "state_grads", "dropout", "training"):
            setattr(self, name, getattr(module, name))

    def parameters(self):
        return self._module.parameters()

    def _operand_padding(self, x):
        return None

    def _layer_operands(self, layer, suffix=""):
        if (layer, suffix) not in self._operands:
            H, Hp, D = self._module.hidden_size, self.hidden_size, 2 if self.bidirectional else 1
            base = self._module._layer_operands(layer, suffix)
            Wx, bx, Wh, bh = base
            # Where no gradient can reach the parameters (inference) and the module opted in
            # (FastLSTM.cache_padded_operands), the padded copies are kept on the module across calls, stamped with the
            # identity and the version counter of each parameter: an optimizer step, a load_state_dict or a new
            # Parameter object makes the stamp differ and the copies are made again.  Off by default: an in-place edit
            # through `.data` (weight clipping, swapping in averaged weights) bypasses the version counter and would
            # leave stale copies.  (A training call needs the pads in its autograd graph and makes them per call.)
            keep = (self.bias and getattr(self._module, "cache_padded_operands", False)
                    and not (torch.is_grad_enabled() and any(t.requires_grad for t in base)))
            key = (layer, suffix, Hp, self.input_size)
            stamp = tuple((id(t), t._version, t.data_ptr(), t.dtype, t.device) for t in base)
            cache = self._module.__dict__.setdefault("_padded_operand_cache", {})
            if keep and key in cache and cache[key][0] == stamp:
                self._operands[(layer, suffix)] = cache[key][1]
                return cache[key][1]
            p = Hp - H
            if layer == 0:
                Wx = F.pad(Wx.reshape(4, H, -1), (0, self.input_size - self._module.input_size, 0, p))
            else:
                Wx = F.pad(Wx.reshape(4, H, D, H), (0, p, 0, 0, 0, p))
            ops = (Wx.reshape(4 * Hp, -1), F.pad(bx.reshape(4, H), (0, p)).reshape(-1),
                   F.pad(Wh.reshape(4, H, H), (0, p, 0, p)).reshape(4 * Hp, Hp), F.pad(bh.reshape(4, H), (0, p)).reshape(-1))
            if keep:
                ops = tuple(t.detach() for t in ops)
                cache[key] = (stamp, ops)
            self._operands[(layer, suffix)] = ops
        return self._operands[(layer, suffix)]

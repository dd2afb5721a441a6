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
import os

import torch
import torch.nn as nn
from torch.amp import custom_bwd, custom_fwd

from . import _lib

dtype_str = {  # fastlstm/lstm.py:24-28
    torch.float32: "fp32",
    torch.float16: "fp16",
    torch.bfloat16: "bf16",
}
_DTYPE_CODE = {torch.float32: _lib.FP32, torch.float16: _lib.FP16, torch.bfloat16: _lib.BF16}

# When set, every recurrent launch is followed by a device sync and a check of the
# workspace status word (barrier time-out detection).  Off by default: the calls
# are fully asynchronous, as in the reference.
CHECK_STATUS = os.environ.get("FASTLSTM_CHECK_STATUS", "0") == "1"


def _code(t):
    if t.dtype not in _DTYPE_CODE:
        raise TypeError("fastlstm_amd supports float32, float16 and bfloat16, got %s" % t.dtype)
    return _DTYPE_CODE[t.dtype]


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "fastlstm_amd runs on the GPU only (tensor on %s); there is no CPU fallback" % t.device)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _plan(device, B, H, code, backward):
    plan = _lib.Plan()
    idx = device.index if device.index is not None else torch.cuda.current_device()
    _lib.check(_lib.load().fastlstm_plan_device(idx, B, H, code, int(backward), plan), "fastlstm_plan_device")
    return plan


# Largest exchange ring (one slot per timestep) a recurrent call may allocate.
RING_MAX_BYTES = 2 << 30


def _workspace(plan, T, H, code, backward, device):
    """Recurrence workspace, with the part the kernels need zeroed (header, counters, flags).

    Plans whose workgroups synchronise across CUs get a ring with one exchange slot per timestep,
    sized by fastlstm_recurrent_workspace_bytes(): no address of it is read before its only
    write, so the kernels can read the exchange data through the caches.  The forward pass then
    uses the XCD-local kernel where the shape allows (the barrier group on one XCD, exchange
    through its L2); the backward pass reads d_ifgo[t] once per XCD instead of once per CU.
    Without room for the ring (RING_MAX_BYTES) the two-slot workspace of the plan is used."""
    if plan.wave_split != 2:
        ring = _lib.load().fastlstm_recurrent_workspace_bytes(plan, T, H, code, 1 if backward else 0)
        if plan.ws_bytes < ring <= RING_MAX_BYTES:
            ws = torch.empty(ring, dtype=torch.uint8, device=device)
            zero = ring if plan.ring_needs_zero else plan.ws_zero_bytes
            ws[:zero].zero_()
            return ws
    return torch.zeros(plan.ws_bytes, dtype=torch.uint8, device=device)


def _check_ws(ws, what):
    if CHECK_STATUS:
        head = ws[:64].cpu().numpy().tobytes()  # synchronises
        _lib.check(_lib.load().fastlstm_ws_status(head), what)


def lstm_persistent_fwd(x, h0, c0, Wx, bx, Wh, bh, version=None):
    """x[T,B,I] (or [B,I]) -> (out[T+1,B,H], cell[T+1,B,H], ifgo[T,B,4H]).

    out[0]/cell[0] hold the initial state (zeros when h0 is None); ifgo holds
    the full gate pre-activations of every step (kept for the backward pass).
    `version` is accepted for signature compatibility; there is one path.
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
    lib = _lib.load()
    with torch.cuda.device(x.device):
        ifgo = torch.empty((seq_len, batch_size, 4 * hidden_size), device=x.device, dtype=x.dtype)
        # two allocations (the reference slices one, lstm.py:84-86): each base pointer must
        # be 16-byte aligned for the vector loads of the weight-gradient GEMM
        out = torch.empty((seq_len + 1, batch_size, hidden_size), device=x.device, dtype=x.dtype)
        cell = torch.empty_like(out)
        if h0 is not None:  # fastlstm/lstm.py:88-90
            out[0] = h0
            cell[0] = c0
        else:
            out[0].zero_()
            cell[0].zero_()
        plan = _plan(x.device, batch_size, hidden_size, code, False)
        ws = _workspace(plan, seq_len, hidden_size, code, False, x.device)
        stream = _stream()
        # input projection + time loop in one call (the library fuses the two where CUs would idle)
        _lib.check(lib.fastlstm_fwd_layer(x.data_ptr(), Wx.data_ptr(), bx.data_ptr(), bh.data_ptr(), Wh.data_ptr(),
                                          ifgo.data_ptr(), out.data_ptr(), cell.data_ptr(), ws.data_ptr(),
                                          ws.numel(), seq_len, batch_size, input_size, hidden_size, code, stream),
                   "fastlstm_fwd_layer")
        _check_ws(ws, "fastlstm_fwd_layer")
    return out, cell, ifgo


def Wgrad(d_ifgo, x, h):
    """(dbx, dbh, dWx, dWh) from d_ifgo[T,B,4H], x[T,B,I], h[T+1,B,H]
    (fastlstm/lstm.py:494-501; the same db tensor is returned twice)."""
    _require_gpu(d_ifgo, x, h)
    code = _code(d_ifgo)
    T, B, G = d_ifgo.shape
    H, I = G // 4, x.shape[-1]
    lib = _lib.load()
    with torch.cuda.device(x.device):
        d_ifgo, x, h = d_ifgo.contiguous(), x.contiguous(), h.contiguous()
        dWx = torch.empty((G, I), device=x.device, dtype=x.dtype)
        dWh = torch.empty((G, H), device=x.device, dtype=x.dtype)
        db = torch.empty((G,), device=x.device, dtype=x.dtype)
        nbytes = lib.fastlstm_wgrad_workspace_bytes(T, B, I, H, code)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        _lib.check(lib.fastlstm_gemm_wgrad(d_ifgo.data_ptr(), x.data_ptr(), h.data_ptr(), dWx.data_ptr(),
                                           dWh.data_ptr(), db.data_ptr(), ws.data_ptr(), ws.numel(), T, B, I,
                                           H, code, _stream()), "fastlstm_gemm_wgrad")
    return db, db, dWx, dWh


def lstm_persistent_bwd(dh, dc_n, dh_n, x, h, cell, ifgo, Wx, Wh):
    """Reverse pass.  dh[T,B,H]: gradient of out[1:]; dc_n, dh_n [B,H]: gradients
    flowing into the last cell / hidden state, overwritten with the gradients of
    the initial state and returned (fastlstm/lstm.py:236-334).
    Returns (d_x, dh_0, dc_0, dWx, dbx, dWh, dbh)."""
    _require_gpu(dh, dc_n, dh_n, x, h, cell, ifgo, Wx, Wh)
    code = _code(ifgo)
    seq_len, batch_size, hidden_size = dh.shape
    input_size = Wx.shape[1]
    lib = _lib.load()
    with torch.cuda.device(x.device):
        dh = dh.contiguous()
        if dh.dtype != ifgo.dtype:
            dh = dh.to(ifgo.dtype)
        assert dc_n.is_contiguous() and dh_n.is_contiguous()
        d_ifgo = torch.empty_like(ifgo)
        plan = _plan(x.device, batch_size, hidden_size, code, True)
        ws = _workspace(plan, seq_len, hidden_size, code, True, x.device)
        stream = _stream()
        x, h = x.contiguous(), h.contiguous()
        d_x = torch.empty_like(x)
        G = 4 * hidden_size
        dWx = torch.empty((G, input_size), device=x.device, dtype=x.dtype)
        dWh = torch.empty((G, hidden_size), device=x.device, dtype=x.dtype)
        db = torch.empty((G,), device=x.device, dtype=x.dtype)
        wws = torch.empty(lib.fastlstm_wgrad_workspace_bytes(seq_len, batch_size, input_size, hidden_size, code),
                          dtype=torch.uint8, device=x.device)
        # reverse time loop + dx + weight gradients in one call (the library fuses them where CUs would idle)
        _lib.check(lib.fastlstm_bwd_layer(dh.data_ptr(), dh_n.data_ptr(), dc_n.data_ptr(), ifgo.data_ptr(),
                                          cell.data_ptr(), d_ifgo.data_ptr(), Wh.data_ptr(), Wx.data_ptr(),
                                          x.data_ptr(), h.data_ptr(), d_x.data_ptr(), dWx.data_ptr(),
                                          dWh.data_ptr(), db.data_ptr(), ws.data_ptr(), ws.numel(),
                                          wws.data_ptr(), wws.numel(), seq_len, batch_size, input_size,
                                          hidden_size, code, stream),
                   "fastlstm_bwd_layer")
        _check_ws(ws, "fastlstm_bwd_layer")
        dbx = dbh = db   # the same tensor twice, as Wgrad returns it (fastlstm/lstm.py:501)
    return d_x, dh_n, dc_n, dWx, dbx, dWh, dbh


class PersistentLSTMfn(torch.autograd.Function):
    """apply(x, h_0|None, c_0|None, Wx[4H,I], bx[4H], Wh[4H,H], bh[4H]) ->
    (out[T,B,H], (h_T[B,H], c_T[B,H])).  The nested tuple makes h_T/c_T
    non-differentiable, as in the reference (fastlstm/lstm.py:504-538)."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, x, h_0, c_0, Wx, bx, Wh, bh):
        if torch.is_autocast_enabled():  # fastlstm/lstm.py:509-515 (h_0/c_0 are not cast)
            target = torch.get_autocast_dtype("cuda")
            x = x.to(target)
            Wx = Wx.to(target)
            Wh = Wh.to(target)
            bx = bx.to(target)
            bh = bh.to(target)
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
        x, out, cell, ifgo, Wx, Wh = ctx.saved_tensors
        if d_out_cell is None:
            dc_n, dh_n = torch.zeros_like(cell[0]), torch.zeros_like(cell[0])
        else:
            raise ValueError("Not implemented")  # fastlstm/lstm.py:528-531
        d_x, dh_0, dc_0, dWx, dbx, dWh, dbh = lstm_persistent_bwd(
            dh, dc_n, dh_n, x, out, cell, ifgo, Wx, Wh
        )
        if ctx.h0_is_nan:
            dh_0 = None
            dc_0 = None
        return d_x, dh_0, dc_0, dWx, dbx, dWh, dbh


class FastLSTM(nn.Module):
    """nn.LSTM-compatible parameters (names, shapes, order, seeded values) and the
    reference's forward contract (fastlstm/lstm.py:586-698): sequence-first input
    x[T,B,I], optional (h_0[L,B,H], c_0[L,B,H]); returns out[T,B,H], (h_n, c_n)."""

    def __init__(self, input_size, hidden_size, num_layers=1, version="persistent", device=None,
                 dtype=None):
        super().__init__()
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.num_layers = num_layers
        self.version = version
        self.device = device
        self.dtype = dtype
        sqrt_k_inv = 1 / hidden_size**0.5
        # same RNG consumption order as nn.LSTM: w_ih, w_hh, b_ih, b_hh per layer
        for layer in range(num_layers):
            shapes = [
                ("weight_ih_l%d" % layer, (4 * hidden_size, input_size if layer == 0 else hidden_size)),
                ("weight_hh_l%d" % layer, (4 * hidden_size, hidden_size)),
                ("bias_ih_l%d" % layer, (4 * hidden_size,)),
                ("bias_hh_l%d" % layer, (4 * hidden_size,)),
            ]
            for name, shape in shapes:
                value = torch.rand(*shape, device=device, dtype=dtype) * 2 * sqrt_k_inv - sqrt_k_inv
                setattr(self, name, nn.Parameter(value))

    def forward(self, x, h_c_0=None):
        if h_c_0 is None:
            h_0, c_0 = [None] * self.num_layers, [None] * self.num_layers
        else:
            h_0, c_0 = h_c_0
        if self.version != "persistent":
            # the reference also offers "graph", "naive-pt" and "v1"; this build has one path
            raise ValueError(f"Not Implemnted: {self.version}")
        fn = PersistentLSTMfn.apply
        h_n, c_n = [], []
        for layer in range(self.num_layers):
            x, (h_i, c_i) = fn(
                x,
                h_0[layer],
                c_0[layer],
                getattr(self, f"weight_ih_l{layer}"),
                getattr(self, f"bias_ih_l{layer}"),
                getattr(self, f"weight_hh_l{layer}"),
                getattr(self, f"bias_hh_l{layer}"),
            )
            h_n += [h_i]
            c_n += [c_i]
        return x, (torch.stack(h_n), torch.stack(c_n))

    def extra_repr(self):
        return "%d, %d, num_layers=%d" % (self.input_size, self.hidden_size, self.num_layers)

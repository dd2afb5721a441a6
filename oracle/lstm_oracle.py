"""ctypes/numpy front-end of oracle/lstm_oracle.c -- TEST INFRASTRUCTURE ONLY.

The C file restates the reference's persistent-path algorithm
(fastlstm/lstm.py:31-146, 236-334, 494-501, 1087-1223 and the rounding points
of fastlstm/kernels.py:631-657, 1301-1390) on the CPU.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module; the product never routes through it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblstm_oracle.so")
_lib = None

ROUND_NONE, ROUND_FP16, ROUND_BF16 = 0, 1, 2


def build(force=False):
    """Compile the oracle with gcc (make).  Called by __graft_entry__.build()."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "liblstm_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_round_fp16.restype = ctypes.c_float
        _lib.oracle_round_fp16.argtypes = [ctypes.c_float]
        _lib.oracle_round_bf16.restype = ctypes.c_float
        _lib.oracle_round_bf16.argtypes = [ctypes.c_float]
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _prep(a, dt):
    return None if a is None else np.ascontiguousarray(np.asarray(a), dtype=dt)


def forward(x, h0, c0, Wx, bx, Wh, bh, dtype=np.float64, round_mode=ROUND_NONE):
    """Returns (out[T+1,B,H], cell[T+1,B,H], ifgo[T,B,4H]); slot 0 of out/cell
    is the initial state (zeros when h0/c0 are None), as fastlstm/lstm.py:84-90."""
    dt = np.dtype(dtype)
    x, Wx, bx, Wh, bh = (_prep(a, dt) for a in (x, Wx, bx, Wh, bh))
    h0, c0 = _prep(h0, dt), _prep(c0, dt)
    if x.ndim == 2:  # fastlstm/lstm.py:33-34
        x = x[None]
    T, B, I = x.shape
    H = Wh.shape[1]
    assert Wx.shape == (4 * H, I) and Wh.shape == (4 * H, H)
    assert bx.shape == (4 * H,) and bh.shape == (4 * H,)
    assert (h0 is None) == (c0 is None)
    if h0 is not None:
        assert h0.shape == (B, H) and c0.shape == (B, H)
    out = np.empty((T + 1, B, H), dt)
    cell = np.empty((T + 1, B, H), dt)
    ifgo = np.empty((T, B, 4 * H), dt)
    fn = lib().oracle_lstm_fwd_f64 if dt == np.float64 else lib().oracle_lstm_fwd_f32
    fn.restype = None
    fn(ctypes.c_int(T), ctypes.c_int(B), ctypes.c_int(I), ctypes.c_int(H), _ptr(x), _ptr(h0),
       _ptr(c0), _ptr(Wx), _ptr(bx), _ptr(Wh), _ptr(bh), _ptr(out), _ptr(cell), _ptr(ifgo),
       ctypes.c_int(round_mode))
    return out, cell, ifgo


def backward(dout, dh_n, dc_n, x, out, cell, ifgo, Wx, Wh, dtype=np.float64,
             round_mode=ROUND_NONE):
    """Returns dict(dx, dh0, dc0, dWx, dWh, db, d_ifgo) -- the quantities of
    fastlstm/lstm.py:236-334 (db is returned once; the reference hands the same
    tensor back for both biases, lstm.py:501)."""
    dt = np.dtype(dtype)
    dout, x, out, cell, ifgo, Wx, Wh = (_prep(a, dt) for a in (dout, x, out, cell, ifgo, Wx, Wh))
    dh_n, dc_n = _prep(dh_n, dt), _prep(dc_n, dt)
    if x.ndim == 2:
        x = x[None]
    T, B, I = x.shape
    H = Wh.shape[1]
    assert dout.shape == (T, B, H) and out.shape == (T + 1, B, H) and cell.shape == (T + 1, B, H)
    assert ifgo.shape == (T, B, 4 * H)
    res = dict(dx=np.empty((T, B, I), dt), dh0=np.empty((B, H), dt), dc0=np.empty((B, H), dt),
               dWx=np.empty((4 * H, I), dt), dWh=np.empty((4 * H, H), dt),
               db=np.empty((4 * H,), dt), d_ifgo=np.empty((T, B, 4 * H), dt))
    fn = lib().oracle_lstm_bwd_f64 if dt == np.float64 else lib().oracle_lstm_bwd_f32
    fn.restype = None
    fn(ctypes.c_int(T), ctypes.c_int(B), ctypes.c_int(I), ctypes.c_int(H), _ptr(dout), _ptr(dh_n),
       _ptr(dc_n), _ptr(x), _ptr(out), _ptr(cell), _ptr(ifgo), _ptr(Wx), _ptr(Wh),
       _ptr(res["dx"]), _ptr(res["dh0"]), _ptr(res["dc0"]), _ptr(res["dWx"]), _ptr(res["dWh"]),
       _ptr(res["db"]), _ptr(res["d_ifgo"]), ctypes.c_int(round_mode))
    return res


def round_fp16(a):
    f = np.vectorize(lambda v: lib().oracle_round_fp16(float(v)), otypes=[np.float32])
    return f(np.asarray(a, np.float32))


def round_bf16(a):
    f = np.vectorize(lambda v: lib().oracle_round_bf16(float(v)), otypes=[np.float32])
    return f(np.asarray(a, np.float32))

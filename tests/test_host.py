"""CPU-side tests: the C ABI loads and exports what include/fastlstm_hip.h and fastlstm_hip_diag.h declare,
argument validation returns error codes before any HIP call, the tiling rule keeps
its invariants, the barrier/version protocol is deadlock- and hazard-free in a model,
and the Python module mirrors the reference's interface (fastlstm/lstm.py:586-698)."""
import ctypes
import os
import random
import re

import numpy as np
import pytest
import torch

from fastlstm_amd import FastLSTM, PersistentLSTMfn, _lib
from helpers import make_problem, to_np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HAS_GPU = torch.cuda.is_available()


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fastlstm_hip.h")).read()
    diag = open(os.path.join(ROOT, "include", "fastlstm_hip_diag.h")).read()
    product = set(re.findall(r"\b(fastlstm_[a-z_0-9]+)\s*\(", header))
    # the boundary header carries no process-wide switches and no measurement code
    assert not any(n.startswith(("fastlstm_set_", "fastlstm_diag_", "fastlstm_get_")) for n in product), product
    declared = product | set(re.findall(r"\b(fastlstm_[a-z_0-9]+)\s*\(", diag))
    assert {"fastlstm_fwd_persistent", "fastlstm_bwd_persistent", "fastlstm_gemm_ifgo", "fastlstm_gemm_dx",
            "fastlstm_gemm_wgrad", "fastlstm_plan_for", "fastlstm_strerror"} <= declared
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(_lib.SIGNATURES), "ctypes signature table out of sync with the header"
    assert b"gfx950" in _lib.load().fastlstm_version()


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    a = 4096  # a fake, aligned, non-null "device pointer": validation fails before it is touched
    assert lib.fastlstm_gemm_ifgo(None, a, a, a, a, 4, 4, 4, 4, 0, None) == _lib.ERR_NULL
    assert lib.fastlstm_gemm_ifgo(a, a, a, a, a, 0, 4, 4, 4, 0, None) == _lib.ERR_DIM
    assert lib.fastlstm_gemm_ifgo(a, a, a, a, a, 4, 4, 4, 4, 3, None) == _lib.ERR_DTYPE
    assert lib.fastlstm_gemm_ifgo(a + 4, a, a, a, a, 4, 4, 4, 4, 0, None) == _lib.ERR_ALIGN
    assert lib.fastlstm_gemm_ifgo(a, a, a, a, a, 1 << 20, 1 << 12, 4, 4, 0, None) == _lib.ERR_DIM
    assert lib.fastlstm_gemm_dx(a, None, a, 4, 4, 4, 4, 0, None) == _lib.ERR_NULL
    assert lib.fastlstm_gemm_dx(a, a, a + 2, 4, 4, 4, 4, 1, None) == _lib.ERR_ALIGN
    assert lib.fastlstm_gemm_wgrad(a, a, a, a, a, a, None, 0, 4, 4, 4, 4, 0, None) == _lib.ERR_NULL
    assert lib.fastlstm_gemm_wgrad(a, a, a, a, a, a, a, 0, 4, 4, 4, 4, 0, None) == _lib.ERR_WORKSPACE
    assert lib.fastlstm_fwd_persistent(a, a, None, a, a, 1 << 20, 4, 4, 4, 0, None) == _lib.ERR_NULL
    assert lib.fastlstm_fwd_persistent(a, a, a, a, a, 1 << 20, 4, -1, 4, 0, None) == _lib.ERR_DIM
    assert lib.fastlstm_fwd_persistent(a, a, a, a, a, 1 << 20, 4, 4, 4, 7, None) == _lib.ERR_DTYPE
    assert lib.fastlstm_bwd_persistent(a, a, a, a, a, a, a, a + 8, 1 << 20, 4, 4, 4, 0, None) == _lib.ERR_ALIGN
    assert lib.fastlstm_bwd_persistent(a, a, a, None, a, a, a, a, 1 << 20, 4, 4, 4, 0, None) == _lib.ERR_NULL
    # the layer entry points (training and inference form) and the stacked ones validate the same way
    for name in ("fastlstm_fwd_layer", "fastlstm_fwd_layer_infer"):
        fn = getattr(lib, name)
        assert fn(a, a, a, a, a, a, a, None, a, 1 << 20, 4, 4, 4, 4, 0, None) == _lib.ERR_NULL
        assert fn(a, a, a, a, a, a, a, a, a, 1 << 20, 4, 4, 0, 4, 0, None) == _lib.ERR_DIM
        assert fn(a, a, a, a, a, a + 8, a, a, a, 1 << 20, 4, 4, 4, 4, 2, None) == _lib.ERR_ALIGN
    for name in ("fastlstm_fwd_stack2", "fastlstm_fwd_stack2_infer"):
        fn = getattr(lib, name)
        assert fn(*([a] * 15), None, 1 << 20, 4, 4, 4, 4, 1, None) == _lib.ERR_NULL
        assert fn(*([a] * 16), 1 << 20, 4, 4, 4, 4, 5, None) == _lib.ERR_DTYPE
    assert lib.fastlstm_recurrent_kernel_kind(4, 4, 4, 9, 0, 1 << 20) == _lib.ERR_DTYPE
    assert lib.fastlstm_recurrent_kernel_kind(0, 4, 4, 0, 0, 1 << 20) == _lib.ERR_DIM
    assert lib.fastlstm_plan_for(256, 163840, 4, 4, 0, 0, None) == _lib.ERR_NULL
    assert lib.fastlstm_ws_status(None) == _lib.ERR_NULL
    if not HAS_GPU:  # with valid arguments the first HIP call fails cleanly on a GPU-less host
        assert lib.fastlstm_fwd_persistent(a, a, a, a, a, 1 << 20, 4, 4, 4, 0, None) == _lib.ERR_HIP
    for code in range(0, -9, -1):
        assert _lib.strerror(code) and "unknown" not in _lib.strerror(code)
    assert "unknown" in _lib.strerror(-99)


def test_ws_status_word():
    lib = _lib.load()
    head = np.zeros(16, np.int32)
    assert lib.fastlstm_ws_status(head.ctypes.data) == _lib.OK
    head[0] = 1
    assert lib.fastlstm_ws_status(head.ctypes.data) == _lib.ERR_TIMEOUT


CUS, LDS = 256, 160 * 1024


@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("backward", [0, 1])
def test_tiling_rule_invariants(dtype, backward):
    lib = _lib.load()
    for B in (1, 4, 16, 44, 64, 100, 128, 256, 600, 2048):
        for H in (1, 16, 33, 64, 65, 128, 257, 512, 768, 1024, 2048, 2100, 3072, 4096, 9000, 16384):
            p = _lib.Plan()
            rc = lib.fastlstm_plan_for(CUS, LDS, B, H, dtype, backward, p)
            assert rc == _lib.OK, (B, H, dtype, backward)   # no hidden size up to 64 units x CUs is refused
            assert p.lds_bytes <= LDS
            assert p.bt % 16 == 0 and p.bt * p.n_btiles * p.batch_chunks >= B
            if H <= 64:  # single hidden tile: barrier-free, any grid size
                assert p.n_htiles == 1 and p.wave_split == 2 and p.batch_chunks == 1 and p.ht >= H
            else:        # every workgroup of a barrier group must be resident (configs.py:56)
                assert p.n_htiles * p.ht >= H and (p.n_htiles - 1) * p.ht < H
                assert p.n_btiles * p.n_htiles <= CUS
                assert (p.n_btiles - 1) * p.bt < B
                assert p.wave_split in (0, 1, 3)
            kstep = 16 if dtype == 0 else 32
            ks = -(-(4 * H if backward else H) // kstep)
            if p.wave_split == 3:
                # streamed weights (the slices do not fit on chip): at most 16 forward / 4 reverse output tiles per
                # workgroup; workspace = header, counters, per batch chunk flags + 2 exchange slots, then all of
                # W_h once in operand order with the k-steps padded to 16
                assert (p.ht // 16) * (p.bt // 16) <= 4 and p.ht in (16, 32, 64)
                ksp = -(-ks // 16) * 16
                flags = -(-(p.n_btiles * (-(-p.n_htiles // 64) * 64) * 4) // 1024) * 1024
                slots = 2 * p.n_btiles * (p.bt // 16) * ksp * 1024
                head = -(-(1024 + 65536 + p.batch_chunks * (flags + slots)) // 4096) * 4096
                assert p.ws_zero_bytes == head
                rows = p.n_htiles * (p.ht // 16 if backward else p.ht // 4)
                assert p.ws_bytes == head + rows * ksp * 1024
            elif p.n_htiles > 1:
                flags = -(-(p.n_btiles * (-(-p.n_htiles // 64) * 64) * 4) // 1024) * 1024
                xbuf = 2 * p.n_btiles * (p.bt // 16) * ks * 1024
                assert p.ws_bytes == 1024 + 65536 + p.batch_chunks * (flags + xbuf)


def test_tiling_rule_headline_configs():
    lib = _lib.load()
    p = _lib.Plan()
    assert lib.fastlstm_plan_for(CUS, LDS, 64, 1024, 1, 0, p) == 0      # config B
    assert p.n_btiles * p.n_htiles == 256                                 # fills every CU
    assert lib.fastlstm_plan_for(CUS, LDS, 128, 2048, 2, 0, p) == 0     # config C: 32 MiB of W_h
    assert p.n_htiles == 256 and p.lds_bytes >= 128 * 1024
    assert lib.fastlstm_plan_for(CUS, LDS, 64, 4096, 1, 0, p) == 0       # 128 MiB of W_h: streamed every step
    assert p.wave_split == 3 and p.n_htiles == 256 and p.bt == 64 and p.ws_bytes > 128 << 20
    assert lib.fastlstm_plan_for(CUS, LDS, 64, 64 * CUS + 1, 1, 0, p) == _lib.ERR_RESIDENCY   # more slices than CUs
    assert lib.fastlstm_plan_for(8, LDS, 64, 1024, 1, 0, p) == _lib.ERR_RESIDENCY  # too few CUs
    assert lib.fastlstm_plan_for(CUS, LDS, 64, 1024, 9, 0, p) == _lib.ERR_DTYPE
    assert lib.fastlstm_plan_for(CUS, LDS, 0, 1024, 1, 0, p) == _lib.ERR_DIM


def test_xcd_major_numbering_is_a_bijection():
    # mirrors xcd_major_id() of csrc/recurrent_common.hpp
    def xcd_major(bid, nwg):
        xcd, slot = bid % 8, bid // 8
        base, rem = nwg // 8, nwg % 8
        return xcd * base + min(xcd, rem) + slot
    for nwg in list(range(1, 40)) + [64, 231, 255, 256]:
        ids = sorted(xcd_major(b, nwg) for b in range(nwg))
        assert ids == list(range(nwg))
        # workgroups of one XCD get consecutive logical ids
        for x in range(min(8, nwg)):
            mine = sorted(xcd_major(b, nwg) for b in range(x, nwg, 8))
            assert mine == list(range(mine[0], mine[0] + len(mine)))


def test_version_barrier_model_has_no_deadlock_and_no_slot_hazard():
    """Randomly interleaved model of the forward protocol: n workgroups, 2 exchange
    slots; step t waits for version t+1 of every peer, reads slot t%2, writes slot
    (t+1)%2, publishes version t+2.  A write must never hit a slot a peer still
    has to read, and every schedule must terminate."""
    rng = random.Random(0)
    for n, T in ((1, 5), (2, 7), (5, 9), (17, 6)):
        flags = [0] * n
        pc = [("publish0", 0)] * n           # (phase, step)
        slot_version = [[0, 0] for _ in range(n)]  # version each WG's part of a slot holds
        done = 0
        for _ in range(200000):
            if done == n:
                break
            w = rng.randrange(n)
            phase, t = pc[w]
            if phase == "publish0":
                slot_version[w][0] = 1
                flags[w] = 1
                pc[w] = ("wait", 0)
            elif phase == "wait":
                if all(f >= t + 1 for f in flags):
                    pc[w] = ("read", t)
            elif phase == "read":
                # every peer's part of slot t%2 must hold exactly version t+1
                assert all(slot_version[p][t % 2] == t + 1 for p in range(n)), (n, w, t)
                pc[w] = ("write", t)
            elif phase == "write":
                slot_version[w][(t + 1) % 2] = t + 2
                flags[w] = t + 2
                if t + 1 == T:
                    pc[w] = ("done", t)
                    done += 1
                else:
                    pc[w] = ("wait", t + 1)
        assert done == n, "schedule did not terminate"


# ---- module interface -------------------------------------------------------------------

def test_init_matches_nn_lstm():  # reference: tests/test_lstm.py:116-129
    torch.manual_seed(123)
    m1 = FastLSTM(8, 3, num_layers=2)
    torch.manual_seed(123)
    m2 = torch.nn.LSTM(8, 3, num_layers=2)
    assert [n for n, _ in m1.named_parameters()] == [n for n, _ in m2.named_parameters()]
    for n, p in m1.named_parameters():
        assert p.shape == getattr(m2, n).shape
        torch.testing.assert_close(p, getattr(m2, n))


@pytest.mark.parametrize("kw", [dict(bias=False), dict(bidirectional=True), dict(bias=False, bidirectional=True),
                                dict(batch_first=True)])
def test_option_surface_parameters_match_nn_lstm(kw):
    """bias / bidirectional change the parameter set: same names, order, shapes and seeded values as
    nn.LSTM (the reference lists these options as unsupported, README.md:92-93), and state dicts load
    in both directions."""
    torch.manual_seed(7)
    m1 = FastLSTM(6, 5, num_layers=3, **kw)
    torch.manual_seed(7)
    m2 = torch.nn.LSTM(6, 5, num_layers=3, **kw)
    assert [n for n, _ in m1.named_parameters()] == [n for n, _ in m2.named_parameters()]
    for n, p in m1.named_parameters():
        torch.testing.assert_close(p, getattr(m2, n))
    m2.load_state_dict(m1.state_dict())
    m1.load_state_dict(m2.state_dict())
    assert "num_layers=3" in m1.extra_repr() and all(k in m1.extra_repr() for k in kw)


def test_state_dict_interop_with_nn_lstm():
    m1 = FastLSTM(5, 7, num_layers=2)
    m2 = torch.nn.LSTM(5, 7, num_layers=2)
    m2.load_state_dict(m1.state_dict())
    m1.load_state_dict(m2.state_dict())
    for n, p in m1.named_parameters():
        assert torch.equal(p, getattr(m2, n))


def test_constructor_attributes_and_dtype():
    m = FastLSTM(4, 6, num_layers=3, dtype=torch.float16)
    assert (m.input_size, m.hidden_size, m.num_layers, m.version) == (4, 6, 3, "persistent")
    assert m.weight_ih_l0.shape == (24, 4) and m.weight_ih_l2.shape == (24, 6)
    assert m.weight_hh_l1.dtype == torch.float16
    k = 1 / 6 ** 0.5
    assert float(m.weight_hh_l0.float().abs().max()) <= k + 1e-3


def test_unknown_version_raises_value_error():  # fastlstm/lstm.py:682-683
    m = FastLSTM(4, 4, version="does-not-exist")
    with pytest.raises(ValueError):
        m(torch.zeros(2, 1, 4))


def test_cpu_tensors_fail_loudly_no_fallback():
    m = FastLSTM(4, 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        m(torch.zeros(2, 1, 4))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        PersistentLSTMfn.apply(torch.zeros(2, 1, 4), None, None, m.weight_ih_l0, m.bias_ih_l0,
                               m.weight_hh_l0, m.bias_hh_l0)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "fastlstm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".inc", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_oracle_matches_golden_vectors(oracle):
    z = np.load(os.path.join(ROOT, "tests", "golden", "lstm_golden.npz"))
    names = sorted({k.split("/")[0] for k in z.files})
    assert names == ["nostate", "onestep", "ragged", "tiny"]
    for name in names:
        g = lambda k: z["%s/in/%s" % (name, k)].astype(np.float64) if "%s/in/%s" % (name, k) in z.files else None
        out, cell, ifgo = oracle.forward(g("x"), g("h0"), g("c0"), g("Wx"), g("bx"), g("Wh"), g("bh"))
        np.testing.assert_allclose(out[1:], z[name + "/out/out"], rtol=1e-10, atol=1e-12)
        np.testing.assert_allclose(cell[-1], z[name + "/out/c_n"], rtol=1e-10, atol=1e-12)
        r = oracle.backward(g("dout"), g("dh_n"), g("dc_n"), g("x"), out, cell, ifgo, g("Wx"), g("Wh"))
        for k, ok in (("dx", "dx"), ("dWx", "dWx"), ("dWh", "dWh"), ("db", "dbx"), ("db", "dbh")):
            np.testing.assert_allclose(r[k], z["%s/out/%s" % (name, ok)], rtol=1e-9, atol=1e-10)
        if g("h0") is not None:
            np.testing.assert_allclose(r["dh0"], z[name + "/out/dh0"], rtol=1e-9, atol=1e-10)
            np.testing.assert_allclose(r["dc0"], z[name + "/out/dc0"], rtol=1e-9, atol=1e-10)


def test_device_status_without_a_planned_device_is_ok():
    """No planning call was made (there is no GPU here), so no status word exists: the query answers OK
    without touching the HIP runtime, and so does the look every recurrent entry point takes first."""
    lib = _lib.load()
    assert lib.fastlstm_device_status(-1, 0) == _lib.OK
    assert lib.fastlstm_device_status(0, 1) == _lib.OK

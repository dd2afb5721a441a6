"""ctypes binding of libfastlstm_hip.so (the C ABI in include/fastlstm_hip.h).

The library is the only compute path of this package: if it is missing the
import of `load()` fails loudly -- there is no eager/PyTorch fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfastlstm_hip.so")

FP32, FP16, BF16 = 0, 1, 2

OK = 0
ERR_NULL, ERR_DIM, ERR_DTYPE, ERR_ALIGN = -1, -2, -3, -4
ERR_RESIDENCY, ERR_WORKSPACE, ERR_HIP, ERR_TIMEOUT = -5, -6, -7, -8


class Plan(ctypes.Structure):
    """struct fastlstm_plan"""
    _fields_ = [("num_cus", ctypes.c_int), ("lds_limit", ctypes.c_int), ("bt", ctypes.c_int),
                ("ht", ctypes.c_int), ("n_btiles", ctypes.c_int), ("n_htiles", ctypes.c_int),
                ("batch_chunks", ctypes.c_int), ("wave_split", ctypes.c_int),
                ("lds_bytes", ctypes.c_int), ("ws_bytes", ctypes.c_size_t),
                ("ws_zero_bytes", ctypes.c_size_t), ("ring_needs_zero", ctypes.c_int)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
SIGNATURES = {
    "fastlstm_plan_for": (_i, [_i, _i, _i, _i, _i, _i, ctypes.POINTER(Plan)]),
    "fastlstm_plan_device": (_i, [_i, _i, _i, _i, _i, ctypes.POINTER(Plan)]),
    "fastlstm_recurrent_workspace_bytes": (_sz, [ctypes.POINTER(Plan), _i, _i, _i, _i]),
    "fastlstm_recurrent_kernel_kind": (_i, [_i, _i, _i, _i, _i, _sz]),
    "fastlstm_recurrent_rows_per_launch": (_i, [_i, _i, _i, _i, _i, _sz]),
    "fastlstm_fwd_stack2": (_i, [_vp] * 16 + [_sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_fwd_stack2_infer": (_i, [_vp] * 16 + [_sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_stack2_workspace_bytes": (_sz, [ctypes.POINTER(Plan), _i, _i, _i]),
    "fastlstm_fwd_stack2_fused": (_i, [_i, _i, _i, _i, _i, _sz]),
    "fastlstm_bwd_stack2": (_i, [_vp] * 27 + [_sz, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_stack2_bwd_workspace_bytes": (_sz, [ctypes.POINTER(Plan), _i, _i, _i]),
    "fastlstm_bwd_stack2_fused": (_i, [_i, _i, _i, _i, _i, _sz]),
    "fastlstm_fwd_persistent_pair": (_i, [_vp] * 9 + [_sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_bwd_persistent_pair": (_i, [_vp] * 15 + [_sz, _i, _i, _i, _i, _vp]),
    "fastlstm_pair_fused": (_i, [_i, _i, _i, _i, _i, _sz]),
    "fastlstm_fwd_persistent_multi": (_i, [_i] + [_vp] * 5 + [_sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_bwd_persistent_multi": (_i, [_i] + [_vp] * 8 + [_sz, _i, _i, _i, _i, _vp]),
    "fastlstm_multi_fused": (_i, [_i, _i, _i, _i, _i, _i, _sz]),
    "fastlstm_multi_workspace_bytes": (_sz, [ctypes.POINTER(Plan), _i, _i, _i, _i, _i]),
    "fastlstm_stack2_bwd_wgrad_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "fastlstm_gemm_ifgo": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_fwd_persistent": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _vp]),
    "fastlstm_fwd_layer": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_fwd_layer_infer": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_fwd_layer_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_noalloc_scratch_bytes": (_sz, []),
    "fastlstm_bwd_layer": (_i, [_vp] * 15 + [_sz, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_bwd_persistent": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _vp]),
    "fastlstm_gemm_dx": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_gemm_dx_split": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "fastlstm_gemm_wgrad": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_wgrad_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "fastlstm_gemm_dx_wgrad": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _vp]),
    "fastlstm_diag_step_probe": (_i, [_i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "fastlstm_diag_step_probe_bytes": (_sz, [_i, _i, _i]),
    "fastlstm_ws_status": (_i, [_vp]),
    "fastlstm_device_status": (_i, [_i, _i]),
    "fastlstm_prepare_forward": (_i, [_vp, _sz, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "fastlstm_set_spin_limit": (None, [ctypes.c_longlong]),
    "fastlstm_set_kernel_families": (None, [_i]),
    "fastlstm_set_gemm_baseline": (None, [_i]),
    "fastlstm_get_kernel_families": (_i, []),
    "fastlstm_set_gemm_trace": (None, [_vp]),
    "fastlstm_set_recurrent_trace": (None, [_vp]),
    "fastlstm_strerror": (ctypes.c_char_p, [_i]),
    "fastlstm_version": (ctypes.c_char_p, []),
}

_lib = None


def load():
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libfastlstm_hip.so is not built (%s). Build it with `python -m fastlstm_amd.build`; "
                "this package has no fallback path." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def strerror(status):
    return load().fastlstm_strerror(status).decode()


def check(status, what):
    if status != OK:
        raise RuntimeError("%s failed: %s (status %d)" % (what, strerror(status), status))

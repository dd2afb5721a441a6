"""Builds libfastlstm_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m fastlstm_amd.build            # build if sources are newer than the library
    python -m fastlstm_amd.build --force    # rebuild everything

The objects are compiled in parallel (one per translation unit) and linked into
fastlstm_amd/lib/libfastlstm_hip.so, which the Python wrappers load with ctypes.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "lib", "obj")
LIB = os.path.join(LIBDIR, "libfastlstm_hip.so")
SOURCES = ["api.hip", "gemm.hip", "gemm_small.hip", "diag.hip", "recurrent_stream.hip", "plan.cpp", "recurrent_f32.hip", "recurrent_f16.hip", "recurrent_bf16.hip",
           "recurrent_wreg_f32.hip", "recurrent_wreg_f16.hip", "recurrent_wreg_bf16.hip",
           "recurrent_xcd_f32.hip", "recurrent_xcd_f16.hip", "recurrent_xcd_bf16.hip",
           "recurrent_wsplit_f16.hip", "recurrent_wsplit_bf16.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _deps():
    out = [os.path.join(CSRC, f) for f in os.listdir(CSRC)]
    out.append(os.path.join(os.path.dirname(HERE), "include", "fastlstm_hip.h"))
    out.append(os.path.join(os.path.dirname(HERE), "include", "fastlstm_hip_diag.h"))
    return out


def _compile(src):
    obj = os.path.join(OBJDIR, src.rsplit(".", 1)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(force=False, verbose=False):
    os.makedirs(OBJDIR, exist_ok=True)
    if not force and os.path.exists(LIB):
        if os.path.getmtime(LIB) >= max(os.path.getmtime(d) for d in _deps()):
            return LIB
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        results = list(ex.map(_compile, SOURCES))
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *[o for o, _ in results]]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))

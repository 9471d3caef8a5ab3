"""Builds libwtconv_hip.so in-tree with hipcc for gfx950 (no JIT, no cache directory)."""
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libwtconv_hip.so")
SOURCES = [os.path.join(CSRC, "api.hip")]
HEADERS = [os.path.join(CSRC, f) for f in ("common.h", "kernels1d.h", "kernels1d_row.h", "kernels2d.h", "kernels2d_stream.h", "plan.h")] + [
    os.path.join(os.path.dirname(PKG_DIR), "include", "wtconv_hip.h")]

# packed-FP32 code generation is switched off on purpose: every float op is a scalar VALU op
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_library(verbose=False):
    """Compile the HIP sources (always recompiles)."""
    cmd = [hipcc_path()] + HIPCC_FLAGS + SOURCES + ["-o", LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + r.stdout[-4000:] + r.stderr[-8000:])
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


def is_stale():
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > t for p in SOURCES + HEADERS)


if __name__ == "__main__":
    print(build_library(verbose=True))

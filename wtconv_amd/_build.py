"""Builds libwtconv_hip.so in-tree with hipcc for gfx950, and the C++ autograd node that PyTorch calls it through
(no JIT, no cache directory)."""
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libwtconv_hip.so")
SOURCES = [os.path.join(CSRC, "api.hip"), os.path.join(CSRC, "mfma2d.hip"), os.path.join(CSRC, "block.hip"),
           os.path.join(CSRC, "haar.hip")]
HEADERS = [os.path.join(CSRC, f) for f in ("common.h", "host_util.h", "kernels1d.h", "kernels1d_row.h", "kernels2d.h", "kernels2d_mfma.h", "kernels2d_mfma_wgrad.h", "kernels_block.h", "kernels_haar.h", "wgrad_finish.h",
                                         "kernels2d_stream.h", "mfma2d.h", "plan.h")] + [
    os.path.join(os.path.dirname(PKG_DIR), "include", "wtconv_hip.h")]

# packed-FP32 code generation is switched off on purpose: every float op is a scalar VALU op
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-mllvm", "-amdgpu-mfma-vgpr-form=1",     # MFMA accumulators in ordinary VGPRs: no copies to and from AGPRs
               "-Wno-unused-command-line-argument"]
OBJ_DIR = os.path.join(PKG_DIR, "build")


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_library(verbose=False):
    """Compile the HIP sources (always recompiles; one hipcc process per source, side by side) and link."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs, procs = [], []
    for src in SOURCES:
        obj = os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(src))[0] + ".o")
        cmd = [hipcc_path()] + HIPCC_FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        objs.append(obj)
        procs.append(subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True))
    errs = []
    for pr in procs:
        so, se = pr.communicate()
        if pr.returncode != 0:
            errs.append(so[-4000:] + se[-8000:])
    if errs:
        raise RuntimeError("hipcc failed:\n" + "\n".join(errs))
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout[-4000:] + r.stderr[-8000:])
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


BINDING_SRC = os.path.join(CSRC, "torch_binding.cpp")
BINDING_NAME = "_wtconv_torch"
BINDING_PATH = os.path.join(PKG_DIR, BINDING_NAME + ".so")


def build_binding(verbose=False):
    """Compile the C++ autograd node (host code only: g++ against the headers of the installed PyTorch).  It calls
    the HIP library through addresses handed over at import, so it links against PyTorch alone."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-w",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-DUSE_ROCM=1", "-D__HIP_PLATFORM_AMD__=1", f"-DTORCH_EXTENSION_NAME={BINDING_NAME}",
           "-DTORCH_API_INCLUDE_EXTENSION_H"]
    cmd += ["-I" + p for p in cpp_extension.include_paths()]
    cmd += ["-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(rocm, "include")]
    cmd += [BINDING_SRC, "-o", BINDING_PATH + ".tmp", "-L" + tlib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch",
            "-ltorch_python"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the PyTorch binding failed:\n" + r.stdout[-4000:] + r.stderr[-8000:])
    os.replace(BINDING_PATH + ".tmp", BINDING_PATH)
    return BINDING_PATH


def is_stale():
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > t for p in SOURCES + HEADERS)


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_binding(verbose=True))

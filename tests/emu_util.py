"""Builds and drives the host emulation of the HIP kernels (tests/emu): the same kernel
sources compiled with g++ -DWT_EMULATE under AddressSanitizer.  Test infrastructure."""
import os
import subprocess
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU_DIR = os.path.join(ROOT, "tests", "emu")
BUILD_DIR = os.path.join(EMU_DIR, "_build")
EXE = os.path.join(BUILD_DIR, "emu_driver")
SOURCES = [os.path.join(ROOT, "wtconv_amd", "csrc", "api.hip"), os.path.join(ROOT, "wtconv_amd", "csrc", "mfma2d.hip"),
           os.path.join(ROOT, "wtconv_amd", "csrc", "block.hip"), os.path.join(ROOT, "wtconv_amd", "csrc", "haar.hip"),
           os.path.join(EMU_DIR, "emu_driver.cpp")]
DEPS = SOURCES + [os.path.join(ROOT, "wtconv_amd", "csrc", f) for f in
                  ("common.h", "host_util.h", "kernels1d.h", "kernels1d_row.h", "kernels2d.h", "kernels2d_mfma.h", "kernels2d_mfma_wgrad.h",
                   "kernels2d_stream.h", "mfma2d.h", "plan.h", "kernels_block.h", "kernels_haar.h", "wgrad_finish.h")] + [
    os.path.join(EMU_DIR, "emu_runtime.h"), os.path.join(ROOT, "include", "wtconv_hip.h")]


def build(force=False):
    os.makedirs(BUILD_DIR, exist_ok=True)
    if not force and os.path.exists(EXE):
        newest = max(os.path.getmtime(p) for p in DEPS)
        if os.path.getmtime(EXE) >= newest:
            return EXE
    # -O0 -g1: the run time is dominated by thread creation, the build time by optimisation.  One object per source,
    # compiled side by side.
    flags = ["-std=c++20", "-O0", "-g1", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
             "-DWT_EMULATE", "-I" + EMU_DIR, "-pthread"]
    objs, procs = [], []
    for src in SOURCES:
        obj = os.path.join(BUILD_DIR, os.path.basename(src) + ".o")
        objs.append(obj)
        procs.append(subprocess.Popen(["g++", *flags, "-x", "c++", "-c", src, "-o", obj], cwd=ROOT))
    failed = [src for src, pr in zip(SOURCES, procs) if pr.wait() != 0]
    if failed:
        raise RuntimeError("emulation build failed for " + ", ".join(failed))
    subprocess.run(["g++", "-fsanitize=address,undefined", "-static-libasan", "-pthread", *objs, "-o", EXE], check=True,
                   cwd=ROOT)
    return EXE


def half_roundtrip(values):
    """float32 array -> the kernels' emulated float -> half -> float conversions of each element."""
    exe = build()
    v = np.ascontiguousarray(values, dtype=np.float32)
    hdr = np.array([0, v.size, 0, 0, 0, 0, 0, 0, 0, 0], dtype=np.int32)
    with tempfile.TemporaryDirectory() as td:
        fin, fout = os.path.join(td, "in.bin"), os.path.join(td, "out.bin")
        with open(fin, "wb") as f:
            f.write(hdr.tobytes() + v.tobytes())
        env = dict(os.environ)
        env["ASAN_OPTIONS"] = "detect_leaks=0"
        r = subprocess.run([exe, fin, fout], capture_output=True, text=True, timeout=120, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"emu_driver failed ({r.returncode}):\n{r.stderr[-4000:]}")
        return np.fromfile(fout, dtype=np.float32)


def run(dims, x, g, base_w, base_b, base_s, wt_ws, wt_ss, K, dtype=0, pdtype=0, timeout=600, lds_limit=None,
        mfma=None, fused_bwd=False):
    """All arrays float32 numpy.  2-D: x (B,C,H,W); 1-D: x (B,C,N).  Returns dict of float32 arrays.
    `lds_limit` (bytes) lowers the LDS budget of the dispatch, so that small planes take the
    level-by-level kernels that real runs only use for planes beyond 160 KB."""
    exe = build()
    if dims == 2:
        B, C, H, W = x.shape
        S, KK = 4, K * K
    else:
        B, C, W = x.shape
        H = 1
        S, KK = 2, K
    L = len(wt_ws)
    has_bias = base_b is not None
    hdr = np.array([dims, B, C, H, W, K, L, dtype, pdtype, int(has_bias)], dtype=np.int32)
    parts = [hdr.tobytes(), x.astype(np.float32).tobytes(), g.astype(np.float32).tobytes(),
             base_w.astype(np.float32).tobytes()]
    if has_bias:
        parts.append(base_b.astype(np.float32).tobytes())
    parts.append(base_s.astype(np.float32).tobytes())
    for w, s in zip(wt_ws, wt_ss):
        parts += [w.astype(np.float32).tobytes(), s.astype(np.float32).tobytes()]
    with tempfile.TemporaryDirectory() as td:
        fin, fout = os.path.join(td, "in.bin"), os.path.join(td, "out.bin")
        with open(fin, "wb") as f:
            f.write(b"".join(parts))
        env = dict(os.environ)
        env["ASAN_OPTIONS"] = "detect_leaks=0"
        env.pop("WT_EMU_LDS_LIMIT", None)
        if lds_limit is not None:
            env["WT_EMU_LDS_LIMIT"] = str(int(lds_limit))
        env.pop("WT_EMU_FUSED_BWD", None)
        if fused_bwd:         # the backward pass as the single call wtconv*_backward instead of its two halves
            env["WT_EMU_FUSED_BWD"] = "1"
        env.pop("WTCONV_MFMA", None)
        if mfma is not None:      # 0: vector-ALU kernels only; 1: matrix cores for bf16; 2: for bf16 and fp32
            env["WTCONV_MFMA"] = str(int(mfma))
        r = subprocess.run([exe, fin, fout], capture_output=True, text=True, timeout=timeout, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"emu_driver failed ({r.returncode}):\n{r.stderr[-4000:]}")
        raw = np.fromfile(fout, dtype=np.float32)
    P = x.size
    pos = 0

    def take(n, shape):
        nonlocal pos
        a = raw[pos:pos + n].reshape(shape)
        pos += n
        return a

    res = {"out": take(P, x.shape), "dx": take(P, x.shape), "dbase_w": take(C * KK, base_w.shape)}
    if has_bias:
        res["dbase_b"] = take(C, (C,))
    res["dbase_s"] = take(C, base_s.shape)
    res["dwt_ws"], res["dwt_ss"] = [], []
    for w, s in zip(wt_ws, wt_ss):
        res["dwt_ws"].append(take(w.size, w.shape))
        res["dwt_ss"].append(take(s.size, s.shape))
    assert pos == raw.size
    return res


def run_block(kind, a0, a1, p0, p1, dtype=0, pdtype=0, nhwc=1, timeout=600):
    """The block passes on the host.  kind = "norm": a0 = x (B,C,H,W), a1 = dy ((B,H,W,C) if nhwc else (B,C,H,W)),
    p0 = weight, p1 = bias; returns out, dx, dweight, dbias.  kind = "residual": a0 = y (B,H,W,C), a1 = shortcut
    (B,C,H,W), p0 = gamma, p1 = dout (B,C,H,W); returns out, dy, dgamma.  float32 numpy arrays."""
    exe = build()
    norm = kind == "norm"
    B, C, H, W = (a0.shape if norm else a1.shape)
    hdr = np.array([3 if norm else 4, B, C, H, W, int(nhwc), 0, dtype, pdtype, 0], dtype=np.int32)
    parts = [hdr.tobytes()] + [np.ascontiguousarray(a, dtype=np.float32).tobytes() for a in (a0, a1, p0, p1)]
    with tempfile.TemporaryDirectory() as td:
        fin, fout = os.path.join(td, "in.bin"), os.path.join(td, "out.bin")
        with open(fin, "wb") as f:
            f.write(b"".join(parts))
        env = dict(os.environ)
        env["ASAN_OPTIONS"] = "detect_leaks=0"
        r = subprocess.run([exe, fin, fout], capture_output=True, text=True, timeout=timeout, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"emu_driver failed ({r.returncode}):\n{r.stderr[-4000:]}")
        raw = np.fromfile(fout, dtype=np.float32)
    P = B * C * H * W
    if norm:
        oshape = (B, H, W, C) if nhwc else (B, C, H, W)
        return raw[:P].reshape(oshape), raw[P:2 * P].reshape(B, C, H, W), raw[2 * P:2 * P + C], raw[2 * P + C:]
    return raw[:P].reshape(B, C, H, W), raw[P:2 * P].reshape(B, H, W, C), raw[2 * P:]

"""Writes tests/golden/wtconv_vectors.npz: small input/output vectors of the WTConv layer.

The reference repository ships no golden vectors for this path, so these are produced by
the float64 brute-force loops in oracle/brute.py (which call no convolution routine and
are themselves cross-checked against the library restatement in tests/test_oracle.py).
They travel to the GPU box as plain data; run from the repository root:

    python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import brute  # noqa: E402

CASES_2D = {  # name: (B, C, H, W, K, L, bias)
    "2d_even": (1, 2, 8, 12, 3, 2, True),
    "2d_odd": (2, 2, 7, 9, 5, 3, True),
    "2d_nobias_k7": (1, 1, 10, 6, 7, 1, False),
}
CASES_1D = {  # name: (B, C, N, K, L, bias)
    "1d_even": (1, 2, 32, 5, 3, True),
    "1d_odd": (2, 1, 21, 3, 4, False),
}


def main():
    rng = np.random.default_rng(20240917)
    f = lambda *s: np.round(rng.standard_normal(s), 3)      # short decimals: exact in float32 text and bf16-friendly
    out = {}
    for name, (B, C, H, W, K, L, bias) in CASES_2D.items():
        x, g = f(B, C, H, W), f(B, C, H, W)
        p = dict(base_w=f(C, K, K) * 0.5, base_b=f(C) if bias else None, base_scale=f(C),
                 wt_ws=[f(C, 4, K, K) * 0.5 for _ in range(L)], wt_scales=[f(C, 4) for _ in range(L)])
        y = brute.wtconv2d_forward(x, **p)
        gr = brute.wtconv2d_backward(x, g, **p)
        out.update(_pack(name, x, g, p, y, gr, L))
    for name, (B, C, N, K, L, bias) in CASES_1D.items():
        x, g = f(B, C, N), f(B, C, N)
        p = dict(base_w=f(C, K) * 0.5, base_b=f(C) if bias else None, base_scale=f(C),
                 wt_ws=[f(C, 2, K) * 0.5 for _ in range(L)], wt_scales=[f(C, 2) for _ in range(L)])
        y = brute.wtconv1d_forward(x, **p)
        gr = brute.wtconv1d_backward(x, g, **p)
        out.update(_pack(name, x, g, p, y, gr, L))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "wtconv_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


def _pack(name, x, g, p, y, gr, L):
    d = {f"{name}/x": x, f"{name}/g": g, f"{name}/base_w": p["base_w"], f"{name}/base_scale": p["base_scale"],
         f"{name}/out": y, f"{name}/dx": gr["dx"], f"{name}/dbase_w": gr["dbase_w"],
         f"{name}/dbase_scale": gr["dbase_scale"], f"{name}/levels": np.array(L)}
    if p["base_b"] is not None:
        d[f"{name}/base_b"] = p["base_b"]
        d[f"{name}/dbase_b"] = gr["dbase_b"]
    for l in range(L):
        d[f"{name}/wt_w{l}"] = p["wt_ws"][l]
        d[f"{name}/wt_s{l}"] = p["wt_scales"][l]
        d[f"{name}/dwt_w{l}"] = gr["dwt_ws"][l]
        d[f"{name}/dwt_s{l}"] = gr["dwt_scales"][l]
    return d


if __name__ == "__main__":
    main()

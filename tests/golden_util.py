"""Loads tests/golden/wtconv_vectors.npz into torch tensors shaped like the module parameters."""
import os

import numpy as np
import torch

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "wtconv_vectors.npz")


def cases():
    z = np.load(PATH)          # allow_pickle defaults to False
    names = sorted({k.split("/")[0] for k in z.files})
    out = {}
    for n in names:
        d = {k.split("/", 1)[1]: z[k] for k in z.files if k.startswith(n + "/")}
        out[n] = d
    return out


def to_layer_tensors(d, dtype=torch.float64):
    """Returns dims, x, g, params (reference tensor layouts), expected dict."""
    L = int(d["levels"])
    dims = d["x"].ndim - 2
    S = 4 if dims == 2 else 2
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dtype)
    C = d["x"].shape[1]
    K = d["base_w"].shape[-1]
    kshape = (K, K) if dims == 2 else (K,)
    ones = (1,) * dims
    params = dict(
        base_w=t(d["base_w"]).reshape(C, 1, *kshape),
        base_b=t(d["base_b"]) if "base_b" in d else None,
        base_s=t(d["base_scale"]).reshape(1, C, *ones),
        wt_ws=[t(d[f"wt_w{l}"]).reshape(S * C, 1, *kshape) for l in range(L)],
        wt_ss=[t(d[f"wt_s{l}"]).reshape(1, S * C, *ones) for l in range(L)])
    exp = dict(out=t(d["out"]), dx=t(d["dx"]), dbase_w=t(d["dbase_w"]).reshape(C, 1, *kshape),
               dbase_s=t(d["dbase_scale"]).reshape(1, C, *ones),
               dbase_b=t(d["dbase_b"]) if "dbase_b" in d else None,
               dwt_ws=[t(d[f"dwt_w{l}"]).reshape(S * C, 1, *kshape) for l in range(L)],
               dwt_ss=[t(d[f"dwt_s{l}"]).reshape(1, S * C, *ones) for l in range(L)])
    return dims, t(d["x"]), t(d["g"]), params, exp

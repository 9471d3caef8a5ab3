"""Brute-force float64 loops for the WTConv layer (test infrastructure only).

Independent of ``oracle/wtconv_ref.py``: nothing here calls a convolution routine.
The forward follows the layer as the reference writes it (``wtconv/wtconv2d.py:38-87``,
``wtconv/wtconv1d.py:38-87``) using the 2x2 sub-band formulas quoted at
``fast_wtconv/cuda_haar/haar_common.cuh:4-15``; the backward is the hand-derived adjoint
(cross-check: ``fast_wtconv/cuda_haar/haar_cuda.py:168-197,379-424,650-676``).  Meant for
tiny shapes: it is O(P*K^2) pure Python/numpy.
"""
from __future__ import annotations

import numpy as np


# ---- 2-D Haar on one plane ------------------------------------------------------------
def haar2(p):
    """p (H,W), zero padded to even -> (4,h,w) in order LL,LH,HL,HH."""
    H, W = p.shape
    h, w = (H + 1) // 2, (W + 1) // 2
    q = np.zeros((2 * h, 2 * w))
    q[:H, :W] = p
    out = np.zeros((4, h, w))
    for i in range(h):
        for j in range(w):
            a, b, c, d = q[2 * i, 2 * j], q[2 * i, 2 * j + 1], q[2 * i + 1, 2 * j], q[2 * i + 1, 2 * j + 1]
            out[0, i, j] = (a + b + c + d) / 2
            out[1, i, j] = (a + b - c - d) / 2
            out[2, i, j] = (a - b + c - d) / 2
            out[3, i, j] = (a - b - c + d) / 2
    return out


def ihaar2(co, H, W):
    """co (4,h,w) -> (H,W): inverse transform cropped to H,W."""
    _, h, w = co.shape
    q = np.zeros((2 * h, 2 * w))
    for i in range(h):
        for j in range(w):
            ll, lh, hl, hh = co[:, i, j]
            q[2 * i, 2 * j] = (ll + lh + hl + hh) / 2
            q[2 * i, 2 * j + 1] = (ll + lh - hl - hh) / 2
            q[2 * i + 1, 2 * j] = (ll - lh + hl - hh) / 2
            q[2 * i + 1, 2 * j + 1] = (ll - lh - hl + hh) / 2
    return q[:H, :W]


def corr2(p, k):
    """'same' zero-padded cross-correlation of plane p (h,w) with k (K,K)."""
    K = k.shape[0]
    R = K // 2
    h, w = p.shape
    out = np.zeros((h, w))
    for i in range(h):
        for j in range(w):
            s = 0.0
            for a in range(K):
                for b in range(K):
                    y, x = i + a - R, j + b - R
                    if 0 <= y < h and 0 <= x < w:
                        s += k[a, b] * p[y, x]
            out[i, j] = s
    return out


def corr2_T(g, k):
    """Adjoint of corr2 with respect to its plane argument."""
    return corr2(g, k[::-1, ::-1])


def corr2_wgrad(g, p, K):
    """d/dk of <g, corr2(p,k)>: (K,K)."""
    R = K // 2
    h, w = p.shape
    out = np.zeros((K, K))
    for a in range(K):
        for b in range(K):
            s = 0.0
            for i in range(h):
                for j in range(w):
                    y, x = i + a - R, j + b - R
                    if 0 <= y < h and 0 <= x < w:
                        s += g[i, j] * p[y, x]
            out[a, b] = s
    return out


def wtconv2d_forward(x, base_w, base_b, base_scale, wt_ws, wt_scales):
    """x (B,C,H,W); base_w (C,K,K); base_b (C,) or None; base_scale (C,);
    wt_ws[l] (C,4,K,K); wt_scales[l] (C,4).  Returns out (B,C,H,W)."""
    B, C, H, W = x.shape
    L = len(wt_ws)
    out = np.zeros_like(x, dtype=np.float64)
    for b in range(B):
        for c in range(C):
            low = x[b, c].astype(np.float64)
            ys, shapes = [], []
            for l in range(L):
                shapes.append(low.shape)
                A = haar2(low)
                low = A[0]
                ys.append(np.stack([wt_scales[l][c, s] * corr2(A[s], wt_ws[l][c, s]) for s in range(4)]))
            z = None
            for l in range(L - 1, -1, -1):
                co = ys[l].copy()
                if z is not None:
                    co[0] += z
                z = ihaar2(co, *shapes[l])
            base = corr2(x[b, c].astype(np.float64), base_w[c])
            if base_b is not None:
                base = base + base_b[c]
            out[b, c] = base_scale[c] * base + z
    return out


def wtconv2d_backward(x, g, base_w, base_b, base_scale, wt_ws, wt_scales):
    """Adjoint of wtconv2d_forward.  Returns dict with dx, dbase_w, dbase_b, dbase_scale,
    dwt_ws[l], dwt_scales[l] in the same layouts as the arguments."""
    B, C, H, W = x.shape
    L = len(wt_ws)
    K = base_w.shape[-1]
    dx = np.zeros((B, C, H, W))
    dbw = np.zeros_like(base_w, dtype=np.float64)
    dbb = np.zeros(C)
    dbs = np.zeros(C)
    dws = [np.zeros_like(w, dtype=np.float64) for w in wt_ws]
    dss = [np.zeros_like(s, dtype=np.float64) for s in wt_scales]
    for b in range(B):
        for c in range(C):
            xp = x[b, c].astype(np.float64)
            gp = g[b, c].astype(np.float64)
            # forward pyramid of x (needed by the weight gradients)
            As, shapes = [], []
            low = xp
            for l in range(L):
                shapes.append(low.shape)
                A = haar2(low)
                As.append(A)
                low = A[0]
            # pyramid of the incoming gradient: dY_l = Haar(pad(dZ_l)), dZ_{l+1} = dY_l[0]
            dYs = []
            dz = gp
            for l in range(L):
                dY = haar2(dz)
                dYs.append(dY)
                dz = dY[0]
            # parameter gradients and dA_l
            dX = None                      # gradient flowing into the raw LL of level l
            for l in range(L - 1, -1, -1):
                dA = np.zeros_like(dYs[l])
                for s in range(4):
                    wfold = wt_scales[l][c, s] * wt_ws[l][c, s]
                    dA[s] = corr2_T(dYs[l][s], wfold)
                    dWt = corr2_wgrad(dYs[l][s], As[l][s], K)
                    dws[l][c, s] += wt_scales[l][c, s] * dWt
                    dss[l][c, s] += np.sum(wt_ws[l][c, s] * dWt)
                if dX is not None:
                    dA[0] += dX
                dX = ihaar2(dA, *shapes[l])
            dWb = corr2_wgrad(gp, xp, K)
            sg = gp.sum()
            dbw[c] += base_scale[c] * dWb
            dbs[c] += np.sum(base_w[c] * dWb) + (base_b[c] * sg if base_b is not None else 0.0)
            dbb[c] += base_scale[c] * sg
            dx[b, c] = dX + corr2_T(gp, base_scale[c] * base_w[c])
    return dict(dx=dx, dbase_w=dbw, dbase_b=dbb if base_b is not None else None,
                dbase_scale=dbs, dwt_ws=dws, dwt_scales=dss)


# ---- 1-D ------------------------------------------------------------------------------
_R2 = 0.7071067811865476


def haar1(v):
    n = v.shape[0]
    m = (n + 1) // 2
    q = np.zeros(2 * m)
    q[:n] = v
    out = np.zeros((2, m))
    for i in range(m):
        out[0, i] = (q[2 * i] + q[2 * i + 1]) * _R2
        out[1, i] = (q[2 * i] - q[2 * i + 1]) * _R2
    return out


def ihaar1(co, n):
    m = co.shape[1]
    q = np.zeros(2 * m)
    for i in range(m):
        q[2 * i] = (co[0, i] + co[1, i]) * _R2
        q[2 * i + 1] = (co[0, i] - co[1, i]) * _R2
    return q[:n]


def corr1(v, k):
    K = k.shape[0]
    R = K // 2
    n = v.shape[0]
    out = np.zeros(n)
    for i in range(n):
        s = 0.0
        for a in range(K):
            y = i + a - R
            if 0 <= y < n:
                s += k[a] * v[y]
        out[i] = s
    return out


def corr1_wgrad(g, v, K):
    R = K // 2
    n = v.shape[0]
    out = np.zeros(K)
    for a in range(K):
        s = 0.0
        for i in range(n):
            y = i + a - R
            if 0 <= y < n:
                s += g[i] * v[y]
        out[a] = s
    return out


def wtconv1d_forward(x, base_w, base_b, base_scale, wt_ws, wt_scales):
    """x (B,C,N); base_w (C,K); wt_ws[l] (C,2,K); wt_scales[l] (C,2)."""
    B, C, N = x.shape
    L = len(wt_ws)
    out = np.zeros((B, C, N))
    for b in range(B):
        for c in range(C):
            low = x[b, c].astype(np.float64)
            ys, ns = [], []
            for l in range(L):
                ns.append(low.shape[0])
                A = haar1(low)
                low = A[0]
                ys.append(np.stack([wt_scales[l][c, s] * corr1(A[s], wt_ws[l][c, s]) for s in range(2)]))
            z = None
            for l in range(L - 1, -1, -1):
                co = ys[l].copy()
                if z is not None:
                    co[0] += z
                z = ihaar1(co, ns[l])
            base = corr1(x[b, c].astype(np.float64), base_w[c])
            if base_b is not None:
                base = base + base_b[c]
            out[b, c] = base_scale[c] * base + z
    return out


def wtconv1d_backward(x, g, base_w, base_b, base_scale, wt_ws, wt_scales):
    B, C, N = x.shape
    L = len(wt_ws)
    K = base_w.shape[-1]
    dx = np.zeros((B, C, N))
    dbw = np.zeros_like(base_w, dtype=np.float64)
    dbb = np.zeros(C)
    dbs = np.zeros(C)
    dws = [np.zeros_like(w, dtype=np.float64) for w in wt_ws]
    dss = [np.zeros_like(s, dtype=np.float64) for s in wt_scales]
    for b in range(B):
        for c in range(C):
            xp = x[b, c].astype(np.float64)
            gp = g[b, c].astype(np.float64)
            As, ns = [], []
            low = xp
            for l in range(L):
                ns.append(low.shape[0])
                A = haar1(low)
                As.append(A)
                low = A[0]
            dYs = []
            dz = gp
            for l in range(L):
                dY = haar1(dz)
                dYs.append(dY)
                dz = dY[0]
            dX = None
            for l in range(L - 1, -1, -1):
                dA = np.zeros_like(dYs[l])
                for s in range(2):
                    wfold = wt_scales[l][c, s] * wt_ws[l][c, s]
                    dA[s] = corr1(dYs[l][s], wfold[::-1])
                    dWt = corr1_wgrad(dYs[l][s], As[l][s], K)
                    dws[l][c, s] += wt_scales[l][c, s] * dWt
                    dss[l][c, s] += np.sum(wt_ws[l][c, s] * dWt)
                if dX is not None:
                    dA[0] += dX
                dX = ihaar1(dA, ns[l])
            dWb = corr1_wgrad(gp, xp, K)
            sg = gp.sum()
            dbw[c] += base_scale[c] * dWb
            dbs[c] += np.sum(base_w[c] * dWb) + (base_b[c] * sg if base_b is not None else 0.0)
            dbb[c] += base_scale[c] * sg
            dx[b, c] = dX + corr1(gp, (base_scale[c] * base_w[c])[::-1])
    return dict(dx=dx, dbase_w=dbw, dbase_b=dbb if base_b is not None else None,
                dbase_scale=dbs, dwt_ws=dws, dwt_scales=dss)

"""Pins the CPU oracle (oracle/wtconv_ref.py) without the reference's code: closed forms,
invariants, an independent brute-force restatement, special cases that collapse to
library routines, and float64 gradcheck."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute
from oracle import wtconv_ref as R

torch.set_num_threads(4)


def _rand_params2d(C, K, L, dtype=torch.float64, bias=True, seed=0):
    g = torch.Generator().manual_seed(seed)
    base_w = torch.randn(C, 1, K, K, generator=g, dtype=dtype) * 0.3
    base_b = torch.randn(C, generator=g, dtype=dtype) if bias else None
    base_s = torch.randn(1, C, 1, 1, generator=g, dtype=dtype)
    ws = [torch.randn(4 * C, 1, K, K, generator=g, dtype=dtype) * 0.3 for _ in range(L)]
    ss = [torch.randn(1, 4 * C, 1, 1, generator=g, dtype=dtype) for _ in range(L)]
    return base_w, base_b, base_s, ws, ss


def _rand_params1d(C, K, L, dtype=torch.float64, bias=True, seed=0):
    g = torch.Generator().manual_seed(seed)
    base_w = torch.randn(C, 1, K, generator=g, dtype=dtype) * 0.3
    base_b = torch.randn(C, generator=g, dtype=dtype) if bias else None
    base_s = torch.randn(1, C, 1, generator=g, dtype=dtype)
    ws = [torch.randn(2 * C, 1, K, generator=g, dtype=dtype) * 0.3 for _ in range(L)]
    ss = [torch.randn(1, 2 * C, 1, generator=g, dtype=dtype) for _ in range(L)]
    return base_w, base_b, base_s, ws, ss


# ---------------------------------------------------------------- transforms
def test_subband_closed_form_2d():
    x = torch.randn(2, 3, 6, 8, dtype=torch.float64)
    dec, _ = R.haar_filters_2d(3, torch.float64)
    co = R.analysis_2d(x, dec)
    a, b = x[..., 0::2, 0::2], x[..., 0::2, 1::2]
    c, d = x[..., 1::2, 0::2], x[..., 1::2, 1::2]
    torch.testing.assert_close(co[:, :, 0], (a + b + c + d) / 2)
    torch.testing.assert_close(co[:, :, 1], (a + b - c - d) / 2)
    torch.testing.assert_close(co[:, :, 2], (a - b + c - d) / 2)
    torch.testing.assert_close(co[:, :, 3], (a - b - c + d) / 2)


def test_subband_closed_form_1d():
    x = torch.randn(2, 3, 10, dtype=torch.float64)
    dec, _ = R.haar_filters_1d(3, torch.float64)
    co = R.analysis_1d(x, dec)
    r = 2 ** -0.5
    torch.testing.assert_close(co[:, :, 0], (x[..., 0::2] + x[..., 1::2]) * r)
    torch.testing.assert_close(co[:, :, 1], (x[..., 0::2] - x[..., 1::2]) * r)


def test_fp32_tap_is_rounded_product():
    dec, rec = R.haar_filters_2d(1, torch.float32)
    r = torch.tensor(0.7071067811865476, dtype=torch.float32)
    assert dec[0, 0, 0, 0].item() == (r * r).item()
    assert torch.equal(dec.abs(), rec.abs())
    assert torch.equal(dec, rec)          # db1: synthesis bank equals analysis bank


def test_perfect_reconstruction_and_parseval():
    x = torch.randn(2, 4, 12, 10, dtype=torch.float64)
    dec, rec = R.haar_filters_2d(4, torch.float64)
    co = R.analysis_2d(x, dec)
    torch.testing.assert_close(R.synthesis_2d(co, rec), x)
    torch.testing.assert_close(co.pow(2).sum(), x.pow(2).sum())
    x1 = torch.randn(2, 4, 14, dtype=torch.float64)
    d1, r1 = R.haar_filters_1d(4, torch.float64)
    c1 = R.analysis_1d(x1, d1)
    torch.testing.assert_close(R.synthesis_1d(c1, r1), x1)
    torch.testing.assert_close(c1.pow(2).sum(), x1.pow(2).sum())


def test_pad_analysis_is_adjoint_of_synthesis_crop():
    H, W = 7, 9
    dec, rec = R.haar_filters_2d(2, torch.float64)
    x = torch.randn(1, 2, H, W, dtype=torch.float64)
    co = torch.randn(1, 2, 4, 4, 5, dtype=torch.float64)
    lhs = (R.analysis_2d(F.pad(x, (0, 1, 0, 1)), dec) * co).sum()
    rhs = (x * R.synthesis_2d(co, rec)[:, :, :H, :W]).sum()
    torch.testing.assert_close(lhs, rhs)


# ---------------------------------------------------------------- brute force vs library restatement
@pytest.mark.parametrize("shape,K,L,bias", [
    ((1, 2, 6, 7), 3, 2, True),
    ((2, 1, 7, 10), 5, 3, True),
    ((1, 2, 8, 8), 5, 2, False),
    ((1, 1, 5, 3), 3, 3, True),
    ((1, 1, 9, 12), 1, 2, True),
])
def test_forward_backward_2d_vs_brute(shape, K, L, bias):
    B, C, H, W = shape
    bw, bb, bs, ws, ss = _rand_params2d(C, K, L, bias=bias)
    x = torch.randn(*shape, dtype=torch.float64)
    g = torch.randn(*shape, dtype=torch.float64)
    leaves = [x, bw, bs] + ws + ss + ([bb] if bias else [])
    for t in leaves:
        t.requires_grad_(True)
    out = R.wtconv2d_ref(x, bw, bb, bs, ws, ss)
    out.backward(g)

    npar = dict(
        base_w=bw.detach().numpy().reshape(C, K, K),
        base_b=bb.detach().numpy() if bias else None,
        base_scale=bs.detach().numpy().reshape(C),
        wt_ws=[w.detach().numpy().reshape(C, 4, K, K) for w in ws],
        wt_scales=[s.detach().numpy().reshape(C, 4) for s in ss])
    ref_out = brute.wtconv2d_forward(x.detach().numpy(), **npar)
    np.testing.assert_allclose(out.detach().numpy(), ref_out, rtol=1e-11, atol=1e-11)
    gr = brute.wtconv2d_backward(x.detach().numpy(), g.numpy(), **npar)
    np.testing.assert_allclose(x.grad.numpy(), gr["dx"], rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(bw.grad.numpy().reshape(C, K, K), gr["dbase_w"], rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(bs.grad.numpy().reshape(C), gr["dbase_scale"], rtol=1e-10, atol=1e-10)
    if bias:
        np.testing.assert_allclose(bb.grad.numpy(), gr["dbase_b"], rtol=1e-10, atol=1e-10)
    for l in range(L):
        np.testing.assert_allclose(ws[l].grad.numpy().reshape(C, 4, K, K), gr["dwt_ws"][l], rtol=1e-10, atol=1e-10)
        np.testing.assert_allclose(ss[l].grad.numpy().reshape(C, 4), gr["dwt_scales"][l], rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("shape,K,L,bias", [
    ((2, 2, 13), 3, 2, True),
    ((1, 3, 32), 5, 4, True),
    ((1, 1, 9), 5, 3, False),
])
def test_forward_backward_1d_vs_brute(shape, K, L, bias):
    B, C, N = shape
    bw, bb, bs, ws, ss = _rand_params1d(C, K, L, bias=bias)
    x = torch.randn(*shape, dtype=torch.float64)
    g = torch.randn(*shape, dtype=torch.float64)
    leaves = [x, bw, bs] + ws + ss + ([bb] if bias else [])
    for t in leaves:
        t.requires_grad_(True)
    out = R.wtconv1d_ref(x, bw, bb, bs, ws, ss)
    out.backward(g)
    npar = dict(
        base_w=bw.detach().numpy().reshape(C, K),
        base_b=bb.detach().numpy() if bias else None,
        base_scale=bs.detach().numpy().reshape(C),
        wt_ws=[w.detach().numpy().reshape(C, 2, K) for w in ws],
        wt_scales=[s.detach().numpy().reshape(C, 2) for s in ss])
    np.testing.assert_allclose(out.detach().numpy(), brute.wtconv1d_forward(x.detach().numpy(), **npar),
                               rtol=1e-11, atol=1e-11)
    gr = brute.wtconv1d_backward(x.detach().numpy(), g.numpy(), **npar)
    np.testing.assert_allclose(x.grad.numpy(), gr["dx"], rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(bw.grad.numpy().reshape(C, K), gr["dbase_w"], rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(bs.grad.numpy().reshape(C), gr["dbase_scale"], rtol=1e-10, atol=1e-10)
    if bias:
        np.testing.assert_allclose(bb.grad.numpy(), gr["dbase_b"], rtol=1e-10, atol=1e-10)
    for l in range(L):
        np.testing.assert_allclose(ws[l].grad.numpy().reshape(C, 2, K), gr["dwt_ws"][l], rtol=1e-10, atol=1e-10)
        np.testing.assert_allclose(ss[l].grad.numpy().reshape(C, 2), gr["dwt_scales"][l], rtol=1e-10, atol=1e-10)


# ---------------------------------------------------------------- special cases
def test_zero_wavelet_scales_leaves_scaled_base_conv():
    C, K, L = 3, 5, 3
    bw, bb, bs, ws, ss = _rand_params2d(C, K, L)
    ss = [torch.zeros_like(s) for s in ss]
    x = torch.randn(2, C, 9, 11, dtype=torch.float64)
    out = R.wtconv2d_ref(x, bw, bb, bs, ws, ss)
    want = bs * F.conv2d(x, bw, bb, padding=K // 2, groups=C)
    torch.testing.assert_close(out, want)


def test_delta_kernels_give_block_mean_pyramid():
    """Centre-tap wavelet kernels with unit scales and a zero base conv: level l adds
    the 2^(l-1) block mean of x (upsampled), and level 1 returns x itself."""
    C, K, L = 2, 5, 3
    x = torch.randn(2, C, 16, 24, dtype=torch.float64)
    delta = torch.zeros(4 * C, 1, K, K, dtype=torch.float64)
    delta[:, 0, K // 2, K // 2] = 1
    ws = [delta.clone() for _ in range(L)]
    ss = [torch.ones(1, 4 * C, 1, 1, dtype=torch.float64) for _ in range(L)]
    bw = torch.zeros(C, 1, K, K, dtype=torch.float64)
    bs = torch.ones(1, C, 1, 1, dtype=torch.float64)
    out = R.wtconv2d_ref(x, bw, None, bs, ws, ss)
    want = x.clone()
    for l in range(1, L):
        f = 2 ** l
        want = want + F.interpolate(F.avg_pool2d(x, f), scale_factor=f, mode="nearest")
    torch.testing.assert_close(out, want)


def test_bias_only_response_and_linearity():
    C, K, L = 2, 3, 2
    bw, bb, bs, ws, ss = _rand_params2d(C, K, L)
    z = torch.zeros(1, C, 7, 6, dtype=torch.float64)
    out0 = R.wtconv2d_ref(z, bw, bb, bs, ws, ss)
    torch.testing.assert_close(out0, (bs * bb.view(1, C, 1, 1)).expand_as(out0))
    x1, x2 = torch.randn(2, 1, C, 7, 6, dtype=torch.float64)
    f = lambda t: R.wtconv2d_ref(t, bw, None, bs, ws, ss)
    torch.testing.assert_close(f(2 * x1 - 3 * x2), 2 * f(x1) - 3 * f(x2))


def test_constant_input_even_plane_without_conv_padding():
    """K=1 has no boundary effect: constant input v, constant kernels -> closed form.
    LL of a constant plane at level l is v*2^l; all detail bands vanish."""
    C, L, v = 1, 3, 1.7
    x = torch.full((1, C, 8, 8), v, dtype=torch.float64)
    wl = [0.3, -0.8, 1.1]
    ws = [torch.full((4 * C, 1, 1, 1), w, dtype=torch.float64) for w in wl]
    ss = [torch.full((1, 4 * C, 1, 1), 0.5, dtype=torch.float64) for _ in range(L)]
    bw = torch.full((C, 1, 1, 1), 2.0, dtype=torch.float64)
    bs = torch.full((1, C, 1, 1), 0.25, dtype=torch.float64)
    bb = torch.tensor([0.4], dtype=torch.float64)
    out = R.wtconv2d_ref(x, bw, bb, bs, ws, ss)
    # each level contributes 0.5*w_l * v (the 2^l gain of analysis is undone by synthesis)
    want = 0.25 * (2.0 * v + 0.4) + sum(0.5 * w * v for w in wl)
    torch.testing.assert_close(out, torch.full_like(out, want))


def test_adjoint_identity_2d():
    C, K, L = 2, 5, 3
    bw, _, bs, ws, ss = _rand_params2d(C, K, L)
    x = torch.randn(1, C, 11, 7, dtype=torch.float64, requires_grad=True)
    g = torch.randn(1, C, 11, 7, dtype=torch.float64)
    out = R.wtconv2d_ref(x, bw, None, bs, ws, ss)
    (gx,) = torch.autograd.grad(out, x, g)
    # the bias-free map is linear: f^T(g) equals f run with 180-degree rotated kernels
    flip = lambda w: torch.flip(w, dims=(-1, -2))
    gx2 = R.wtconv2d_ref(g, flip(bw), None, bs, [flip(w) for w in ws], ss)
    torch.testing.assert_close(gx, gx2)


def test_adjoint_identity_1d():
    C, K, L = 2, 5, 3
    bw, _, bs, ws, ss = _rand_params1d(C, K, L)
    x = torch.randn(1, C, 21, dtype=torch.float64, requires_grad=True)
    g = torch.randn(1, C, 21, dtype=torch.float64)
    out = R.wtconv1d_ref(x, bw, None, bs, ws, ss)
    (gx,) = torch.autograd.grad(out, x, g)
    flip = lambda w: torch.flip(w, dims=(-1,))
    gx2 = R.wtconv1d_ref(g, flip(bw), None, bs, [flip(w) for w in ws], ss)
    torch.testing.assert_close(gx, gx2)


def test_gradcheck_fp64():
    C, K, L = 1, 3, 2
    bw, bb, bs, ws, ss = _rand_params2d(C, K, L)
    x = torch.randn(1, C, 5, 6, dtype=torch.float64)
    ins = [x, bw, bb, bs, ws[0], ws[1], ss[0], ss[1]]
    for t in ins:
        t.requires_grad_(True)
    fn = lambda x, bw, bb, bs, w0, w1, s0, s1: R.wtconv2d_ref(x, bw, bb, bs, [w0, w1], [s0, s1])
    assert torch.autograd.gradcheck(fn, ins, eps=1e-6, atol=1e-6)


# ---------------------------------------------------------------- shapes, stride, init
def test_shape_chain_and_odd_sizes():
    assert R.level_shapes(7, 7, 2) == [(7, 7), (4, 4), (2, 2)]
    assert R.level_shapes(28, 28, 3) == [(28, 28), (14, 14), (7, 7), (4, 4)]
    m = R.RefWTConv2d(3, 3, 5, wt_levels=2)
    assert m(torch.randn(2, 3, 7, 7)).shape == (2, 3, 7, 7)
    m1 = R.RefWTConv1d(3, 3, 5, wt_levels=3)
    assert m1(torch.randn(2, 3, 37)).shape == (2, 3, 37)


def test_stride_semantics():
    m = R.RefWTConv2d(2, 2, 3, stride=2, wt_levels=2)
    x = torch.randn(1, 2, 9, 10)
    full = R.wtconv2d_ref(x, m.base_conv.weight, m.base_conv.bias, m.base_scale.weight,
                          [c.weight for c in m.wavelet_convs], [s.weight for s in m.wavelet_scale])
    torch.testing.assert_close(m(x), full[:, :, ::2, ::2])        # sub-sampling in 2-D
    m1 = R.RefWTConv1d(2, 2, 3, stride=2, wt_levels=2)
    x1 = torch.randn(1, 2, 11)
    full1 = R.wtconv1d_ref(x1, m1.base_conv.weight, m1.base_conv.bias, m1.base_scale.weight,
                           [c.weight for c in m1.wavelet_convs], [s.weight for s in m1.wavelet_scale])
    torch.testing.assert_close(m1(x1), (full1[:, :, 0:10:2] + full1[:, :, 1:10:2]) / 2)  # true mean in 1-D


def test_seeded_default_init_draw_order():
    """Parameters are drawn base conv first, then the level convs in order, each with
    nn.Conv2d's default initialisation; the scales are the constants 1.0 and 0.1."""
    C, K, L = 4, 5, 2
    torch.manual_seed(0)
    m = R.RefWTConv2d(C, C, K, wt_levels=L)
    torch.manual_seed(0)
    base = torch.nn.Conv2d(C, C, K, padding='same', groups=C, bias=True)
    lv = [torch.nn.Conv2d(4 * C, 4 * C, K, padding='same', groups=4 * C, bias=False) for _ in range(L)]
    assert torch.equal(m.base_conv.weight, base.weight) and torch.equal(m.base_conv.bias, base.bias)
    for i in range(L):
        assert torch.equal(m.wavelet_convs[i].weight, lv[i].weight)
        assert torch.all(m.wavelet_scale[i].weight == 0.1)
    assert torch.all(m.base_scale.weight == 1.0)
    n_params = sum(p.numel() for p in m.parameters())
    assert n_params == (59 + 104 * L) * C            # includes the two frozen filter banks
    keys = set(m.state_dict().keys())
    assert {"base_conv.weight", "base_conv.bias", "base_scale.weight", "wavelet_convs.0.weight",
            "wavelet_scale.1.weight", "wt_filter", "iwt_filter"} <= keys


def _block_mean_zero_padded(t):
    """B(t)[i, j] = (sum of the 2 x 2 block of t zero-padded to even sizes) / 4, written out with
    loops (no conv, no padding helper): the hand-made side of the odd-size check below."""
    H, W = t.shape
    h, w = (H + 1) // 2, (W + 1) // 2
    out = torch.zeros(h, w, dtype=t.dtype)
    for i in range(h):
        for j in range(w):
            s = 0.0
            for a in (0, 1):
                for b in (0, 1):
                    y, x = 2 * i + a, 2 * j + b
                    if y < H and x < W:          # positions beyond the plane are the zero padding
                        s = s + t[y, x]
            out[i, j] = s / 4
    return out


def _upsample_crop(t, H, W):
    """U(t): every value repeated over its 2 x 2 block, cropped to H x W (loops)."""
    out = torch.zeros(H, W, dtype=t.dtype)
    for y in range(H):
        for x in range(W):
            out[y, x] = t[y // 2, x // 2]
    return out


@pytest.mark.parametrize("H,W,L", [(5, 7, 2), (6, 10, 3), (7, 7, 3), (9, 4, 2)])
def test_delta_kernels_odd_sizes_closed_form(H, W, L):
    """Odd sizes pin the pad side (right/bottom), the per-level padding and the crop of the whole
    layer: with centre-tap wavelet kernels, unit scales and no base conv the layer is
        out = x + U(B x) + U U(B B x) + ...   (L - 1 terms)
    where B is the mean over 2 x 2 blocks of the zero-padded plane and U repeats and crops
    (reference wtconv2d.py:49-51,66-76).  (6, 10, 3) has an odd level-2 grid (3 x 5), (7, 7, 3) is odd
    at levels 1 and 3, (9, 4, 2) mixes an odd and an even side."""
    C, K = 2, 3
    ref = R.RefWTConv2d(C, C, K, wt_levels=L, bias=True).double()
    with torch.no_grad():
        ref.base_conv.weight.zero_()
        ref.base_conv.bias.zero_()
        for conv, sc in zip(ref.wavelet_convs, ref.wavelet_scale):
            conv.weight.zero_()
            conv.weight[:, 0, K // 2, K // 2] = 1.0
            sc.weight.fill_(1.0)
    x = torch.randn(1, C, H, W, dtype=torch.float64)
    got = ref(x)
    for c in range(C):
        want = x[0, c].clone()
        level = x[0, c]
        shapes = []
        for _ in range(L - 1):
            shapes.append(level.shape)
            level = _block_mean_zero_padded(level)
            term = level
            for (h, w) in reversed(shapes):
                term = _upsample_crop(term, h, w)
            want = want + term
        torch.testing.assert_close(got[0, c], want, rtol=1e-12, atol=1e-12)


def test_seeded_default_init_draw_order_1d():
    """The 1-D layer draws like its 2-D twin: base Conv1d (weight, then bias), then the level convs
    in order (wtconv1d.py:23-31), against a plain nn.Conv1d sequence under the same seed."""
    C, K, L = 3, 5, 3
    torch.manual_seed(0)
    m = R.RefWTConv1d(C, C, K, wt_levels=L)
    torch.manual_seed(0)
    base = torch.nn.Conv1d(C, C, K, padding='same', groups=C, bias=True)
    lv = [torch.nn.Conv1d(2 * C, 2 * C, K, padding='same', groups=2 * C, bias=False) for _ in range(L)]
    assert torch.equal(m.base_conv.weight, base.weight) and torch.equal(m.base_conv.bias, base.bias)
    for i in range(L):
        assert torch.equal(m.wavelet_convs[i].weight, lv[i].weight)
        assert torch.all(m.wavelet_scale[i].weight == 0.1)
    assert torch.all(m.base_scale.weight == 1.0)
    from wtconv.wtconv1d import WTConv1d
    torch.manual_seed(0)
    p = WTConv1d(C, C, K, wt_levels=L)            # the product module draws the same numbers
    assert torch.equal(p.base_conv.weight, base.weight) and torch.equal(p.base_conv.bias, base.bias)
    for i in range(L):
        assert torch.equal(p.wavelet_convs[i].weight, lv[i].weight)

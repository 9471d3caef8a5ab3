"""Runs the HIP kernel sources on the host (g++ -DWT_EMULATE, AddressSanitizer + UBSan,
one std::thread per GPU thread) through the same C ABI and checks them against the
oracle.  This exercises the kernels' indexing, halo/padding/crop logic and reductions
without a GPU; the arithmetic on the GPU itself is covered by the -m gpu tests."""
import numpy as np
import pytest
import torch

import emu_util
from oracle import wtconv_ref as R


def _bf16_round(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).to(torch.float32).numpy()


def _f16_round(a):
    return np.ascontiguousarray(a).astype(np.float16).astype(np.float32)


def _case2d(B, C, H, W, K, L, bias, dtype=0, pdtype=0, seed=0):
    rng = np.random.default_rng(seed)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    x, g = f(B, C, H, W), f(B, C, H, W)
    bw, bb, bs = f(C, 1, K, K) * 0.3, (f(C) if bias else None), f(1, C, 1, 1)
    ws = [f(4 * C, 1, K, K) * 0.3 for _ in range(L)]
    ss = [f(1, 4 * C, 1, 1) for _ in range(L)]
    if dtype:
        rd = _f16_round if dtype == 2 else _bf16_round
        x, g = rd(x), rd(g)
    if pdtype:
        rd = _f16_round if pdtype == 2 else _bf16_round
        bw, bs = rd(bw), rd(bs)
        bb = rd(bb) if bias else None
        ws, ss = [rd(w) for w in ws], [rd(s) for s in ss]
    return x, g, bw, bb, bs, ws, ss


def _oracle(dims, x, g, bw, bb, bs, ws, ss):
    t = lambda a: torch.from_numpy(a).double().requires_grad_(True)
    tx, tbw, tbs = t(x), t(bw), t(bs)
    tbb = t(bb) if bb is not None else None
    tws, tss = [t(w) for w in ws], [t(s) for s in ss]
    fn = R.wtconv2d_ref if dims == 2 else R.wtconv1d_ref
    out = fn(tx, tbw, tbb, tbs, tws, tss)
    out.backward(torch.from_numpy(g).double())
    res = {"out": out.detach().numpy(), "dx": tx.grad.numpy(), "dbase_w": tbw.grad.numpy(),
           "dbase_s": tbs.grad.numpy(), "dwt_ws": [w.grad.numpy() for w in tws],
           "dwt_ss": [s.grad.numpy() for s in tss]}
    if bb is not None:
        res["dbase_b"] = tbb.grad.numpy()
    return res


def _compare(got, want, rtol, atol_scale, act_tol=None):
    """`act_tol`: its own (rtol, atol_scale) for the two activation-typed results, out and dx."""
    def chk(a, b, name, rt=rtol, at=atol_scale):
        scale = max(float(np.sqrt(np.mean(b.astype(np.float64) ** 2))), 1e-6)
        np.testing.assert_allclose(a, b, rtol=rt, atol=at * scale, err_msg=name)
    for k in ("out", "dx"):
        chk(got[k], want[k], k, *(act_tol or (rtol, atol_scale)))
    for k in ("dbase_w", "dbase_s"):
        chk(got[k], want[k], k)
    if "dbase_b" in want:
        chk(got["dbase_b"], want["dbase_b"], "dbase_b")
    for l, (a, b) in enumerate(zip(got["dwt_ws"], want["dwt_ws"])):
        chk(a, b, f"dwt_w[{l}]")
    for l, (a, b) in enumerate(zip(got["dwt_ss"], want["dwt_ss"])):
        chk(a, b, f"dwt_s[{l}]")


@pytest.fixture(scope="module", autouse=True)
def _built():
    emu_util.build()


@pytest.mark.parametrize("B,C,H,W,K,L,bias", [
    (2, 2, 8, 8, 3, 2, True),       # even sizes, 128-bit load path
    (1, 2, 7, 7, 5, 2, True),       # odd at level 1 (7 -> 4 -> 2), scalar load path
    (1, 1, 14, 14, 5, 2, False),    # odd at level 2, no bias
    (1, 2, 9, 13, 3, 3, True),      # odd everywhere, H != W
    (1, 1, 12, 20, 7, 1, True),     # K = 7, single level
    (2, 1, 6, 10, 1, 2, True),      # K = 1 (no conv halo)
    (1, 1, 28, 28, 5, 5, True),     # five levels: 28 14 7 4 2 1
    (5, 3, 7, 7, 5, 2, True),       # several small planes per workgroup / per wave, ragged batch tail
    (3, 2, 14, 14, 3, 2, True),     # 16 threads per plane, stacked planes in the weight-gradient kernel
])
def test_emulated_2d_fp32(B, C, H, W, K, L, bias):
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, bias)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-5, atol_scale=2e-5)


# The level-by-level kernels for pyramids larger than LDS, reached here with small planes by
# lowering the dispatch's LDS budget (real runs take them from about 100 x 100 pixels on).
@pytest.mark.parametrize("B,C,H,W,K,L,bias,limit", [
    (1, 1, 21, 37, 5, 3, True, 1024),    # odd sizes at levels 1-3: scalar tile staging, ragged tiles
    (2, 1, 24, 48, 5, 2, True, 1024),    # widths 48/24/12: 16-byte tile staging and stores; batch-tile chunks
    (1, 1, 20, 136, 3, 2, False, 1024),  # three column tiles at level 0, two at level 1, no bias
    (1, 1, 18, 24, 7, 1, True, 1024),    # K = 7 halo of 3
    (1, 1, 36, 36, 3, 2, False, 12000),  # plane-resident forward, level-by-level weight gradients
])
def test_emulated_2d_level_by_level(B, C, H, W, K, L, bias, limit):
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, bias)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K, lds_limit=limit)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-5, atol_scale=2e-5)


@pytest.mark.parametrize("B,C,H,W,K,L,bias,limit,dtype", [
    (1, 2, 21, 37, 5, 3, True, 1024, 0),     # both passes level by level: one pyramid of grad_out serves both
    (1, 1, 24, 48, 3, 2, False, 1024, 2),    # the same on fp16 tensors
    (1, 1, 18, 24, 7, 1, True, 1024, 0),     # a single level: nothing to share, the two passes run as they are
    (1, 1, 36, 36, 3, 2, False, 12000, 0),   # plane-resident input gradient, level-by-level weight gradients: not shared
    (2, 3, 14, 14, 5, 2, True, None, 0),     # plane-resident both: the plain sequence of the two passes
])
def test_emulated_2d_fused_backward(B, C, H, W, K, L, bias, limit, dtype):
    """wtconv2d_backward as one call, against the oracle (and so against the two separate passes)."""
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, bias, dtype=dtype)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K, dtype=dtype, lds_limit=limit, fused_bwd=True)
    act = (1e-3, 1e-3) if dtype == 2 else None
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-5, atol_scale=2e-5, act_tol=act)


# A single tiny plane: the pyramids take less LDS than the final reduction of the
# weight-gradient kernel ([8 waves][sets * K * K + 1] floats), which the plan must cover.
@pytest.mark.parametrize("B,C,H,W,K,L", [
    (1, 1, 1, 1, 7, 4), (1, 1, 2, 2, 7, 5), (1, 1, 4, 4, 7, 2), (1, 1, 1, 1, 7, 1), (1, 1, 1, 1, 5, 2),
])
def test_emulated_2d_tiny_plane_reduction_fits_lds(B, C, H, W, K, L):
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, True)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-5, atol_scale=2e-5)


# The matrix-core (MFMA) kernels: bf16 tensors take them by default; mfma=2 sends fp32 tensors
# through them as three bf16 split planes, which must hold the fp32 bar.  The emulation computes
# each MFMA from the operands the 64 lanes of a wave hold, in the hardware's register layout.
@pytest.mark.parametrize("B,C,H,W,K,L,bias", [
    (2, 2, 8, 8, 3, 2, True),       # vector loads, two planes per unit
    (1, 2, 7, 7, 5, 2, True),       # odd at level 1, scalar loads
    (1, 2, 9, 13, 3, 3, True),      # odd everywhere, level 3 through the LDS analysis phase
    (2, 1, 6, 10, 1, 2, True),      # K = 1 embedded in the 5 x 5 frame
    (1, 1, 28, 28, 5, 5, True),     # five levels
    (5, 3, 7, 7, 5, 2, True),       # ragged last unit
    (1, 1, 56, 56, 5, 3, True),     # the stage-1 plane: one block-row per tile, chained patch halves
    (1, 1, 64, 60, 5, 3, False),    # widest plane the tiles cover, no bias
    (2, 1, 33, 17, 5, 4, True),
    (1, 1, 1, 1, 3, 1, True),
])
def test_emulated_2d_mfma_fp32_split(B, C, H, W, K, L, bias):
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, bias)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K, mfma=2)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-5, atol_scale=2e-5)


@pytest.mark.parametrize("B,C,H,W,K,L,bias,pdtype", [
    (1, 2, 8, 12, 5, 2, True, 1),
    (3, 2, 28, 28, 5, 3, True, 0),
    (2, 2, 14, 14, 5, 2, False, 0),
    (1, 1, 56, 56, 5, 3, True, 0),
    (2, 2, 7, 7, 5, 2, False, 0),      # gradients: fewer row tiles than lane groups (idle groups read zeros)
    (3, 1, 9, 13, 3, 3, True, 0),      # gradients: K = 3 in the 5 x 5 frame, odd sizes, level 3 through LDS
    (1, 1, 64, 64, 5, 3, True, 0),     # gradients: a single plane beyond the LDS of two workgroups (eight waves)
    (2, 1, 33, 20, 1, 2, True, 1),     # gradients: K = 1, two column tiles at level 0
])
def test_emulated_2d_mfma_bf16(B, C, H, W, K, L, bias, pdtype):
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, bias, dtype=1, pdtype=pdtype)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K, dtype=1, pdtype=pdtype, mfma=1)
    want = _oracle(2, x, g, bw, bb, bs, ws, ss)
    # coefficients and folded weights are rounded to bf16 inside: the bf16 bar (2e-2)
    _compare(got, want, rtol=2e-2, atol_scale=2e-2)


def _random_mfma_cases(n, seed):
    import random
    rnd = random.Random(seed)
    cases = []
    for _ in range(n):
        H, W = rnd.randint(1, 26), rnd.randint(1, 26)
        L = rnd.randint(1, 4)
        cases.append((rnd.randint(1, 5), rnd.randint(1, 2), H, W, rnd.choice([1, 3, 5]), L, rnd.random() < 0.7))
    return cases


@pytest.mark.parametrize("B,C,H,W,K,L,bias", _random_mfma_cases(14, 20241))
def test_emulated_2d_mfma_bf16_random_shapes(B, C, H, W, K, L, bias):
    """Seeded random small shapes through the matrix-core kernels (forward, input gradient, parameter gradients)
    under the address sanitizer: every narrow-level variant of the gradient tiles, idle lane groups, ragged units."""
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, bias, dtype=1, pdtype=0)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K, dtype=1, pdtype=0, mfma=1)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-2, atol_scale=2e-2)


def test_emulated_2d_bf16_vector_alu_kernels():
    """bf16 tensors on the vector-ALU kernels (what K = 7 or planes wider than 64 take)."""
    x, g, bw, bb, bs, ws, ss = _case2d(1, 2, 8, 12, 5, 2, True, dtype=1, pdtype=1)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, 5, dtype=1, pdtype=1, mfma=0)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=1e-2, atol_scale=1e-2)


def test_emulated_2d_bf16_io_and_params():
    x, g, bw, bb, bs, ws, ss = _case2d(1, 2, 8, 12, 5, 2, True, dtype=1, pdtype=1)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, 5, dtype=1, pdtype=1)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-2, atol_scale=2e-2)


@pytest.mark.parametrize("B,C,H,W,K,L,bias,pdtype,limit", [
    (1, 2, 8, 12, 5, 2, True, 2, None),      # rows of whole 4-element vectors, half parameters
    (2, 1, 9, 7, 3, 2, True, 0, None),       # odd sizes: element-wise loads and stores
    (1, 1, 24, 40, 7, 3, False, 0, None),
    (2, 1, 24, 48, 5, 2, True, 0, 1024),     # level-by-level kernels (reached by lowering the LDS budget), vector tiles
    (1, 1, 21, 37, 5, 3, True, 0, 1024),     # the same, scalar tile staging
])
def test_emulated_2d_fp16(B, C, H, W, K, L, bias, pdtype, limit):
    """IEEE half tensors: the vector-ALU kernels read and write them and compute in fp32, so the outputs differ from
    the oracle by their final rounding (2^-11 relative) and the parameter gradients hold the fp32 bar."""
    x, g, bw, bb, bs, ws, ss = _case2d(B, C, H, W, K, L, bias, dtype=2, pdtype=pdtype)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, K, dtype=2, pdtype=pdtype, lds_limit=limit)
    want = _oracle(2, x, g, bw, bb, bs, ws, ss)
    # half parameters get their gradients as fp32 as well: the fp32 bar either way
    _compare(got, want, rtol=2e-5, atol_scale=2e-5, act_tol=(1e-3, 1e-3))


def test_emulated_half_conversions():
    """The emulation's own half <-> float conversions against numpy's, over every half bit pattern and a float sweep
    that crosses the subnormal, normal and overflow ranges (the GPU uses the hardware conversion instead)."""
    h = np.arange(65536, dtype=np.uint16)
    vals = h.view(np.float16).astype(np.float32)
    finite = np.isfinite(vals)
    got = emu_util.half_roundtrip(vals[finite])
    np.testing.assert_array_equal(got.view(np.uint32), vals[finite].view(np.uint32))
    rng = np.random.default_rng(5)
    f = (rng.standard_normal(20000) * np.exp(rng.uniform(-20, 12, 20000))).astype(np.float32)
    f = np.concatenate([f, np.float32([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25,
                                       1.5 * 2.0 ** -25, 6.1e-5, 6.0e-5])])
    got = emu_util.half_roundtrip(f)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_emulated_2d_stage1_plane():
    """One plane of the WTConvNeXt-T stage-1 shape (56x56, K=5, L=3)."""
    x, g, bw, bb, bs, ws, ss = _case2d(1, 1, 56, 56, 5, 3, True)
    got = emu_util.run(2, x, g, bw, bb, bs, ws, ss, 5)
    _compare(got, _oracle(2, x, g, bw, bb, bs, ws, ss), rtol=2e-5, atol_scale=2e-5)


def _case1d(B, C, N, K, L, bias, seed=0):
    rng = np.random.default_rng(seed)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    return (f(B, C, N), f(B, C, N), f(C, 1, K) * 0.3, (f(C) if bias else None), f(1, C, 1),
            [f(2 * C, 1, K) * 0.3 for _ in range(L)], [f(1, 2 * C, 1) for _ in range(L)])


@pytest.mark.parametrize("B,C,N,K,L,bias", [
    (2, 2, 64, 5, 3, True),
    (1, 2, 37, 5, 3, True),        # odd lengths at several levels
    (1, 1, 9, 3, 4, False),        # row shorter than 2^L
    (1, 1, 2500, 5, 4, True),      # row-resident kernels: 79 lanes of 32 samples, ragged last lane
    (1, 2, 100, 7, 2, True),
    (1, 1, 40, 1, 2, True),
    (2, 2, 1024, 5, 4, True),      # row-resident, exactly 32 full lanes, two rows per chunk
    (1, 2, 517, 5, 3, True),       # row-resident, 16 samples per lane, odd length, scalar HBM path
    (1, 1, 700, 7, 3, False),      # row-resident, K = 7: level 3 holds 2 < R entries per lane
    (1, 1, 600, 3, 5, True),       # row-resident, five levels
    (1, 1, 800, 5, 5, True),       # row-resident, one level-5 entry per lane: edges from two lanes away
])                                 # (rows beyond 512 lanes, on the tiled kernels: test_emulated_1d_fused_backward)
def test_emulated_1d_fp32(B, C, N, K, L, bias):
    x, g, bw, bb, bs, ws, ss = _case1d(B, C, N, K, L, bias)
    got = emu_util.run(1, x, g, bw, bb, bs, ws, ss, K)
    _compare(got, _oracle(1, x, g, bw, bb, bs, ws, ss), rtol=2e-5, atol_scale=2e-5)


@pytest.mark.parametrize("B,C,N,K,L", [(2, 2, 1000, 5, 4), (1, 2, 517, 5, 3), (1, 1, 37, 3, 3)])
def test_emulated_1d_fp16(B, C, N, K, L):
    x, g, bw, bb, bs, ws, ss = _case1d(B, C, N, K, L, True)
    x, g = _f16_round(x), _f16_round(g)
    got = emu_util.run(1, x, g, bw, bb, bs, ws, ss, K, dtype=2)
    want = _oracle(1, x, g, bw, bb, bs, ws, ss)
    _compare(got, want, rtol=2e-5, atol_scale=2e-5, act_tol=(1e-3, 1e-3))


def test_emulated_1d_row_resident_bf16():
    x, g, bw, bb, bs, ws, ss = _case1d(2, 2, 1000, 5, 4, True)
    x, g = _bf16_round(x), _bf16_round(g)
    got = emu_util.run(1, x, g, bw, bb, bs, ws, ss, 5, dtype=1)
    _compare(got, _oracle(1, x, g, bw, bb, bs, ws, ss), rtol=1e-2, atol_scale=1e-2)


@pytest.mark.parametrize("B,C,N,K,L,bias,dtype,pdtype", [
    (3, 2, 1024, 5, 4, True, 0, 0),      # 32 full lanes; three batch items: chunks of uneven length, tickets of two channels
    (1, 1, 2500, 5, 4, True, 0, 0),      # ragged last lane
    (2, 2, 517, 5, 3, False, 0, 0),      # 16 samples per lane, odd length, element-wise HBM path, no bias
    (1, 1, 700, 7, 3, True, 0, 0),       # K = 7
    (1, 2, 800, 3, 5, True, 0, 0),       # five levels
    (2, 1, 1000, 5, 4, True, 1, 1),      # bf16 rows and parameters
    (1, 1, 17000, 5, 4, True, 0, 0),     # longer than 512 lanes: every pass on the tiled kernels (17 tiles)
])
def test_emulated_1d_fused_backward(B, C, N, K, L, bias, dtype, pdtype):
    """wtconv1d_backward as one call: grad_x and every parameter gradient from the fused row kernel (the last
    workgroup of a channel runs the second stage)."""
    x, g, bw, bb, bs, ws, ss = _case1d(B, C, N, K, L, bias)
    if dtype:
        x, g = _bf16_round(x), _bf16_round(g)
    if pdtype:
        bw, bs = _bf16_round(bw), _bf16_round(bs)
        bb = _bf16_round(bb) if bias else None
        ws, ss = [_bf16_round(w) for w in ws], [_bf16_round(s) for s in ss]
    got = emu_util.run(1, x, g, bw, bb, bs, ws, ss, K, dtype=dtype, pdtype=pdtype, fused_bwd=True)
    tol = 1e-2 if dtype else 2e-5
    _compare(got, _oracle(1, x, g, bw, bb, bs, ws, ss), rtol=tol, atol_scale=tol)


@pytest.mark.parametrize("B,C,H,W,dtype,pdtype,nhwc", [
    (2, 6, 5, 3, 0, 0, 1),        # odd pixel count: element-wise rows, a ragged last tile
    (1, 10, 9, 13, 0, 0, 0),      # NCHW output (LayerNorm2d), two tiles
    (2, 4, 1, 1, 0, 0, 1),        # a single pixel
    (1, 96, 6, 6, 1, 1, 1),       # bf16 tensors and parameters, 4-element vector rows
    (1, 24, 8, 10, 1, 0, 0),      # bf16 tensors, fp32 parameters, NCHW output from registers
    (2, 10, 4, 6, 0, 0, 1),       # fp32 vector rows: five channel pairs over 32 pair slots, two-dword pair words
    (1, 200, 4, 4, 1, 0, 1),      # 100 channel pairs: four pixel groups per tile, four pairs per thread, idle slots
])
def test_emulated_channel_norm(B, C, H, W, dtype, pdtype, nhwc):
    """wtconv_channel_norm and its backward on the host under the sanitizers, against torch in float64."""
    rng = np.random.default_rng(B * 100 + C)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    x, w, b = f(B, C, H, W) * 2 + 0.5, f(C) * 0.5 + 1, f(C)
    dy = f(B, H, W, C) if nhwc else f(B, C, H, W)
    if dtype:
        x, dy = _bf16_round(x), _bf16_round(dy)
    if pdtype:
        w, b = _bf16_round(w), _bf16_round(b)
    out, dx, dw, db = emu_util.run_block("norm", x, dy, w, b, dtype, pdtype, nhwc)
    tx, tw, tb = (torch.from_numpy(a).double().requires_grad_(True) for a in (x, w, b))
    ref = torch.nn.functional.layer_norm(tx.permute(0, 2, 3, 1), (C,), tw, tb, 1e-6)
    ref = ref if nhwc else ref.permute(0, 3, 1, 2)
    ref.backward(torch.from_numpy(dy).double())
    tol = 1e-2 if dtype else 2e-5
    terms = float(np.sqrt(np.mean((dy.astype(np.float64) * 2.0) ** 2)))      # scale of the terms dx cancels between
    np.testing.assert_allclose(out, ref.detach().numpy(), rtol=tol, atol=tol)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=tol, atol=tol * max(terms, 1.0))
    np.testing.assert_allclose(dw, tw.grad.numpy(), rtol=tol, atol=tol * max(1.0, float(np.abs(tw.grad.numpy()).max())))
    np.testing.assert_allclose(db, tb.grad.numpy(), rtol=tol, atol=tol * max(1.0, float(np.abs(tb.grad.numpy()).max())))


@pytest.mark.parametrize("B,C,H,W,dtype", [(2, 6, 5, 3, 0), (1, 10, 9, 13, 0), (2, 4, 1, 1, 0), (1, 96, 6, 6, 1),
                                           (2, 10, 4, 6, 0), (1, 200, 4, 4, 1)])     # the last three: vector rows
def test_emulated_block_residual(B, C, H, W, dtype):
    """wtconv_block_residual and its backward on the host under the sanitizers, against torch in float64."""
    rng = np.random.default_rng(B * 7 + C)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    y, sc, gamma, dout = f(B, H, W, C), f(B, C, H, W), f(C) * 0.7, f(B, C, H, W)
    if dtype:
        y, sc, gamma, dout = (_bf16_round(a) for a in (y, sc, gamma, dout))
    out, dy, dg = emu_util.run_block("residual", y, sc, gamma, dout, dtype, dtype)
    ty, ts, tg = (torch.from_numpy(a).double().requires_grad_(True) for a in (y, sc, gamma))
    ref = ty.permute(0, 3, 1, 2) * tg.reshape(1, -1, 1, 1) + ts
    ref.backward(torch.from_numpy(dout).double())
    tol = 1e-2 if dtype else 2e-5
    np.testing.assert_allclose(out, ref.detach().numpy(), rtol=tol, atol=tol)
    np.testing.assert_allclose(dy, ty.grad.numpy(), rtol=tol, atol=tol)
    np.testing.assert_allclose(dg, tg.grad.numpy(), rtol=tol, atol=tol * max(1.0, float(np.abs(tg.grad.numpy()).max())))

"""wtconv2d_forward_static (the entry point that allocates nothing: its scratch is a static
device array) against wtconv2d_forward, through the C ABI, on two calls in a row, the second
with a smaller input.  Collected last on purpose: a failure here must not hide other tests."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _call_pair(lib, L, K, x, params, dtype_code):
    from wtconv_amd import _lib
    B, C, H, W = x.shape
    tab = _lib.Params()
    bw, bb, bs, ws, ss = params
    tab.base_weight, tab.base_bias, tab.base_scale = bw.data_ptr(), bb.data_ptr(), bs.data_ptr()
    for i in range(L):
        tab.wt_weight[i] = ws[i].data_ptr()
        tab.wt_scale[i] = ss[i].data_ptr()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = lib.wtconv2d_workspace_bytes(B, C, H, W, K, L, _lib.PASS_FORWARD)
    wsp = torch.empty(need, dtype=torch.uint8, device=x.device)
    out_ws = torch.full_like(x, float("nan"))
    out_st = torch.full_like(x, float("nan"))
    rc = lib.wtconv2d_forward(x.data_ptr(), out_ws.data_ptr(), ctypes.byref(tab), B, C, H, W, K, L, dtype_code, 0,
                              wsp.data_ptr(), need, stream)
    assert rc == 0, lib.wtconv_last_error()
    rc = lib.wtconv2d_forward_static(x.data_ptr(), out_st.data_ptr(), ctypes.byref(tab), B, C, H, W, K, L,
                                     dtype_code, 0, stream)
    assert rc == 0, lib.wtconv_last_error()
    torch.cuda.synchronize()
    return out_ws, out_st


def test_forward_static_matches_forward(hip_device):
    from wtconv_amd import _lib
    from oracle import wtconv_ref as R
    lib = _lib.load()
    assert lib.wtconv_static_scratch_bytes() == 4 << 20
    dev = hip_device
    for (B, C, H, W, K, L, dt) in [(3, 40, 28, 30, 5, 3, torch.float32),      # first call
                                   (2, 6, 9, 7, 3, 2, torch.float32),          # smaller: stale scratch beyond its own must not matter
                                   (2, 16, 56, 56, 5, 3, torch.bfloat16)]:
        gen = torch.Generator().manual_seed(B * 1000 + C)
        r = lambda *s: torch.randn(*s, generator=gen).to(dev)
        params = (r(C, 1, K, K) * 0.2, r(C), r(1, C, 1, 1), [r(4 * C, 1, K, K) * 0.2 for _ in range(L)],
                  [r(1, 4 * C, 1, 1) * 0.3 for _ in range(L)])
        x = r(B, C, H, W).to(dt)
        out_ws, out_st = _call_pair(lib, L, K, x, params, _lib.F32 if dt == torch.float32 else _lib.BF16)
        assert torch.isfinite(out_st.float()).all()
        assert torch.equal(out_ws, out_st)           # same kernels, same folded parameters: bit-identical
        # and both are the layer: compare with the oracle on the same values
        want = R.wtconv2d_ref(x.float().cpu().double(), params[0].cpu().double(), params[1].cpu().double(),
                              params[2].cpu().double(), [w.cpu().double() for w in params[3]],
                              [s.cpu().double() for s in params[4]])
        if dt == torch.float32:
            torch.testing.assert_close(out_st.cpu().double(), want, rtol=1e-5, atol=1e-4)
        else:
            rms = want.pow(2).mean().sqrt().item()
            torch.testing.assert_close(out_st.float().cpu().double(), want, rtol=2e-2, atol=2e-2 * rms)


def test_forward_static_rejects_what_does_not_fit(hip_device):
    from wtconv_amd import _lib
    lib = _lib.load()
    B, C, H, W, K, L = 1, 8, 400, 400, 5, 3           # the level-by-level path stages a pyramid in the workspace
    assert lib.wtconv2d_workspace_bytes(B, C, H, W, K, L, _lib.PASS_FORWARD) > lib.wtconv_static_scratch_bytes()
    x = torch.zeros(B, C, H, W, device=hip_device)
    out = torch.zeros_like(x)
    p = torch.zeros(4 * C * K * K, device=hip_device)
    tab = _lib.Params()
    tab.base_weight = tab.base_bias = tab.base_scale = p.data_ptr()
    for i in range(L):
        tab.wt_weight[i] = p.data_ptr()
        tab.wt_scale[i] = p.data_ptr()
    rc = lib.wtconv2d_forward_static(x.data_ptr(), out.data_ptr(), ctypes.byref(tab), B, C, H, W, K, L, 0, 0, None)
    assert rc == -2
    assert b"static buffer" in lib.wtconv_last_error()

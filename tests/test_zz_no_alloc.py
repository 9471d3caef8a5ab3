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
    # a warmed call (the device's scratch address is known by now) must leave the free device memory as it is
    free0, _ = torch.cuda.mem_get_info()
    rc = lib.wtconv2d_forward_static(x.data_ptr(), out_st.data_ptr(), ctypes.byref(tab), B, C, H, W, K, L,
                                     dtype_code, 0, stream)
    assert rc == 0, lib.wtconv_last_error()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"wtconv2d_forward_static changed the free device memory by {free0 - free1} B"
    return out_ws, out_st


def test_forward_static_matches_forward(hip_device):
    from wtconv_amd import _lib
    from oracle import wtconv_ref as R
    lib = _lib.load()
    assert lib.wtconv_static_scratch_bytes() == 4 << 20
    dev = hip_device
    for (B, C, H, W, K, L, dt) in [(3, 40, 28, 30, 5, 3, torch.float32),      # first call
                                   (2, 6, 9, 7, 3, 2, torch.float32),          # smaller: stale scratch beyond its own must not matter
                                   (2, 16, 56, 56, 5, 3, torch.float16),       # vector kernels again: reads the static array after a smaller call
                                   (2, 16, 56, 56, 5, 3, torch.bfloat16)]:     # (matrix-core kernels: no scratch at all)
        gen = torch.Generator().manual_seed(B * 1000 + C)
        r = lambda *s: torch.randn(*s, generator=gen).to(dev)
        params = (r(C, 1, K, K) * 0.2, r(C), r(1, C, 1, 1), [r(4 * C, 1, K, K) * 0.2 for _ in range(L)],
                  [r(1, 4 * C, 1, 1) * 0.3 for _ in range(L)])
        x = r(B, C, H, W).to(dt)
        code = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}[dt]
        out_ws, out_st = _call_pair(lib, L, K, x, params, code)
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
            tol = 2e-2 if dt == torch.bfloat16 else 2e-3
            torch.testing.assert_close(out_st.float().cpu().double(), want, rtol=tol, atol=tol * rms)


def test_forward_static_inside_graph_capture(hip_device):
    """The call recorded into a HIP graph (after one warm-up call outside the capture, which looks up the scratch
    address of the device): every replay, with new inputs and eager work in between, must equal the eager result."""
    from wtconv_amd import _lib
    lib = _lib.load()
    dev = hip_device
    B, C, H, W, K, L = 2, 12, 28, 28, 5, 3
    gen = torch.Generator().manual_seed(5)
    r = lambda *s: torch.randn(*s, generator=gen).to(dev)
    params = (r(C, 1, K, K) * 0.2, r(C), r(1, C, 1, 1), [r(4 * C, 1, K, K) * 0.2 for _ in range(L)],
              [r(1, 4 * C, 1, 1) * 0.3 for _ in range(L)])
    tab = _lib.Params()
    tab.base_weight, tab.base_bias, tab.base_scale = params[0].data_ptr(), params[1].data_ptr(), params[2].data_ptr()
    for i in range(L):
        tab.wt_weight[i] = params[3][i].data_ptr()
        tab.wt_scale[i] = params[4][i].data_ptr()
    xs = torch.zeros(B, C, H, W, device=dev)
    out_g = torch.zeros_like(xs)

    def call(x, out):
        rc = lib.wtconv2d_forward_static(x.data_ptr(), out.data_ptr(), ctypes.byref(tab), B, C, H, W, K, L, _lib.F32,
                                         _lib.F32, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.wtconv_last_error()

    call(xs, out_g)                                   # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(xs, out_g)
    for it in range(3):
        xn = r(B, C, H, W)
        xs.copy_(xn)
        graph.replay()
        torch.cuda.synchronize()
        got = out_g.clone()
        out_e = torch.empty_like(xn)
        call(xn * 1.0, out_e)                         # eager work between the replays (shares the scratch, same stream order)
        torch.cuda.synchronize()
        assert torch.equal(got, out_e), it


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

"""CPU-side checks of the C-ABI library and the host layer (no GPU compute): the library
loads, exports every symbol the header declares, validates arguments before touching the
device, and the Python modules keep the reference's constructor/state-dict surface."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from wtconv_amd import _build, _lib
    if _build.is_stale():
        _build.build_library()
    return _lib.load()


def test_header_symbols_are_exported(lib):
    from wtconv_amd import _lib
    hdr = open(os.path.join(ROOT, "include", "wtconv_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(wtconv[0-9a-z_]*)\s*\(", hdr))
    assert declared == set(_lib.EXPORTS), (declared ^ set(_lib.EXPORTS))
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.wtconv_abi_version() == _lib.ABI_VERSION == 5
    assert lib.wtconv_max_kernel_size() == 7


def test_workspace_sizes(lib):
    C, K, L = 96, 5, 3
    fwd = lib.wtconv2d_workspace_bytes(128, C, 56, 56, K, L, 0)
    assert fwd >= 4 * (C * (1 + 4 * L) * K * K + C) and fwd % 256 == 0
    assert lib.wtconv2d_workspace_bytes(128, C, 56, 56, K, L, 1) == fwd
    par = lib.wtconv2d_workspace_bytes(128, C, 56, 56, K, L, 2)
    assert par >= 4 * C * ((1 + 4 * L) * K * K + 1)
    # the one-call backward pass shares one workspace between its two passes
    assert lib.wtconv2d_workspace_bytes(128, C, 56, 56, K, L, 3) == max(fwd, par)
    assert lib.wtconv1d_workspace_bytes(64, 64, 4096, K, 4, 3) == max(
        lib.wtconv1d_workspace_bytes(64, 64, 4096, K, 4, 1), lib.wtconv1d_workspace_bytes(64, 64, 4096, K, 4, 2))
    assert lib.wtconv1d_workspace_bytes(64, 64, 4096, 5, 4, 0) >= 4 * (64 * 9 * 5 + 64)
    assert lib.wtconv2d_workspace_bytes(0, C, 56, 56, K, L, 0) == 0
    assert lib.wtconv2d_workspace_bytes(1, 1, 20000, 20000, K, L, 0) == 0     # plane beyond 2^28 elements
    # planes whose pyramid exceeds LDS: the workspace also holds the fp32 pyramid(s)
    big = lib.wtconv2d_workspace_bytes(2, 4, 400, 400, K, L, 0)
    assert big >= 4 * 2 * 4 * (400 * 400 + 200 * 200 * 4 // 4)
    assert lib.wtconv2d_workspace_bytes(2, 4, 400, 400, K, L, 2) >= 2 * (big - fwd)


def _params(L=2):
    from wtconv_amd import _lib
    p = _lib.Params()
    p.base_weight = p.base_scale = 0x1000          # never dereferenced: validation fails first
    for i in range(L):
        p.wt_weight[i] = 0x1000
        p.wt_scale[i] = 0x1000
    return p


@pytest.mark.parametrize("kw,code,needle", [
    (dict(K=4), -1, "odd and positive"),
    (dict(K=9), -2, "largest built kernel"),
    (dict(L=6), -1, "wt_levels"),
    (dict(L=0), -1, "wt_levels"),
    (dict(B=0), -1, "positive"),
    (dict(H=0), -1, "spatial size"),
    (dict(dtype=7), -1, "dtype"),
    (dict(x=0), -1, "null"),
    (dict(H=400, W=400), -3, "workspace"),     # larger than LDS: the HBM pyramid needs a larger workspace
    (dict(ws_bytes=16), -3, "workspace"),
    (dict(H=20000, W=20000), -2, "2^28"),      # 32-bit offsets inside a plane
])
def test_forward_argument_validation(lib, kw, code, needle):
    """Bad arguments are rejected with a code and a message before any kernel launch."""
    a = dict(x=0x1000, out=0x2000, B=2, C=4, H=8, W=8, K=5, L=2, dtype=0, pdtype=0, ws=0x3000, ws_bytes=1 << 20)
    a.update(kw)
    p = _params(2)
    rc = lib.wtconv2d_forward(a["x"], a["out"], ctypes.byref(p), a["B"], a["C"], a["H"], a["W"], a["K"], a["L"],
                              a["dtype"], a["pdtype"], a["ws"], a["ws_bytes"], None)
    assert rc == code
    assert needle in lib.wtconv_last_error().decode()


def test_null_parameter_pointer_rejected(lib):
    from wtconv_amd import _lib
    p = _lib.Params()
    rc = lib.wtconv1d_forward(0x1000, 0x2000, ctypes.byref(p), 1, 2, 64, 5, 2, 0, 0, 0x3000, 1 << 20, None)
    assert rc == -1 and "null parameter" in lib.wtconv_last_error().decode()
    g = _lib.ParamGrads()
    rc = lib.wtconv2d_backward_params(0x1000, 0x2000, ctypes.byref(_params(2)), ctypes.byref(g), 1, 2, 8, 8, 5, 2,
                                      0, 0, 0x3000, 1 << 20, None)
    assert rc == -1 and "gradient pointer" in lib.wtconv_last_error().decode()


def test_one_call_backward_validates_like_its_passes(lib):
    """wtconv2d_backward / wtconv1d_backward reject bad arguments before any launch, with the
    message of the pass that found them."""
    from wtconv_amd import _lib
    g = _lib.ParamGrads()
    rc = lib.wtconv2d_backward(0x1000, 0x2000, 0x3000, ctypes.byref(_params(2)), ctypes.byref(g), 2, 4, 8, 8, 4, 2,
                               0, 0, 0x4000, 1 << 20, None)
    assert rc == -1 and "odd and positive" in lib.wtconv_last_error().decode()
    rc = lib.wtconv1d_backward(0x1000, 0x2000, 0, ctypes.byref(_params(2)), ctypes.byref(g), 1, 2, 64, 5, 2,
                               0, 0, 0x4000, 1 << 20, None)
    assert rc == -1 and "null" in lib.wtconv_last_error().decode()
    rc = lib.wtconv2d_backward(0x1000, 0x2000, 0x3000, ctypes.byref(_params(2)), ctypes.byref(g), 2, 4, 8, 8, 5, 2,
                               0, 0, 0x4000, 16, None)
    assert rc == -3 and "workspace" in lib.wtconv_last_error().decode()


def test_check_raises_python_exceptions(lib):
    from wtconv_amd import _lib
    p = _params(2)
    rc = lib.wtconv2d_forward(0x1000, 0x2000, ctypes.byref(p), 2, 4, 8, 8, 4, 2, 0, 0, 0x3000, 1 << 20, None)
    with pytest.raises(ValueError, match="odd and positive"):
        _lib.check(rc, "forward")
    rc = lib.wtconv2d_forward(0x1000, 0x2000, ctypes.byref(p), 2, 4, 400, 400, 5, 2, 0, 0, 0x3000, 1 << 20, None)
    with pytest.raises(RuntimeError, match="workspace of"):
        _lib.check(rc, "forward")


# ------------------------------------------------------------------ module surface
def test_reference_module_surface_and_init(lib):
    import wtconv
    from wtconv.wtconv1d import WTConv1d
    from oracle import wtconv_ref as R
    torch.manual_seed(0)
    m = wtconv.WTConv2d(8, 8, kernel_size=5, stride=1, bias=True, wt_levels=3, wt_type='db1')
    torch.manual_seed(0)
    r = R.RefWTConv2d(8, 8, 5, wt_levels=3)
    assert list(m.state_dict().keys()) == list(r.state_dict().keys())
    for (k, a), (_, b) in zip(m.state_dict().items(), r.state_dict().items()):
        assert torch.equal(a, b), k
    assert (m.in_channels, m.wt_levels, m.stride, m.dilation) == (8, 3, 1, 1)
    assert sum(p.numel() for p in m.parameters()) == (59 + 104 * 3) * 8
    assert not m.wt_filter.requires_grad and not m.iwt_filter.requires_grad
    torch.manual_seed(1)
    m1 = WTConv1d(4, 4, 3, wt_levels=2)
    torch.manual_seed(1)
    r1 = R.RefWTConv1d(4, 4, 3, wt_levels=2)
    for (k, a), (_, b) in zip(m1.state_dict().items(), r1.state_dict().items()):
        assert torch.equal(a, b), k


def test_fast_twin_surface(lib):
    from fast_wtconv.wtconv_cuda import WTConv2d as Fast
    import fast_wtconv
    assert fast_wtconv.WTConv2d is Fast
    m = Fast(4, 4, 5, 1, 2, False)       # positional: kernel_size, stride, wt_levels, bias
    assert m.base_bias is None and m.wt_levels == 2 and m.kernel_size == 5 and m.stride == 1
    assert set(m.state_dict()) == {"base_weight", "base_scale", "wt_weights.0", "wt_weights.1",
                                   "wt_scales.0", "wt_scales.1"}
    assert m.wt_weights[0].shape == (16, 1, 5, 5) and torch.all(m.wt_scales[1] == 0.1)
    with pytest.raises(AssertionError):
        Fast(4, 8)
    with pytest.raises(AssertionError):
        Fast(4, 4, wt_levels=6)


def test_constructor_errors(lib):
    import wtconv
    with pytest.raises(AssertionError):
        wtconv.WTConv2d(4, 8)
    with pytest.raises(NotImplementedError, match="db1"):
        wtconv.WTConv2d(4, 4, wt_type='db2')
    with pytest.raises(ValueError, match="odd and positive"):
        wtconv.WTConv2d(4, 4, kernel_size=4)
    with pytest.raises(ValueError, match="largest built kernel"):
        wtconv.WTConv2d(4, 4, kernel_size=9)


def test_cpu_tensor_is_refused_loudly(lib):
    """No CPU fallback: a CPU tensor is an error, not a silent slow path."""
    import wtconv
    m = wtconv.WTConv2d(4, 4, 3, wt_levels=1)
    with pytest.raises(RuntimeError, match="GPU only"):
        m(torch.randn(1, 4, 8, 8))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from wtconv_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setenv("WTCONV_HIP_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.WTConvLibraryError, match="no fallback"):
        _lib.load()


def test_cpp_autograd_node_builds_loads_and_declines_host_tensors(lib):
    """The C++ autograd node (host code only) compiles against the installed PyTorch, takes the library's entry
    points by address, and hands anything that is not a GPU tensor in a kernel dtype back to the Python path."""
    from wtconv_amd import _build, _ext
    if (not os.path.exists(_build.BINDING_PATH)
            or os.path.getmtime(_build.BINDING_PATH) < os.path.getmtime(_build.BINDING_SRC)):
        _build.build_binding()
        _ext._tried, _ext._mod = False, None
    ext = _ext.get()
    assert ext is not None
    C, K = 4, 3
    x = torch.randn(1, C, 8, 8)
    args = (torch.randn(C, 1, K, K), torch.randn(C), torch.randn(1, C, 1, 1), [torch.randn(4 * C, 1, K, K)],
            [torch.randn(1, 4 * C, 1, 1)])
    assert ext.layer(x, *args, 2, K, 1) is None
    assert ext.layer(x, args[0], None, *args[2:], 2, K, 1) is None

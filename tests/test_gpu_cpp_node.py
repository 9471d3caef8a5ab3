"""The C++ autograd node (wtconv_amd/csrc/torch_binding.cpp) against the Python autograd function it replaces on
the hot path: same library calls, so every result must be bit-identical; plus the cases the node hands back to the
Python path.  The kernels themselves are checked against the oracle in test_gpu_parity.py, which runs through this
node as well (it is what the modules call)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _params(dims, C, K, L, bias, dtype, dev, seed=0):
    gen = torch.Generator().manual_seed(seed)
    S = 4 if dims == 2 else 2
    kshape = (K, K) if dims == 2 else (K,)
    ones = (1,) * dims
    r = lambda *s: torch.randn(*s, generator=gen).to(device=dev, dtype=dtype).requires_grad_(True)
    return (r(C, 1, *kshape), r(C) if bias else None, r(1, C, *ones),
            [r(S * C, 1, *kshape) for _ in range(L)], [r(1, S * C, *ones) for _ in range(L)])


def _run(fn, x, g, params, need_x=True, need_p=True):
    bw, bb, bs, ws, ss = params
    leaves = [t for t in (bw, bb, bs, *ws, *ss) if t is not None]
    for t in leaves:
        t.grad = None
        t.requires_grad_(need_p)
    x = x.clone().requires_grad_(need_x)
    out = fn(x, bw, bb, bs, ws, ss)
    out.backward(g)
    torch.cuda.synchronize()
    return out.detach(), x.grad, [t.grad for t in leaves]


def _both(dims, x, params, K, L):
    from wtconv_amd import _ext, functional as Fn
    ext = _ext.get()
    assert ext is not None, "the C++ node is not built (python -m wtconv_amd._build)"

    def cpp(x, bw, bb, bs, ws, ss):
        out = ext.layer(x, bw, bb, bs, list(ws), list(ss), dims, K, L)
        assert out is not None, "canonical arguments must take the C++ node"
        return out

    def py(x, bw, bb, bs, ws, ss):
        return Fn._WTConvFn.apply(x, bw, bb, bs, dims, K, L, *ws, *ss)
    return cpp, py


def _same(a, b):
    if a is None or b is None:
        return a is None and b is None
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b)


@pytest.mark.parametrize("dims,shape,K,L,bias,dtype,pdtype", [
    (2, (3, 6, 20, 24), 5, 2, True, torch.float32, torch.float32),
    (2, (2, 4, 17, 9), 3, 3, False, torch.float32, torch.float32),
    (2, (4, 8, 28, 28), 5, 3, True, torch.bfloat16, torch.bfloat16),
    (2, (4, 8, 14, 14), 5, 2, True, torch.bfloat16, torch.float32),      # autocast-style: bf16 activations, fp32 parameters
    (2, (2, 4, 12, 12), 5, 2, True, torch.float16, torch.float16),
    (1, (2, 6, 640), 5, 3, True, torch.float32, torch.float32),
    (1, (2, 4, 4096), 5, 4, False, torch.bfloat16, torch.bfloat16),
])
def test_cpp_node_matches_python_function(dev, dims, shape, K, L, bias, dtype, pdtype):
    params = _params(dims, shape[1], K, L, bias, pdtype, dev)
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(*shape, generator=gen).to(device=dev, dtype=dtype)
    g = torch.randn(*shape, generator=gen).to(device=dev, dtype=dtype)
    cpp, py = _both(dims, x, params, K, L)
    for need_x, need_p in ((True, True), (True, False), (False, True)):
        a = _run(cpp, x, g, params, need_x, need_p)
        b = _run(py, x, g, params, need_x, need_p)
        assert _same(a[0], b[0]), "out"
        assert _same(a[1], b[1]), f"grad_x (need_x={need_x}, need_p={need_p})"
        assert len(a[2]) == len(b[2])
        for i, (u, v) in enumerate(zip(a[2], b[2])):
            assert _same(u, v), f"parameter gradient {i} (need_x={need_x}, need_p={need_p})"


def test_cpp_node_launches_on_the_current_stream(dev):
    """Work queued on a side stream before the layer must be seen by it: the node has to launch on PyTorch's current
    stream, not on the default one."""
    params = _params(2, 8, 5, 2, True, torch.float32, dev)
    cpp, _ = _both(2, None, params, 5, 2)
    x = torch.randn(4, 8, 56, 56, device=dev)
    g = torch.randn(4, 8, 56, 56, device=dev)
    want = _run(cpp, x, g, params)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        big = torch.randn(64, 1024, 1024, device=dev)
        for _ in range(10):
            big = big * 1.0001                   # keeps the side stream busy for a while
        x2 = x * (big[0, 0, 0] * 0 + 1)          # depends on that work
        bw, bb, bs, ws, ss = params
        out = cpp(x2, bw, bb, bs, ws, ss)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert torch.equal(out.detach(), want[0])


def test_arguments_that_need_conversion_take_the_python_path(dev):
    from wtconv_amd import _ext, functional as Fn
    ext = _ext.get()
    assert ext is not None
    bw, bb, bs, ws, ss = _params(2, 4, 5, 1, True, torch.float32, dev)
    x = torch.randn(2, 4, 10, 10, device=dev)
    # mixed parameter dtypes, a transposed (non-contiguous) weight, a parameter on the host: None from the node ...
    assert ext.layer(x, bw, bb, bs.bfloat16(), ws, ss, 2, 5, 1) is None
    assert ext.layer(x, bw.transpose(2, 3), bb, bs, ws, ss, 2, 5, 1) is None
    assert ext.layer(x, bw, bb.cpu(), bs, ws, ss, 2, 5, 1) is None
    assert ext.layer(x.double(), bw, bb, bs, ws, ss, 2, 5, 1) is None
    # ... and the public function still computes them
    ref = Fn.wtconv2d(x, bw, bb, bs, ws, ss)
    got = Fn.wtconv2d(x, bw.transpose(2, 3).contiguous().transpose(2, 3), bb.cpu(), bs, ws, ss)
    assert torch.equal(ref, got)


def test_cpp_node_reports_library_errors(dev):
    from wtconv_amd import _ext
    ext = _ext.get()
    bw, bb, bs, ws, ss = _params(2, 4, 9, 1, True, torch.float32, dev)     # kernel size 9: not built
    x = torch.randn(2, 4, 10, 10, device=dev)
    with pytest.raises(RuntimeError, match="kernel_size"):
        ext.layer(x, bw, bb, bs, ws, ss, 2, 9, 1)


def test_double_backward_is_refused(dev):
    params = _params(2, 4, 5, 1, True, torch.float32, dev)
    cpp, _ = _both(2, None, params, 5, 1)
    x = torch.randn(2, 4, 10, 10, device=dev, requires_grad=True)
    bw, bb, bs, ws, ss = params
    out = cpp(x, bw, bb, bs, ws, ss)
    (gx,) = torch.autograd.grad(out.sum(), x, create_graph=True)
    with pytest.raises(RuntimeError):
        gx.sum().backward()


def test_gradient_penalty_is_refused_not_dropped(dev):
    """A loss that mixes the output with a function of grad_x: the second-order term cannot be differentiated, and
    both autograd paths must say so instead of treating it as a constant."""
    params = _params(2, 4, 5, 1, True, torch.float32, dev)
    for fn in _both(2, None, params, 5, 1):
        x = torch.randn(2, 4, 10, 10, device=dev, requires_grad=True)
        bw, bb, bs, ws, ss = params
        out = fn(x, bw, bb, bs, ws, ss)
        (gx,) = torch.autograd.grad(out.sum(), x, create_graph=True)
        loss = out.sum() + gx.pow(2).sum()
        with pytest.raises(RuntimeError):
            loss.backward()


def test_create_graph_without_second_order_use_still_works(dev):
    """create_graph=True alone is harmless as long as nothing differentiates the gradients."""
    params = _params(2, 4, 5, 1, True, torch.float32, dev)
    cpp, py = _both(2, None, params, 5, 1)
    bw, bb, bs, ws, ss = params
    x = torch.randn(2, 4, 10, 10, device=dev, requires_grad=True)
    (ga,) = torch.autograd.grad(cpp(x, bw, bb, bs, ws, ss).sum(), x, create_graph=True)
    (gb,) = torch.autograd.grad(py(x, bw, bb, bs, ws, ss).sum(), x, create_graph=True)
    assert torch.equal(ga.detach(), gb.detach())

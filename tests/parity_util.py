"""Shared helpers of the GPU parity tests: seeded cases, oracle runs, comparisons."""
import torch

from oracle import wtconv_ref as R

# Tolerances stated for this layer: fp32 1e-5 relative / 1e-4 absolute; bf16 2e-2 relative
# (absolute floor 2e-2 of the oracle's RMS).
FP32_RTOL, FP32_ATOL = 1e-5, 1e-4
BF16_RTOL = 2e-2


def seeded_case(kind, C, K, L, shape, bias=True, seed=0, stride=1):
    """torch.manual_seed(seed) -> oracle module with default init -> x -> g (fp32, CPU)."""
    torch.manual_seed(seed)
    cls = R.RefWTConv2d if kind == "2d" else R.RefWTConv1d
    ref = cls(C, C, K, stride=stride, bias=bias, wt_levels=L)
    x = torch.randn(*shape)
    with torch.no_grad():
        oshape = ref(x[:1]).shape
    g = torch.randn(shape[0], *oshape[1:])
    return ref, x, g


def randomize_scales(ref, seed=1):
    """Default scales are constants (1.0 / 0.1); draw them so scale gradients are exercised."""
    gen = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        ref.base_scale.weight.copy_(torch.randn(ref.base_scale.weight.shape, generator=gen))
        for s in ref.wavelet_scale:
            s.weight.copy_(torch.randn(s.weight.shape, generator=gen) * 0.5)


def copy_to_hip_module(ref, hip_cls, kind, K, L, stride=1, bias=True):
    """Instantiate the product module and load the oracle's state dict (same key names)."""
    C = ref.in_channels
    m = hip_cls(C, C, K, stride=stride, bias=bias, wt_levels=L)
    missing, unexpected = m.load_state_dict(ref.state_dict(), strict=True)
    assert not missing and not unexpected
    return m


def oracle_run(ref, x, g, dtype=torch.float64):
    """Forward+backward of the oracle in `dtype` on CPU; returns out, dx, grads (by name)."""
    import copy
    r = copy.deepcopy(ref).to(dtype)
    return R.layer_grads(r, x.to(dtype), g.to(dtype))


def hip_run(mod, x, g, device, dtype=torch.float32, param_dtype=None):
    mod = mod.to(device)
    if param_dtype is not None:
        mod = mod.to(param_dtype)
    for p in mod.parameters():
        p.grad = None
    xd = x.to(device=device, dtype=dtype).requires_grad_(True)
    out = mod(xd)
    out.backward(g.to(device=device, dtype=dtype))
    torch.cuda.synchronize()
    grads = {n: p.grad.detach().float().cpu() for n, p in mod.named_parameters() if p.grad is not None}
    return out.detach().float().cpu(), xd.grad.detach().float().cpu(), grads


def assert_fp32(got, want, name):
    torch.testing.assert_close(got.double(), want.double(), rtol=FP32_RTOL, atol=FP32_ATOL,
                               msg=lambda m: f"{name}: {m}")


def assert_bf16(got, want, name):
    rms = want.double().pow(2).mean().sqrt().item()
    torch.testing.assert_close(got.double(), want.double(), rtol=BF16_RTOL, atol=BF16_RTOL * max(rms, 1e-12),
                               msg=lambda m: f"{name}: {m}")


def compare_all(got, want, check):
    go, gdx, gg = got
    wo, wdx, wg = want
    check(go, wo, "out")
    check(gdx, wdx, "grad_x")
    trainable = [n for n in wg if n not in ("wt_filter", "iwt_filter")]
    assert set(trainable) <= set(gg), f"missing grads: {set(trainable) - set(gg)}"
    for n in trainable:
        check(gg[n], wg[n], n)

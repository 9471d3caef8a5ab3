"""GPU parity of the block-epilogue kernels (wtconv_channel_norm, wtconv_block_residual) against
torch's own LayerNorm / permute / mul / add in float64 on the CPU, through the C ABI.  Floating-point
kernels: the reference here is the plain torch formulation of wtconvnext.py:132-140 of the reference."""
import pytest
import torch
import torch.nn.functional as F

import parity_util as U

pytestmark = pytest.mark.gpu

SHAPES = [(2, 96, 56, 56), (3, 192, 28, 28), (2, 384, 14, 14), (3, 768, 7, 7), (1, 6, 5, 3), (2, 2, 1, 1),
          (1, 1538, 3, 3), (2, 10, 9, 13)]


def _ref_norm(x, w, b, eps, nhwc):
    y = F.layer_norm(x.double().permute(0, 2, 3, 1), (x.shape[1],), w.double(), b.double(), eps)
    return y if nhwc else y.permute(0, 3, 1, 2)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype,pdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("nhwc", [True, False])
def test_channel_norm(hip_device, shape, dtype, pdtype, nhwc):
    from wtconv_amd import block_ops
    B, C, H, W = shape
    gen = torch.Generator().manual_seed(B * 1000 + C)
    x = (torch.randn(shape, generator=gen) * 2 + 0.5).to(dtype)
    w = (torch.randn(C, generator=gen) * 0.5 + 1).to(pdtype)
    b = torch.randn(C, generator=gen).to(pdtype)
    assert block_ops.usable(x.to(hip_device), w.to(hip_device), b.to(hip_device))
    got = block_ops.channel_norm(x.to(hip_device), w.to(hip_device), b.to(hip_device), 1e-6, nhwc).float().cpu()
    want = _ref_norm(x.float(), w.float(), b.float(), 1e-6, nhwc)
    assert got.shape == want.shape
    (U.assert_fp32 if dtype == torch.float32 else U.assert_bf16)(got, want.float(), f"channel_norm {shape} nhwc={nhwc}")


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype,pdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("with_gamma", [True, False])
def test_block_residual(hip_device, shape, dtype, pdtype, with_gamma):
    from wtconv_amd import block_ops
    B, C, H, W = shape
    gen = torch.Generator().manual_seed(B * 77 + C)
    y = torch.randn(B, H, W, C, generator=gen).to(dtype)
    sc = torch.randn(shape, generator=gen).to(dtype)
    gamma = (torch.randn(C, generator=gen) * 0.7).to(pdtype) if with_gamma else None
    got = block_ops.block_residual(y.to(hip_device), sc.to(hip_device),
                                   gamma.to(hip_device) if with_gamma else None).float().cpu()
    want = y.double().permute(0, 3, 1, 2)
    if with_gamma:
        want = want * gamma.double().reshape(1, -1, 1, 1)
    want = (want + sc.double()).float()
    (U.assert_fp32 if dtype == torch.float32 else U.assert_bf16)(got, want, f"block_residual {shape}")


def test_argument_checks(hip_device):
    from wtconv_amd import block_ops
    x = torch.randn(1, 3, 4, 4, device=hip_device)
    w = torch.ones(3, device=hip_device)
    assert not block_ops.usable(x, w, w)                      # odd channel count: the caller keeps the plain path
    with pytest.raises(RuntimeError, match="even"):
        block_ops.channel_norm(x, w, w, 1e-6, True)
    x = torch.randn(1, 4, 4, 4, device=hip_device)
    assert not block_ops.usable(x.requires_grad_(True))       # training: nothing here is differentiable
    assert not block_ops.usable(torch.randn(1, 4, 4, 4))      # CPU tensor
    with pytest.raises(ValueError, match="does not match"):
        block_ops.block_residual(torch.randn(1, 4, 4, 3, device=hip_device), torch.randn(1, 4, 4, 4, device=hip_device), None)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_inference_fused_blocks_match_plain_blocks(hip_device, dtype, monkeypatch):
    """A small WTConvNeXt at inference with the fused block passes against the same model on the plain
    torch passes (what training runs), same WTConv kernels in both."""
    import wtconvnext
    from wtconv_amd import block_ops
    torch.manual_seed(0)
    m = wtconvnext.WTConvNeXt(depths=(1, 1, 2, 1), dims=(16, 32, 64, 128), num_classes=10, ls_init_value=0.5).to(hip_device).to(dtype).eval()
    x = torch.randn(3, 3, 64, 64, device=hip_device).to(dtype)
    calls = {"n": 0}
    real = block_ops.channel_norm

    def counting(*a, **k):
        calls["n"] += 1
        return real(*a, **k)
    monkeypatch.setattr(block_ops, "channel_norm", counting)
    with torch.no_grad():
        fused = m(x).float().cpu()
    assert calls["n"] == 5 + 4 + 1          # block norms, stem + 3 downsample norms, head norm
    monkeypatch.setattr(block_ops, "usable", lambda *a, **k: False)
    with torch.no_grad():
        plain = m(x).float().cpu()
    if dtype == torch.float32:
        torch.testing.assert_close(fused, plain, rtol=1e-4, atol=1e-4)
    else:
        U.assert_bf16(fused, plain, "model logits")

"""The WTConvNeXt harness reproduces the parameter counts the reference logs hold
(logs/val_tiny.out:4, val_small.out:4, val_base.out:4) -- the only known answers the
reference has for the model shell."""
import pytest
import torch


@pytest.mark.parametrize("name,count", [("wtconvnext_tiny", 30595624), ("wtconvnext_small", 54448936),
                                        ("wtconvnext_base", 94225128)])
def test_param_counts(name, count):
    import wtconvnext
    with torch.device("meta"):
        m = getattr(wtconvnext, name)()
    assert sum(p.numel() for p in m.parameters()) == count


def test_structure_and_init():
    import wtconvnext
    from oracle import wtconv_ref as R
    torch.manual_seed(0)
    m = wtconvnext.wtconvnext_tiny(depths=(1, 1, 1, 1), num_classes=10)
    levels = [s.blocks[0].conv_dw.wt_levels for s in m.stages]
    assert levels == [5, 4, 3, 2]
    blk = m.stages[0].blocks[0]
    # the model init re-draws the WTConv convolutions (trunc-normal 0.02) and zeroes biases
    w = torch.cat([c.weight.flatten() for c in blk.conv_dw.wavelet_convs])
    assert abs(w.std().item() - 0.02) < 2e-3 and w.abs().max() < 0.15
    assert torch.all(blk.conv_dw.base_conv.bias == 0)
    assert torch.all(blk.conv_dw.wavelet_scale[0].weight == 0.1)
    assert torch.all(blk.gamma == 1e-6)
    nwd = m.no_weight_decay()
    assert "stages.0.blocks.0.conv_dw.base_scale.weight" in nwd
    assert "stages.3.blocks.0.conv_dw.wavelet_scale.1.weight" in nwd
    keys = set(m.state_dict())
    assert {"stem.0.weight", "stem.1.weight", "stages.1.downsample.1.weight", "stages.2.blocks.0.mlp.fc1.weight",
            "stages.0.blocks.0.conv_dw.wavelet_convs.4.weight", "head.norm.weight", "head.fc.bias"} <= keys
    # the oracle class plugs into the same hook and yields the same state-dict keys
    torch.manual_seed(0)
    r = wtconvnext.wtconvnext_tiny(depths=(1, 1, 1, 1), num_classes=10, wtconv_class=R.RefWTConv2d)
    assert set(r.state_dict()) == keys
    out = r(torch.randn(1, 3, 64, 64))
    assert out.shape == (1, 10)


def test_drop_path_schedule_and_head_options():
    """drop_path_rate spreads linearly over all blocks (reference wtconvnext.py:309), is the identity
    in eval mode and keeps the expectation in training; head_init_scale scales the classifier
    (wtconvnext.py:483-493); reset_classifier / forward_head(pre_logits) follow the reference's API."""
    import wtconvnext
    from oracle import wtconv_ref as R
    torch.manual_seed(0)
    m = wtconvnext.wtconvnext_tiny(depths=(1, 2, 1, 1), num_classes=7, drop_path_rate=0.4, head_init_scale=0.5,
                                   wtconv_class=R.RefWTConv2d)
    rates = [getattr(b.drop_path, "drop_prob", 0.0) for s in m.stages for b in s.blocks]
    assert rates == pytest.approx([0.0, 0.1, 0.2, 0.3, 0.4])
    torch.manual_seed(0)
    ref = wtconvnext.wtconvnext_tiny(depths=(1, 2, 1, 1), num_classes=7, wtconv_class=R.RefWTConv2d)
    assert torch.allclose(m.head.fc.weight, 0.5 * ref.head.fc.weight)
    x = torch.randn(2, 3, 64, 64)
    m.eval()
    ref.eval()
    with torch.no_grad():
        ref.head.fc.load_state_dict(m.head.fc.state_dict())
        assert torch.equal(m(x), ref(x))                     # stochastic depth is off in eval mode
        feats = m.forward_features(x)
        assert m.forward_head(feats, pre_logits=True).shape == (2, 768)
    dp = wtconvnext.wtconvnext.DropPath(0.25).train()
    y = dp(torch.ones(4000, 3))
    kept = (y[:, 0] != 0).float().mean().item()
    assert abs(kept - 0.75) < 0.03 and torch.all((y == 0) | (y == 1 / 0.75))
    m.reset_classifier(3)
    assert m(x).shape == (2, 3) and m.num_classes == 3
    m.set_grad_checkpointing(True)
    m.train()
    m(x.requires_grad_(True)).sum().backward()
    assert x.grad is not None

"""The library-routine oracle reproduces the committed golden vectors (float64)."""
import pytest
import torch

import golden_util as G
from oracle import wtconv_ref as R

CASES = G.cases()


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_matches_golden(name):
    dims, x, g, p, exp = G.to_layer_tensors(CASES[name])
    leaves = [x, p["base_w"], p["base_s"]] + p["wt_ws"] + p["wt_ss"] + ([p["base_b"]] if p["base_b"] is not None else [])
    for t in leaves:
        t.requires_grad_(True)
    fn = R.wtconv2d_ref if dims == 2 else R.wtconv1d_ref
    out = fn(x, p["base_w"], p["base_b"], p["base_s"], p["wt_ws"], p["wt_ss"])
    out.backward(g)
    tol = dict(rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out.detach(), exp["out"], **tol)
    torch.testing.assert_close(x.grad, exp["dx"], **tol)
    torch.testing.assert_close(p["base_w"].grad, exp["dbase_w"], **tol)
    torch.testing.assert_close(p["base_s"].grad, exp["dbase_s"], **tol)
    if p["base_b"] is not None:
        torch.testing.assert_close(p["base_b"].grad, exp["dbase_b"], **tol)
    for l in range(len(p["wt_ws"])):
        torch.testing.assert_close(p["wt_ws"][l].grad, exp["dwt_ws"][l], **tol)
        torch.testing.assert_close(p["wt_ss"][l].grad, exp["dwt_ss"][l], **tol)

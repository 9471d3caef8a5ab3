"""HIP layer against the committed golden vectors (through the functional C-ABI wrapper)."""
import pytest
import torch

import golden_util as G
import parity_util as U

pytestmark = pytest.mark.gpu
CASES = G.cases()


@pytest.mark.parametrize("name", sorted(CASES))
def test_hip_matches_golden(hip_device, name):
    from wtconv_amd import wtconv1d, wtconv2d
    dims, x, g, p, exp = G.to_layer_tensors(CASES[name], torch.float32)
    dev = lambda t: None if t is None else t.to(hip_device).requires_grad_(True)
    x, bw, bb, bs = dev(x), dev(p["base_w"]), dev(p["base_b"]), dev(p["base_s"])
    ws, ss = [dev(w) for w in p["wt_ws"]], [dev(s) for s in p["wt_ss"]]
    fn = wtconv2d if dims == 2 else wtconv1d
    out = fn(x, bw, bb, bs, ws, ss)
    out.backward(g.to(hip_device))
    torch.cuda.synchronize()
    chk = lambda a, b, n: U.assert_fp32(a.detach().cpu(), b, f"{name}:{n}")
    chk(out, exp["out"], "out")
    chk(x.grad, exp["dx"], "dx")
    chk(bw.grad, exp["dbase_w"], "dbase_w")
    chk(bs.grad, exp["dbase_s"], "dbase_s")
    if bb is not None:
        chk(bb.grad, exp["dbase_b"], "dbase_b")
    for l in range(len(ws)):
        chk(ws[l].grad, exp["dwt_ws"][l], f"dwt_w{l}")
        chk(ss[l].grad, exp["dwt_ss"][l], f"dwt_s{l}")

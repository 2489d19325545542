"""Golden fixtures (tests/golden/lce_golden.json): the oracle must reproduce them on the CPU, and the HIP path
must match them on the GPU within the operator's tolerances."""
import json
import os

import pytest
import torch

from helpers import make_inputs

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = json.load(open(os.path.join(HERE, "golden", "lce_golden.json")))


def _inputs(c):
    return make_inputs(c["N"], c["H"], c["V"], getattr(torch, c["dtype"]), c["seed"], ignore_frac=c["ignore_frac"],
                       zipf=c.get("zipf", False))


@pytest.mark.parametrize("name", sorted(GOLD))
def test_oracle_reproduces_golden(name):
    from oracle import lce_forward_backward_fp64

    g = GOLD[name]
    c = g["config"]
    x, y, w = _inputs(c)
    assert y[:16].tolist() == g["label_head"]
    r = lce_forward_backward_fp64(x.double(), y, w.double(), -1, c["z_reg"], c["scale"])
    assert r.n_valid == g["n_valid"]
    for k in ("loss", "z_reg", "logit_max", "logit_entropy", "logit_norm"):
        assert abs(getattr(r, k).item() - g[k]) <= 1e-10 * abs(g[k]), k
    assert torch.allclose(r.lse[:16], torch.tensor(g["lse_head"], dtype=torch.float64), rtol=1e-12)
    assert abs(r.dx.norm().item() - g["dx_norm"]) <= 1e-9 * g["dx_norm"]
    assert abs(r.dw.norm().item() - g["dw_norm"]) <= 1e-9 * g["dw_norm"]
    for i, j, v in g["dx_probes"]:
        assert abs(r.dx[i % c["N"], j % c["H"]].item() - v) <= 1e-9 * abs(v) + 1e-18
    for i, j, v in g["dw_probes"]:
        assert abs(r.dw[i % c["H"], j % c["V"]].item() - v) <= 1e-9 * abs(v) + 1e-18


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(GOLD))
def test_hip_path_matches_golden(name):
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    g = GOLD[name]
    c = g["config"]
    print("golden case", name, flush=True)
    x, y, w = _inputs(c)
    xd = x.cuda().requires_grad_(True)
    wd = w.cuda().requires_grad_(True)
    out = linear_cross_entropy(xd, y.cuda(), wd, -1, c["z_reg"], c["scale"], 512, True)
    out[0].backward()
    torch.cuda.synchronize()
    # fp32 tensors are computed as bf16 pairs and held to 1e-5 (loss) / 1e-3 (gradients); 16-bit ones to 1e-3 / 2e-2
    f32 = c["dtype"] == "float32"
    ltol, gtol = (1e-5, 1e-3) if f32 else (1e-3, 2e-2)
    assert abs(out[0].item() - g["loss"]) <= ltol * abs(g["loss"])
    assert abs(out[1].item() - g["z_reg"]) <= ltol * abs(g["z_reg"])
    assert abs(out[2].item() - g["logit_max"]) <= 1e-3 * abs(g["logit_max"])
    assert abs(out[3].item() - g["logit_entropy"]) <= 2e-3 * abs(g["logit_entropy"])
    assert abs(out[4].item() - g["logit_norm"]) <= 2e-3 * abs(g["logit_norm"])
    dx, dw = xd.grad.double().cpu(), wd.grad.double().cpu()
    # norms within the gradient tolerance, probes within it relative to the largest entry
    assert abs(dx.norm().item() - g["dx_norm"]) <= gtol * g["dx_norm"]
    assert abs(dw.norm().item() - g["dw_norm"]) <= gtol * g["dw_norm"]
    dx_scale, dw_scale = dx.abs().max().item(), dw.abs().max().item()
    for i, j, v in g["dx_probes"]:
        assert abs(dx[i % c["N"], j % c["H"]].item() - v) <= gtol * dx_scale
    for i, j, v in g["dw_probes"]:
        assert abs(dw[i % c["H"], j % c["V"]].item() - v) <= gtol * dw_scale

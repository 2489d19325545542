"""Writes tests/golden/lce_golden.json: expected outputs of the operator on seeded inputs.

The reference ships no golden vectors for this path, so these come from the fp64 oracle, cross-checked here
against ``F.cross_entropy`` + autograd in fp64 before anything is written.  Inputs are NOT stored: they are
regenerated from the seed with ``tests/helpers.make_inputs`` (CPU ``torch.Generator``), so the file stays small.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from helpers import make_inputs  # noqa: E402
from oracle import lce_forward_backward_fp64  # noqa: E402

CASES = [
    dict(name="bf16_plain", N=512, H=256, V=4096, dtype="bfloat16", seed=101, ignore_frac=0.0, z_reg=0.0, scale=1.0),
    dict(name="bf16_ignore_zreg", N=512, H=256, V=4096, dtype="bfloat16", seed=102, ignore_frac=0.1, z_reg=1e-4, scale=1.0),
    dict(name="f16_scale_half", N=512, H=256, V=4096, dtype="float16", seed=103, ignore_frac=0.1, z_reg=1e-4, scale=0.5),
    dict(name="f16_zipf", N=1024, H=256, V=8192, dtype="float16", seed=104, ignore_frac=0.1, z_reg=0.0, scale=1.0, zipf=True),
    dict(name="f32_ignore_zreg", N=512, H=264, V=4104, dtype="float32", seed=105, ignore_frac=0.1, z_reg=1e-4, scale=1.0),
]
PROBES = [(0, 0), (1, 7), (17, 100), (255, 255), (100, 3)]


def main():
    out = {}
    for c in CASES:
        dt = getattr(torch, c["dtype"])
        x, y, w = make_inputs(c["N"], c["H"], c["V"], dt, c["seed"], ignore_frac=c["ignore_frac"], zipf=c.get("zipf", False))
        xd, wd = x.double(), w.double()
        r = lce_forward_backward_fp64(xd, y, wd, -1, c["z_reg"], c["scale"])
        # cross-check against the library definition before trusting the numbers
        xa, wa = xd.clone().requires_grad_(True), wd.clone().requires_grad_(True)
        z = (xa @ wa) * c["scale"]
        loss = F.cross_entropy(z, y, ignore_index=-1) + c["z_reg"] * z.logsumexp(-1)[y != -1].pow(2).mean()
        loss.backward()
        assert torch.allclose(loss.detach(), r.loss, rtol=1e-12)
        assert torch.allclose(xa.grad, r.dx, rtol=1e-9, atol=1e-14) and torch.allclose(wa.grad, r.dw, rtol=1e-9, atol=1e-14)
        out[c["name"]] = dict(
            config=c,
            n_valid=r.n_valid,
            loss=r.loss.item(), z_reg=r.z_reg.item(), logit_max=r.logit_max.item(),
            logit_entropy=r.logit_entropy.item(), logit_norm=r.logit_norm.item(),
            lse_head=r.lse[:16].tolist(),
            label_head=y[:16].tolist(),
            dx_sum=r.dx.sum().item(), dx_abs_sum=r.dx.abs().sum().item(), dx_norm=r.dx.norm().item(),
            dw_sum=r.dw.sum().item(), dw_abs_sum=r.dw.abs().sum().item(), dw_norm=r.dw.norm().item(),
            dx_probes=[[i, j, r.dx[i % c["N"], j % c["H"]].item()] for i, j in PROBES],
            dw_probes=[[i, j, r.dw[i % c["H"], j % c["V"]].item()] for i, j in PROBES],
        )
    with open(os.path.join(HERE, "lce_golden.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", len(out), "cases")


if __name__ == "__main__":
    main()

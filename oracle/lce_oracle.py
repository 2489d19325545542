"""fp64 restatement of the reference's linear + cross-entropy semantics.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  It runs on the CPU (or
on whatever device its inputs live on), evaluates everything in float64 and is
chunked over tokens so that the vocabulary-sized logits of a chunk are the
only large temporary.

What each function follows in the reference (paths relative to the reference
checkout):

* ``lce_forward_fp64``      -- ``linear_cross_entropy/ops.py:9-17`` (``reference_torch``:
  scaled logits, mean cross-entropy over valid tokens, z-regularisation term,
  max logit, mean entropy over valid tokens, mean logit norm over all tokens)
  and ``ops.py:212-213`` (a label equal to ``ignore_index`` never matches a
  column, even when ``ignore_index`` is a legal column).
* ``lce_forward_backward_fp64`` -- ``ops.py:309-314`` and ``ops.py:415-422``
  (``dz = softmax * (1 + 2*zreg*lse) - onehot``, ignored rows zeroed by
  selection), ``ops.py:332`` and ``ops.py:443-447`` (``/R * logit_scale`` after
  accumulation), ``ops.py:804-810`` (upstream gradient multiplies both).
* chunking protocol         -- ``bench_fusions.py:400-418`` (fp64 reference
  evaluated in row chunks).
* ``eager_fp32_step``       -- ``bench_fusions.py:30-33`` (the eager torch
  provider used as the baseline).
* ``eager_fp32_step_chunked`` -- the same step as an N-chunked eager loop
  (``bench_fusions.py:71-83`` without the checkpointing), for workloads whose
  N x V fp32 logits do not fit the host.

Pinning status: every function here is pinned by ``tests/test_oracle.py``
against library routines (``F.cross_entropy`` + autograd in fp64), central
finite differences, closed forms (W = 0, x = 0, row-sum invariants) and a
pure-Python brute force on tiny inputs.  The reference ships no golden
vectors for this path, so none are used.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class OracleResult:
    loss: torch.Tensor          # 0-dim float64
    z_reg: torch.Tensor         # 0-dim float64, mean over valid rows of lse^2
    logit_max: torch.Tensor     # 0-dim float64, max over ALL rows
    logit_entropy: torch.Tensor  # 0-dim float64, mean over valid rows
    logit_norm: torch.Tensor    # 0-dim float64, mean over ALL rows of ||z_i||_2
    lse: torch.Tensor           # (N,) float64
    n_valid: int
    dx: Optional[torch.Tensor] = None   # (N, H) float64
    dw: Optional[torch.Tensor] = None   # (H, V) float64


def _prep(x, y, w):
    x2 = x.reshape(-1, x.shape[-1]).to(torch.float64)
    y1 = y.reshape(-1).to(torch.int64)
    w2 = w.to(torch.float64)
    assert w2.shape[0] == x2.shape[1], "weight must be (H, V)"
    assert y1.shape[0] == x2.shape[0]
    return x2, y1, w2


def lce_forward_fp64(x, y, w, ignore_index=-100, z_regularization=0.0, logit_scale=1.0,
                     chunk=512) -> OracleResult:
    """Loss and monitoring metrics; ``w`` is the transposed (H, V) weight."""
    x2, y1, w2 = _prep(x, y, w)
    N, V = x2.shape[0], w2.shape[1]
    valid = y1 != ignore_index
    R = int(valid.sum().item())
    lse = torch.empty(N, dtype=torch.float64, device=x2.device)
    tgt = torch.zeros(N, dtype=torch.float64, device=x2.device)
    ent = torch.zeros(N, dtype=torch.float64, device=x2.device)
    nrm = torch.zeros(N, dtype=torch.float64, device=x2.device)
    zmax = torch.tensor(-math.inf, dtype=torch.float64, device=x2.device)
    for s in range(0, N, chunk):
        e = min(N, s + chunk)
        z = (x2[s:e] @ w2) * logit_scale
        l = torch.logsumexp(z, dim=-1)
        lse[s:e] = l
        yy = y1[s:e]
        ok = valid[s:e] & (yy >= 0) & (yy < V)
        idx = torch.where(ok, yy, torch.zeros_like(yy))
        tgt[s:e] = torch.where(ok, z.gather(1, idx[:, None])[:, 0], torch.zeros_like(l))
        logp = z - l[:, None]
        ent[s:e] = -(logp.exp() * logp).sum(-1)
        nrm[s:e] = z.pow(2).sum(-1).sqrt()
        zmax = torch.maximum(zmax, z.max())
    vf = valid.to(torch.float64)
    ce = ((lse - tgt) * vf).sum() / R if R > 0 else torch.tensor(math.nan, dtype=torch.float64)
    z_reg = (lse.pow(2) * vf).sum() / R if R > 0 else torch.tensor(math.nan, dtype=torch.float64)
    loss = ce + z_regularization * z_reg
    entropy = (ent * vf).sum() / R if R > 0 else torch.tensor(math.nan, dtype=torch.float64)
    return OracleResult(loss=loss, z_reg=z_reg, logit_max=zmax, logit_entropy=entropy,
                        logit_norm=nrm.mean(), lse=lse, n_valid=R)


def lce_forward_backward_fp64(x, y, w, ignore_index=-100, z_regularization=0.0, logit_scale=1.0,
                              grad_output=1.0, chunk=512) -> OracleResult:
    """Forward plus closed-form gradients ``dx`` (N, H) and ``dw`` (H, V)."""
    res = lce_forward_fp64(x, y, w, ignore_index, z_regularization, logit_scale, chunk)
    x2, y1, w2 = _prep(x, y, w)
    N, H = x2.shape
    V = w2.shape[1]
    R = res.n_valid
    valid = y1 != ignore_index
    dx = torch.zeros(N, H, dtype=torch.float64, device=x2.device)
    dw = torch.zeros(H, V, dtype=torch.float64, device=x2.device)
    coef = float(grad_output) * logit_scale / R if R > 0 else math.nan
    for s in range(0, N, chunk):
        e = min(N, s + chunk)
        z = (x2[s:e] @ w2) * logit_scale
        l = res.lse[s:e]
        p = (z - l[:, None]).exp()
        dz = p * (1.0 + 2.0 * z_regularization * l)[:, None]
        yy = y1[s:e]
        ok = valid[s:e] & (yy >= 0) & (yy < V)
        rows = torch.nonzero(ok)[:, 0]
        dz[rows, yy[rows]] -= 1.0
        dz = torch.where(valid[s:e, None], dz, torch.zeros_like(dz))
        dx[s:e] = (dz @ w2.t()) * coef
        dw += (x2[s:e].t() @ dz) * coef
    res.dx = dx.reshape(*x.shape[:-1], H)
    res.dw = dw
    return res


def lce_bruteforce(x, y, w, ignore_index=-100, z_regularization=0.0, logit_scale=1.0):
    """Pure-Python double loops (tiny inputs only): returns (loss, z_reg, lse list, n_valid)."""
    xs = x.reshape(-1, x.shape[-1]).tolist()
    ys = y.reshape(-1).tolist()
    ws = w.tolist()
    H, V = len(ws), len(ws[0])
    tot = 0.0
    tot2 = 0.0
    R = 0
    lses = []
    for i, row in enumerate(xs):
        z = [logit_scale * sum(row[h] * ws[h][v] for h in range(H)) for v in range(V)]
        m = max(z)
        l = m + math.log(sum(math.exp(t - m) for t in z))
        lses.append(l)
        if ys[i] == ignore_index:
            continue
        R += 1
        tot += l - (z[ys[i]] if 0 <= ys[i] < V else 0.0)
        tot2 += l * l
    if R == 0:
        return math.nan, math.nan, lses, 0
    return tot / R + z_regularization * tot2 / R, tot2 / R, lses, R


def eager_fp32_step(x, y, w, ignore_index=-100, z_regularization=0.0, logit_scale=1.0):
    """Eager fp32 linear + ``F.cross_entropy`` forward+backward (the CPU baseline).

    Returns (loss, dx, dw) as fp32 tensors.  Materialises the full logits, so
    callers bound N themselves.
    """
    import torch.nn.functional as F

    x32 = x.reshape(-1, x.shape[-1]).float().detach().requires_grad_(True)
    w32 = w.float().detach().requires_grad_(True)
    z = (x32 @ w32) * logit_scale
    y1 = y.reshape(-1)
    loss = F.cross_entropy(z, y1, ignore_index=ignore_index)
    if z_regularization > 0:
        loss = loss + z_regularization * torch.logsumexp(z, -1)[y1 != ignore_index].pow(2).mean()
    loss.backward()
    return loss.detach(), x32.grad, w32.grad


def eager_fp32_step_chunked(x, y, w, ignore_index=-100, z_regularization=0.0, logit_scale=1.0, chunk=2048):
    """The same step over all tokens, `chunk` rows at a time, so that only chunk x V logits exist at once:
    the mathematically identical N-chunked eager loop (the pattern of bench_fusions.py:71-83, without the
    checkpointing).  Every chunk's loss terms are summed and divided by the number of valid labels of the whole
    batch, its backward adds into the same dW, and its rows of dx are its own.  Returns (loss, dx, dw) in fp32.
    """
    import torch.nn.functional as F

    x2 = x.reshape(-1, x.shape[-1])
    y1 = y.reshape(-1)
    R = (y1 != ignore_index).sum()
    w32 = w.float().detach().requires_grad_(True)
    dx = torch.empty(x2.shape, dtype=torch.float32)
    loss = torch.zeros((), dtype=torch.float32)
    for r0 in range(0, x2.shape[0], chunk):
        xc = x2[r0:r0 + chunk].float().detach().requires_grad_(True)
        yc = y1[r0:r0 + chunk]
        z = (xc @ w32) * logit_scale
        part = F.cross_entropy(z, yc, ignore_index=ignore_index, reduction="sum")
        if z_regularization > 0:
            part = part + z_regularization * torch.logsumexp(z, -1)[yc != ignore_index].pow(2).sum()
        part = part / R
        part.backward()
        dx[r0:r0 + chunk] = xc.grad
        loss += part.detach()
    return loss, dx, w32.grad

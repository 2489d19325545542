"""Pins the fp64 oracle without the reference: library routines, finite differences, closed forms, brute force.

Each check is chosen so that a plausible mistake (dropped z-reg term, wrong sign, wrong mean denominator, a
transposed weight, ignored rows multiplied instead of selected) fails at least one of them.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import lce_forward_fp64, lce_forward_backward_fp64, lce_bruteforce


def _rand(N, H, V, seed, ignore_frac=0.25, ignore_index=-1):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, H, generator=g, dtype=torch.float64)
    w = torch.randn(H, V, generator=g, dtype=torch.float64) * 0.4
    y = torch.randint(0, V, (N,), generator=g)
    y[torch.rand(N, generator=g) < ignore_frac] = ignore_index
    if (y != ignore_index).sum() == 0:
        y[0] = 1
    return x, y, w


def _library(x, y, w, ignore_index, zreg, scale):
    """The reference's semantic definition (its reference_torch), written with library calls in fp64."""
    x = x.clone().requires_grad_(True)
    w = w.clone().requires_grad_(True)
    z = F.linear(x, w.t()) * scale            # reference_torch takes the (V, H) weight
    loss = F.cross_entropy(z, y, ignore_index=ignore_index)
    keep = y != ignore_index
    zr = z.logsumexp(-1)[keep].pow(2).mean()
    loss = loss + zreg * zr
    lp = torch.log_softmax(z, -1)[keep]
    ent = (-lp.exp() * lp).sum(-1).mean()
    return loss, zr, z.max(), ent, z.norm(dim=-1).mean(), x, w


@pytest.mark.parametrize("zreg,scale,ignore_index", [(0.0, 1.0, -1), (1e-2, 0.5, -100), (0.3, 2.0, 5)])
def test_matches_library_cross_entropy_and_autograd(zreg, scale, ignore_index):
    x, y, w = _rand(24, 16, 40, seed=7, ignore_index=ignore_index)
    loss, zr, zmax, ent, nrm, xg, wg = _library(x, y, w, ignore_index, zreg, scale)
    (loss * 1.3).backward()
    r = lce_forward_backward_fp64(x, y, w, ignore_index, zreg, scale, grad_output=1.3, chunk=7)
    assert r.n_valid == int((y != ignore_index).sum())
    assert torch.allclose(r.loss, loss.detach(), rtol=1e-12, atol=1e-12)
    assert torch.allclose(r.z_reg, zr.detach(), rtol=1e-12)
    assert torch.allclose(r.logit_max, zmax.detach(), rtol=1e-12)
    assert torch.allclose(r.logit_entropy, ent.detach(), rtol=1e-11)
    assert torch.allclose(r.logit_norm, nrm.detach(), rtol=1e-12)
    assert torch.allclose(r.dx, xg.grad, rtol=1e-10, atol=1e-13)
    assert torch.allclose(r.dw, wg.grad, rtol=1e-10, atol=1e-13)


def test_nonnegative_ignore_index_never_matches_a_column():
    x, y, w = _rand(16, 8, 12, seed=3, ignore_frac=0.0)
    y[:5] = 5
    r = lce_forward_backward_fp64(x, y, w, 5, 0.0, 1.0)
    assert r.n_valid == int((y != 5).sum())
    assert (r.dx[:5] == 0).all()
    loss = F.cross_entropy(x[5:] @ w, y[5:]) if (y[5:] != 5).all() else None
    if loss is not None:
        assert torch.allclose(r.loss, loss, rtol=1e-12)


def test_central_finite_differences():
    x, y, w = _rand(8, 16, 32, seed=11)
    zreg, scale = 0.05, 0.7
    r = lce_forward_backward_fp64(x, y, w, -1, zreg, scale)
    eps = 1e-6
    g = torch.Generator().manual_seed(0)
    for _ in range(6):
        i, h = int(torch.randint(0, 8, (1,), generator=g)), int(torch.randint(0, 16, (1,), generator=g))
        xp, xm = x.clone(), x.clone()
        xp[i, h] += eps
        xm[i, h] -= eps
        fd = (lce_forward_fp64(xp, y, w, -1, zreg, scale).loss - lce_forward_fp64(xm, y, w, -1, zreg, scale).loss) / (2 * eps)
        assert abs(fd - r.dx[i, h]) <= 1e-7 * max(1.0, abs(fd))
        h, v = int(torch.randint(0, 16, (1,), generator=g)), int(torch.randint(0, 32, (1,), generator=g))
        wp, wm = w.clone(), w.clone()
        wp[h, v] += eps
        wm[h, v] -= eps
        fd = (lce_forward_fp64(x, y, wp, -1, zreg, scale).loss - lce_forward_fp64(x, y, wm, -1, zreg, scale).loss) / (2 * eps)
        assert abs(fd - r.dw[h, v]) <= 1e-7 * max(1.0, abs(fd))


def test_bruteforce_loops_tiny():
    x, y, w = _rand(6, 5, 9, seed=5)
    for zreg, scale in ((0.0, 1.0), (0.2, 1.5)):
        loss, zr, lses, R = lce_bruteforce(x, y, w, -1, zreg, scale)
        r = lce_forward_fp64(x, y, w, -1, zreg, scale)
        assert R == r.n_valid
        assert abs(loss - r.loss.item()) < 1e-12
        assert abs(zr - r.z_reg.item()) < 1e-12
        assert torch.allclose(torch.tensor(lses, dtype=torch.float64), r.lse, rtol=1e-13)


def test_closed_form_zero_weight():
    N, H, V, lam = 10, 4, 16, 0.3
    x, y, _ = _rand(N, H, V, seed=1)
    w = torch.zeros(H, V, dtype=torch.float64)
    r = lce_forward_backward_fp64(x, y, w, -1, lam, 1.0)
    logV = math.log(V)
    assert torch.allclose(r.lse, torch.full((N,), logV, dtype=torch.float64), rtol=1e-14)
    assert abs(r.loss.item() - (logV + lam * logV ** 2)) < 1e-12
    assert abs(r.logit_entropy.item() - logV) < 1e-12
    assert r.logit_max.item() == 0.0 and r.logit_norm.item() == 0.0
    assert (r.dx == 0).all()   # W = 0 => dz W^T = 0


def test_closed_form_zero_input():
    N, H, V, lam, s = 12, 6, 20, 0.1, 0.8
    _, y, w = _rand(N, H, V, seed=2)
    x = torch.zeros(N, H, dtype=torch.float64)
    r = lce_forward_backward_fp64(x, y, w, -1, lam, s)
    R = r.n_valid
    assert (r.dw == 0).all()
    logV = math.log(V)
    for i in range(N):
        if y[i] == -1:
            assert (r.dx[i] == 0).all()
        else:
            want = (s / R) * ((1 + 2 * lam * logV) * w.mean(1) - w[:, y[i]])
            assert torch.allclose(r.dx[i], want, rtol=1e-12, atol=1e-15)


def test_row_sum_invariants():
    x, y, w = _rand(16, 8, 24, seed=9)
    # zreg = 0: every dz row sums to 0, so dW summed over columns vanishes
    r0 = lce_forward_backward_fp64(x, y, w, -1, 0.0, 1.0)
    assert r0.dw.sum(1).abs().max() < 1e-14
    # zreg = lam: the dz row sum is 2*lam*lse_i/R for valid rows
    lam = 0.2
    r1 = lce_forward_backward_fp64(x, y, w, -1, lam, 1.0)
    valid = (y != -1).double()
    want = x.t() @ (2 * lam * r1.lse * valid / r1.n_valid)
    assert torch.allclose(r1.dw.sum(1), want, rtol=1e-10, atol=1e-14)


def test_scaling_permutation_and_chunk_invariance():
    x, y, w = _rand(32, 8, 24, seed=13)
    a = lce_forward_backward_fp64(x, y, w, -1, 0.1, 0.9, grad_output=1.0, chunk=32)
    b = lce_forward_backward_fp64(x, y, w, -1, 0.1, 0.9, grad_output=2.5, chunk=5)
    assert torch.allclose(b.dx, 2.5 * a.dx, rtol=1e-12) and torch.allclose(b.dw, 2.5 * a.dw, rtol=1e-12)
    perm = torch.randperm(32, generator=torch.Generator().manual_seed(0))
    c = lce_forward_backward_fp64(x[perm], y[perm], w, -1, 0.1, 0.9)
    assert torch.allclose(c.loss, a.loss, rtol=1e-13)
    assert torch.allclose(c.dx, a.dx[perm], rtol=1e-12)
    assert torch.allclose(c.dw, a.dw, rtol=1e-11, atol=1e-15)


def test_ignored_rows_are_selected_not_multiplied():
    x, y, w = _rand(16, 8, 24, seed=17, ignore_frac=0.4)
    a = lce_forward_backward_fp64(x, y, w, -1, 0.05, 1.0)
    xg = x.clone()
    xg[y == -1] = 1e30   # finite garbage in ignored rows
    b = lce_forward_backward_fp64(xg, y, w, -1, 0.05, 1.0)
    assert torch.equal(a.loss, b.loss)
    assert torch.equal(a.dx, b.dx)
    assert (b.dx[y == -1] == 0).all()
    assert torch.equal(a.dw, b.dw)


def test_all_ignored_gives_nan_like_cross_entropy():
    x, y, w = _rand(4, 4, 8, seed=19)
    y[:] = -1
    r = lce_forward_fp64(x, y, w, -1, 0.0, 1.0)
    assert r.n_valid == 0 and math.isnan(r.loss.item())
    assert math.isnan(F.cross_entropy(x @ w, y, ignore_index=-1).item())


@pytest.mark.parametrize("zreg,scale,ignore_index", [(0.0, 1.0, -1), (1e-2, 0.5, -1), (0.3, 2.0, 5)])
def test_eager_fp32_step_is_the_same_function_in_single_precision(zreg, scale, ignore_index):
    """The CPU baseline (eager fp32 matmul + F.cross_entropy through autograd) against the fp64 closed forms:
    same loss and gradients up to fp32 rounding, with z-regularisation and ignored labels present."""
    from oracle import eager_fp32_step

    x, y, w = _rand(48, 24, 40, seed=17, ignore_frac=0.3, ignore_index=ignore_index)
    ref = lce_forward_backward_fp64(x, y, w, ignore_index, zreg, scale)
    loss, dx, dw = eager_fp32_step(x, y, w, ignore_index, zreg, scale)
    assert loss.dtype == torch.float32 and dx.dtype == torch.float32 and dw.dtype == torch.float32
    assert abs(loss.item() - ref.loss.item()) <= 1e-5 * abs(ref.loss.item())
    assert torch.allclose(dx.double(), ref.dx, rtol=1e-4, atol=1e-6 * ref.dx.abs().max().item())
    assert torch.allclose(dw.double(), ref.dw, rtol=1e-4, atol=1e-6 * ref.dw.abs().max().item())
    assert (dx[y == ignore_index] == 0).all()
    # a dropped z-reg term or a wrong sign would not survive this: the two differ visibly when zreg changes
    if zreg > 0:
        loss0, dx0, _ = eager_fp32_step(x, y, w, ignore_index, 0.0, scale)
        assert abs(loss0.item() - loss.item()) > 1e-3 * abs(loss.item())
        assert (dx0 - dx).abs().max() > 1e-3 * dx.abs().max()


@pytest.mark.parametrize("zreg,scale,ignore_index,chunk", [(0.0, 1.0, -1, 16), (1e-2, 0.5, -1, 7), (0.3, 2.0, 5, 48), (0.0, 1.0, -1, 1000)])
def test_chunked_eager_fp32_step_equals_the_unchunked_one(zreg, scale, ignore_index, chunk):
    """The N-chunked form of the CPU baseline (what bench.py times on the whole workload): same loss and gradients
    as the unchunked step up to fp32 summation order and as the fp64 closed forms, for chunk sizes that divide the
    token count, that do not, and that exceed it; a chunk whose labels are all ignored contributes exact zeros."""
    from oracle import eager_fp32_step, eager_fp32_step_chunked

    x, y, w = _rand(48, 24, 40, seed=23, ignore_frac=0.3, ignore_index=ignore_index)
    y[:7] = ignore_index  # the first chunk of 7 holds no valid label
    ref = lce_forward_backward_fp64(x, y, w, ignore_index, zreg, scale)
    loss1, dx1, dw1 = eager_fp32_step(x, y, w, ignore_index, zreg, scale)
    loss, dx, dw = eager_fp32_step_chunked(x, y, w, ignore_index, zreg, scale, chunk=chunk)
    assert loss.dtype == torch.float32 and dx.dtype == torch.float32 and dw.dtype == torch.float32
    assert abs(loss.item() - loss1.item()) <= 1e-5 * abs(loss1.item())
    assert abs(loss.item() - ref.loss.item()) <= 1e-5 * abs(ref.loss.item())
    for got, one, want in ((dx, dx1, ref.dx), (dw, dw1, ref.dw)):
        assert torch.allclose(got, one, rtol=1e-4, atol=1e-6 * one.abs().max().item())
        assert torch.allclose(got.double(), want, rtol=1e-4, atol=1e-6 * want.abs().max().item())
    assert (dx[y == ignore_index] == 0).all()

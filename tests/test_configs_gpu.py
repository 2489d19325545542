"""The benchmark configurations at their own sizes, against the fp64 oracle evaluated on the GPU.

config 3: fp16, N=16384, H=4096, V=131072, logit_scale 0.5, z-regularisation 1e-4, monitoring, Zipf(1.1)
          labels, 10 % ignored.
config 4: bf16, N=16384, H=2048, V in {32768, 65536, 131072, 262144} x N_chunk_size in {2048, 4096, 8192}:
          every V against the oracle at N_chunk_size 4096, the other points through properties that do not
          depend on the size (loss ~ log V + 1/2, sum_v dW = 0, invariance under N_chunk_size) and every
          point's scratch against its bound N_chunk_size * V * 4 bytes.
config 5: fp16 activations, fp32 master weight (8192, 262144), N=65536, N_chunk_size 8192, fp32 dW.

Inputs follow the recipes of the benchmark (x ~ N(0,1), W truncated normal with std 1/sqrt(H), seeds 3/4/5),
generated on the device.  Tolerances: loss 1e-3 relative, gradients 2e-2 as max|d|/max|ref| and as L2 ratio.
"""
import math

import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.pack_auto]

LOSS_RTOL = 1e-3
GRAD_TOL = 2e-2


def _inputs(N, H, V, dtype, seed, ignore, zipf=False, w_dtype=None):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(N, H, device="cuda", generator=g, dtype=torch.float32).to(dtype)
    std = 1.0 / math.sqrt(H)
    w = torch.empty(H, V, device="cuda", dtype=torch.float32)
    torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-3 * std, b=3 * std, generator=g)
    if w_dtype is None:
        w = w.to(dtype)
    if zipf:
        p = torch.arange(1, V + 1, dtype=torch.float64, device="cuda") ** -1.1
        cdf = torch.cumsum(p, 0) / p.sum()
        y = torch.searchsorted(cdf, torch.rand(N, device="cuda", generator=g, dtype=torch.float64)).clamp_(max=V - 1)
    else:
        y = torch.randint(0, V, (N,), device="cuda", generator=g)
    if ignore > 0:
        y[torch.rand(N, device="cuda", generator=g) < ignore] = -1
    return x, y, w


def _step(x, y, w, z_reg, scale, n_chunk, mon, g=1.0):
    """One forward + backward; also the peak of device memory beyond the inputs and the two gradients."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    xd = x.detach().requires_grad_(True)
    wd = w.detach().requires_grad_(True)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    out = linear_cross_entropy(xd, y, wd, -1, z_reg, scale, n_chunk, mon)
    (out[0] * g).backward()
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    grads = xd.grad.numel() * xd.grad.element_size() + wd.grad.numel() * wd.grad.element_size()
    return [o.detach() for o in out], xd.grad, wd.grad, peak - grads


def _errors(got, want, rows=1024):
    """(max|d|/max|ref|, ||d||_2/||ref||_2) of a large matrix against its fp64 reference, in row blocks."""
    dmax = rmax = 0.0
    d2 = r2 = 0.0
    for s in range(0, got.shape[0], rows):
        r = want[s:s + rows]
        d = got[s:s + rows].double() - r
        dmax = max(dmax, d.abs().max().item())
        rmax = max(rmax, r.abs().max().item())
        d2 += d.pow(2).sum().item()
        r2 += r.pow(2).sum().item()
    return dmax / rmax, math.sqrt(d2 / r2)


def _check_against_oracle(out, dx, dw, ref, y, mon):
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item()), (out[0].item(), ref.loss.item())
    assert abs(out[1].item() - ref.z_reg.item()) <= LOSS_RTOL * abs(ref.z_reg.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    for name, got, want in (("dx", dx, ref.dx), ("dw", dw, ref.dw)):
        emax, el2 = _errors(got, want)
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (name, emax, el2)
    assert (dx[y == -1] == 0).all()


def test_config3_fp16_all_features_full_size():
    from oracle import lce_forward_backward_fp64

    print("config 3: N=16384 H=4096 V=131072 fp16, scale 0.5, z-reg 1e-4, monitoring, Zipf labels, 10 % ignored",
          flush=True)
    N, H, V = 16384, 4096, 131072
    x, y, w = _inputs(N, H, V, torch.float16, seed=3, ignore=0.10, zipf=True)
    # A mean loss over 14.7k tokens has dx entries of order 1e-6, far below fp16's normal range (6.1e-5): like
    # any fp16 training step the backward runs under a loss scale (torch.amp.GradScaler starts at 65536; 4096
    # here), which enters as the upstream gradient of the loss.
    S = 4096.0
    out, dx, dw, extra = _step(x, y, w, 1e-4, 0.5, 4096, True, g=S)
    assert dx.dtype == torch.float16 and dw.dtype == torch.float16
    assert extra <= 4096 * V * 4, extra
    ref = lce_forward_backward_fp64(x, y, w, -1, 1e-4, 0.5, grad_output=S, chunk=1024)
    assert ref.n_valid == int((y != -1).sum().item())
    _check_against_oracle(out, dx, dw, ref, y, True)
    del ref
    # Without the loss scale the same gradients come out rounded to fp16's subnormal grid (spacing 2^-24): each
    # entry is within half a grid step (plus fp16's relative half ulp) of the scaled run's value.
    _, dx1, dw1, _ = _step(x, y, w, 1e-4, 0.5, 4096, True)
    for got, scaled in ((dx1, dx), (dw1, dw)):
        want = scaled.float() / S
        assert ((got.float() - want).abs() <= 2.0 ** -25 * 1.001 + 2.0 ** -10 * want.abs()).all()
    torch.cuda.empty_cache()


def test_config5_long_sequence_fp32_master_weight_full_size():
    from oracle import lce_forward_backward_fp64

    print("config 5: N=65536 H=8192 V=262144, fp16 x, fp32 master W, N_chunk 8192, fp32 dW, Zipf, 10 % ignored",
          flush=True)
    N, H, V = 65536, 8192, 262144
    x, y, w = _inputs(N, H, V, torch.float16, seed=5, ignore=0.10, zipf=True, w_dtype=torch.float32)
    assert w.dtype == torch.float32
    S = 4096.0  # loss scale, as in the fp16 case above: the fp16 dx of a mean over 59k tokens is of order 1e-7
    out, dx, dw, extra = _step(x, y, w, 0.0, 1.0, 8192, False, g=S)
    print(f"  loss {out[0].item():.5f}; scratch {extra / 2**30:.2f} GiB of {8192 * V * 4 / 2**30:.0f} GiB", flush=True)
    assert dx.dtype == torch.float16 and dw.dtype == torch.float32
    assert extra <= 8192 * V * 4, extra
    ref = lce_forward_backward_fp64(x, y, w, -1, 0.0, 1.0, grad_output=S, chunk=1024)
    _check_against_oracle(out, dx, dw, ref, y, False)
    del ref, dx, dw, x, w
    torch.cuda.empty_cache()


def test_long_hidden_size_with_activations_beyond_the_infinity_cache():
    """N=16384, H=8192, V=65536, bf16: a chunk of x is 256 MiB, so the forward runs as two launches of 32768
    columns, and a band of W tiles is 32 MiB, so forward and dz keep two bands in flight instead of eight (the
    tile order of lce_gemm.h) -- paths no benchmark configuration with a 16-bit weight takes."""
    from oracle import lce_forward_backward_fp64

    print("N=16384 H=8192 V=65536 bf16, 5 % ignored", flush=True)
    N, H, V = 16384, 8192, 65536
    x, y, w = _inputs(N, H, V, torch.bfloat16, seed=8, ignore=0.05)
    out, dx, dw, extra = _step(x, y, w, 1e-4, 1.0, 4096, True)
    assert extra <= 4096 * V * 4 + N * H * 4, extra  # (the bound is widened by the fp32 running dx when it cannot be met)
    ref = lce_forward_backward_fp64(x, y, w, -1, 1e-4, 1.0, chunk=1024)
    _check_against_oracle(out, dx, dw, ref, y, True)
    del ref, dx, dw, x, w
    torch.cuda.empty_cache()


# config 4: inputs of one vocabulary size at a time, and what the N_chunk_size = 4096 point of that size gave
_c4 = {}


def _c4_inputs(V):
    if _c4.get("V") != V:
        _c4.clear()
        torch.cuda.empty_cache()
        x, y, w = _inputs(16384, 2048, V, torch.bfloat16, seed=4, ignore=0.0)
        _c4.update(V=V, x=x, y=y, w=w)
    return _c4["x"], _c4["y"], _c4["w"]


@pytest.mark.parametrize("n_chunk", [4096, 2048, 8192])  # (varies fastest; 4096, the oracle-checked point, first)
@pytest.mark.parametrize("V", [32768, 65536, 131072, 262144])
def test_config4_vocabulary_sweep_point(V, n_chunk):
    from oracle import lce_forward_backward_fp64

    print(f"config 4: V={V} N_chunk_size={n_chunk}", flush=True)
    N, H = 16384, 2048
    x, y, w = _c4_inputs(V)
    out, dx, dw, extra = _step(x, y, w, 0.0, 1.0, n_chunk, False)
    budget = n_chunk * V * 4
    print(f"  loss {out[0].item():.5f}; scratch {extra / 2**20:.0f} MiB of {budget / 2**20:.0f} MiB", flush=True)
    assert extra <= budget, (extra, budget)
    # logits ~ N(0, ~1), uniform labels: loss ~ log V + 1/2
    assert abs(out[0].item() - (math.log(V) + 0.5)) < 0.05
    # without z-regularisation every row of dz sums to zero, so every row of dW does (up to the rounding of
    # its stored 16-bit entries)
    s = dw.float().sum(1).abs().max().item()
    a = dw.float().abs().sum(1).max().item()
    assert s <= 2e-3 * a, (s, a)
    assert torch.isfinite(dx.float()).all() and torch.isfinite(dw.float()).all()
    if n_chunk == 4096:
        ref = lce_forward_backward_fp64(x, y, w, -1, 0.0, 1.0, chunk=1024)
        _check_against_oracle(out, dx, dw, ref, y, False)
        del ref
        _c4["at4096"] = (out[0].clone(), dx, dw)
    else:
        # N_chunk_size only moves the vocabulary split of the backward: the loss does not depend on it at all;
        # dx is summed over the slabs in fp32 and dW tiles of a narrow slab are cut along the tokens, so both
        # move by the order of an fp32 sum and one rounding to bf16
        loss0, dx0, dw0 = _c4["at4096"]
        assert torch.equal(out[0], loss0)
        for got, want in ((dx, dx0), (dw, dw0)):
            emax, el2 = _errors(got, want.double())
            assert emax <= 1e-2 and el2 <= 2e-3, (emax, el2)
    torch.cuda.empty_cache()

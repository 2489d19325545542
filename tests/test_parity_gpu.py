"""GPU parity: the HIP path (through the C ABI) against the fp64 oracle on identical seeded inputs.

Tolerances (the ones the operator is specified to): loss within 1e-3 relative; dx and dW within 2e-2 both
as max_abs(diff)/max_abs(ref) and as an L2 ratio, for 16-bit compute; valid-token count and ignore_index
masking bit-exact.
"""
import pytest
import torch

from helpers import make_inputs, rel_errors

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-3
GRAD_TOL = 2e-2


def _run(x, y, w, ignore_index, z_reg, scale, n_chunk, monitoring, grad_output=1.0):
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    xd = x.cuda().requires_grad_(True)
    wd = w.cuda().requires_grad_(True)
    out = linear_cross_entropy(xd, y.cuda(), wd, ignore_index, z_reg, scale, n_chunk, monitoring)
    (out[0] * grad_output).backward()
    torch.cuda.synchronize()
    return out, xd.grad, wd.grad


def _oracle(x, y, w, ignore_index, z_reg, scale, grad_output=1.0):
    from oracle import lce_forward_backward_fp64

    return lce_forward_backward_fp64(x.double(), y, w.double(), ignore_index, z_reg, scale, grad_output)


CASES = [
    # N, H, V, dtype, w_dtype, ignore_frac, z_reg, scale, n_chunk, monitoring
    (512, 256, 4096, torch.bfloat16, None, 0.0, 0.0, 1.0, 512, False),
    (512, 256, 4096, torch.float16, None, 0.1, 1e-4, 0.5, 512, True),
    (1024, 512, 8192, torch.bfloat16, None, 0.05, 0.0, 1.0, 512, True),
    (1024, 512, 8192, torch.float16, torch.float32, 0.1, 1e-3, 2.0, 512, False),
    (512, 768, 4096, torch.bfloat16, torch.float32, 0.0, 1e-2, 1.0, 4096, True),
    (512, 256, 4096, torch.float32, None, 0.05, 1e-4, 1.0, 512, True),
    (2048, 256, 12288, torch.bfloat16, None, 0.5, 0.0, 0.7, 512, False),
]


@pytest.mark.parametrize("N,H,V,dtype,w_dtype,ign,z_reg,scale,n_chunk,mon", CASES)
def test_forward_backward_matches_oracle(N, H, V, dtype, w_dtype, ign, z_reg, scale, n_chunk, mon):
    print(f"case N={N} H={H} V={V} {dtype} w={w_dtype} ign={ign} zreg={z_reg} scale={scale} chunk={n_chunk}",
          flush=True)
    x, y, w = make_inputs(N, H, V, dtype, seed=N + H + V, ignore_frac=ign, w_dtype=w_dtype)
    out, dx, dw = _run(x, y, w, -1, z_reg, scale, n_chunk, mon, grad_output=1.7)
    ref = _oracle(x, y, w, -1, z_reg, scale, grad_output=1.7)
    loss = out[0].item()
    assert abs(loss - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item()), (loss, ref.loss.item())
    assert abs(out[1].item() - ref.z_reg.item()) <= LOSS_RTOL * abs(ref.z_reg.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-2 * abs(ref.logit_max.item()) + 1e-3
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    else:
        assert out[2].item() == 0 and out[3].item() == 0 and out[4].item() == 0
    assert dx.dtype == x.dtype and dw.dtype == w.dtype
    for name, got, want in (("dx", dx, ref.dx), ("dw", dw, ref.dw)):
        emax, el2 = rel_errors(got, want)
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (name, emax, el2)
    # bit-exact masking
    ignored = (y == -1)
    if ignored.any():
        assert (dx.cpu()[ignored] == 0).all()
        assert torch.equal(dx.cpu()[ignored].view(torch.int16 if dx.element_size() == 2 else torch.int32),
                           torch.zeros_like(dx.cpu()[ignored]).view(
                               torch.int16 if dx.element_size() == 2 else torch.int32))


MID_CASES = [
    # N, H, V, dtype, w_dtype, zipf, ignore_frac, z_reg, scale, n_chunk, monitoring
    (2048, 1024, 32768, torch.float16, None, True, 0.1, 1e-4, 0.5, 4096, True),        # config-3 style: all features
    (2048, 1024, 32768, torch.float16, torch.float32, True, 0.1, 0.0, 1.0, 512, False),  # config-5 style: fp32 master W
    (4096, 512, 65536, torch.bfloat16, None, False, 0.05, 0.0, 1.0, 512, False),        # several vocabulary slabs
    (2048, 2048, 16384, torch.float32, None, False, 0.0, 0.0, 1.0, 4096, False),        # config 1 (fp32 tensors)
]


@pytest.mark.parametrize("N,H,V,dtype,w_dtype,zipf,ign,z_reg,scale,n_chunk,mon", MID_CASES)
def test_mid_size_matches_fp64_oracle_evaluated_on_gpu(N, H, V, dtype, w_dtype, zipf, ign, z_reg, scale, n_chunk, mon):
    """Same comparison as above at sizes where the oracle is evaluated in fp64 on the GPU (row chunks)."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy
    from oracle import lce_forward_backward_fp64

    print(f"mid case N={N} H={H} V={V} {dtype} w={w_dtype} zipf={zipf} ign={ign} zreg={z_reg} scale={scale} "
          f"chunk={n_chunk}", flush=True)
    x, y, w = make_inputs(N, H, V, dtype, seed=7 * N + V, ignore_frac=ign, zipf=zipf, w_dtype=w_dtype, device="cuda")
    xd = x.clone().requires_grad_(True)
    wd = w.clone().requires_grad_(True)
    out = linear_cross_entropy(xd, y, wd, -1, z_reg, scale, n_chunk, mon)
    out[0].backward()
    torch.cuda.synchronize()
    ref = lce_forward_backward_fp64(x, y, w, -1, z_reg, scale, chunk=512)
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-2 * abs(ref.logit_max.item()) + 1e-3
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    for name, got, want in (("dx", xd.grad, ref.dx), ("dw", wd.grad, ref.dw)):
        d = got.double() - want
        emax = (d.abs().max() / want.abs().max()).item()
        el2 = (d.norm() / want.norm()).item()
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (name, emax, el2)
    assert (xd.grad[y == -1] == 0).all()

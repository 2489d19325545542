"""GPU parity: the HIP path (through the C ABI) against the fp64 oracle on identical seeded inputs.

Tolerances (the ones the operator is specified to): loss within 1e-3 relative; dx and dW within 2e-2 both
as max_abs(diff)/max_abs(ref) and as an L2 ratio, for 16-bit compute; valid-token count and ignore_index
masking bit-exact.  fp32 tensors are computed as bf16 pairs (16 bits of mantissa, better than the tf32
products the reference's tl.dot uses for fp32 tensors, ops.py:195) and are held to 1e-5 on the loss and
1e-3 on the gradients.
"""
import pytest
import torch

from helpers import make_inputs, rel_errors

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-3
GRAD_TOL = 2e-2


def _tols(dtype):
    """(loss, gradient) tolerance for tensors of `dtype`."""
    return (1e-5, 1e-3) if dtype == torch.float32 else (LOSS_RTOL, GRAD_TOL)


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
    (512, 16384, 4096, torch.bfloat16, None, 0.1, 1e-4, 1.0, 512, True),              # a hidden size beyond any config's
    (256, 12288, 2048, torch.float16, torch.float32, 0.0, 0.0, 1.0, 4096, False),
]


@pytest.mark.parametrize("N,H,V,dtype,w_dtype,ign,z_reg,scale,n_chunk,mon", CASES)
def test_forward_backward_matches_oracle(N, H, V, dtype, w_dtype, ign, z_reg, scale, n_chunk, mon):
    print(f"case N={N} H={H} V={V} {dtype} w={w_dtype} ign={ign} zreg={z_reg} scale={scale} chunk={n_chunk}",
          flush=True)
    x, y, w = make_inputs(N, H, V, dtype, seed=N + H + V, ignore_frac=ign, w_dtype=w_dtype)
    out, dx, dw = _run(x, y, w, -1, z_reg, scale, n_chunk, mon, grad_output=1.7)
    ref = _oracle(x, y, w, -1, z_reg, scale, grad_output=1.7)
    loss = out[0].item()
    loss_tol, grad_tol = _tols(dtype)
    assert abs(loss - ref.loss.item()) <= loss_tol * abs(ref.loss.item()), (loss, ref.loss.item())
    assert abs(out[1].item() - ref.z_reg.item()) <= loss_tol * abs(ref.z_reg.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    else:
        assert out[2].item() == 0 and out[3].item() == 0 and out[4].item() == 0
    assert dx.dtype == x.dtype and dw.dtype == w.dtype
    for name, got, want in (("dx", dx, ref.dx), ("dw", dw, ref.dw)):
        emax, el2 = rel_errors(got, want)
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= grad_tol and el2 <= grad_tol, (name, emax, el2)
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
    (300001, 72, 1000, torch.bfloat16, None, False, 0.2, 1e-4, 1.0, 512, True),         # many tokens: 19 forward chunks
    (131073, 64, 520, torch.float16, torch.float32, True, 0.5, 0.0, 2.0, 64, False),     # fp32 W: 3 forward chunks
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
    loss_tol, grad_tol = _tols(dtype)
    assert abs(out[0].item() - ref.loss.item()) <= loss_tol * abs(ref.loss.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    for name, got, want in (("dx", xd.grad, ref.dx), ("dw", wd.grad, ref.dw)):
        d = got.double() - want
        emax = (d.abs().max() / want.abs().max()).item()
        el2 = (d.norm() / want.norm()).item()
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= grad_tol and el2 <= grad_tol, (name, emax, el2)
    assert (xd.grad[y == -1] == 0).all()


# ---------------------------------------------------------------------------------------------------------
# Shapes that are not multiples of the tile sizes (the reference refuses them, ops.py:689-691, and names
# them as an open caveat, README.md:30).  Covers: token / vocabulary / hidden tails, a hidden size below
# one K loop, sizes that are not multiples of 8 (padded row strides), a single row, several uneven
# vocabulary slabs, strided inputs, a target in the last valid column, fp32 tensors, fp32 master weight.
# ---------------------------------------------------------------------------------------------------------
ODD_CASES = [
    # N, H, V, dtype, w_dtype, ignore_frac, z_reg, scale, n_chunk, monitoring
    (1000, 520, 5000, torch.bfloat16, None, 0.05, 0.0, 1.0, 4096, False),
    (777, 264, 10008, torch.float16, None, 0.1, 1e-4, 0.5, 512, True),
    (300, 100, 1001, torch.bfloat16, None, 0.1, 1e-3, 1.0, 4096, True),
    (1, 8, 8, torch.bfloat16, None, 0.0, 0.0, 1.0, 4096, True),
    (33, 72, 263, torch.float16, None, 0.0, 0.0, 2.0, 16, False),
    (513, 1024, 4104, torch.float32, None, 0.05, 1e-4, 1.0, 512, True),
    (640, 328, 3003, torch.float16, torch.float32, 0.1, 0.0, 1.0, 64, False),
    (2049, 136, 2500, torch.bfloat16, None, 0.3, 0.0, 0.7, 32, True),
    (257, 101, 515, torch.bfloat16, None, 0.0, 0.0, 1.0, 4096, True),
    (130, 77, 333, torch.float32, None, 0.1, 1e-3, 1.0, 4096, False),
]


@pytest.mark.parametrize("N,H,V,dtype,w_dtype,ign,z_reg,scale,n_chunk,mon", ODD_CASES)
def test_arbitrary_shapes_match_oracle(N, H, V, dtype, w_dtype, ign, z_reg, scale, n_chunk, mon):
    print(f"odd case N={N} H={H} V={V} {dtype} w={w_dtype} ign={ign} zreg={z_reg} scale={scale} chunk={n_chunk}",
          flush=True)
    x, y, w = make_inputs(N, H, V, dtype, seed=N + H + V, ignore_frac=ign, w_dtype=w_dtype)
    y[0] = V - 1  # a target in the last valid column
    out, dx, dw = _run(x, y, w, -1, z_reg, scale, n_chunk, mon, grad_output=0.9)
    ref = _oracle(x, y, w, -1, z_reg, scale, grad_output=0.9)
    loss_tol, grad_tol = _tols(dtype)
    assert abs(out[0].item() - ref.loss.item()) <= loss_tol * abs(ref.loss.item()), (out[0].item(), ref.loss.item())
    assert abs(out[1].item() - ref.z_reg.item()) <= loss_tol * abs(ref.z_reg.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item()) + 1e-4
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    assert dx.shape == x.shape and dw.shape == w.shape and dx.dtype == x.dtype and dw.dtype == w.dtype
    for name, got, want in (("dx", dx, ref.dx), ("dw", dw, ref.dw)):
        emax, el2 = rel_errors(got, want)
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= grad_tol and el2 <= grad_tol, (name, emax, el2)
    ignored = (y == -1)
    if ignored.any():
        assert (dx.cpu()[ignored] == 0).all()


def test_a_vocabulary_of_a_million_columns():
    """V = 1000003 (not a multiple of anything), few tokens: 3907 vocabulary tiles per token tile, a target in the
    last column, many vocabulary slabs under a small N_chunk_size; oracle in fp64 on the GPU."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy
    from oracle import lce_forward_backward_fp64

    print("vocabulary of 1000003", flush=True)
    N, H, V = 300, 128, 1000003
    x, y, w = make_inputs(N, H, V, torch.bfloat16, seed=1000003, ignore_frac=0.1, device="cuda")
    y[0] = V - 1
    xd = x.clone().requires_grad_(True)
    wd = w.clone().requires_grad_(True)
    out = linear_cross_entropy(xd, y, wd, -1, 1e-4, 1.0, 64, True)
    out[0].backward()
    ref = lce_forward_backward_fp64(x, y, w, -1, 1e-4, 1.0, chunk=64)
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item())
    assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
    for name, got, want in (("dx", xd.grad, ref.dx), ("dw", wd.grad, ref.dw)):
        d = got.double() - want
        emax = (d.abs().max() / want.abs().max()).item()
        el2 = (d.norm() / want.norm()).item()
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (name, emax, el2)
    assert (xd.grad[y == -1] == 0).all()


def test_strided_inputs_and_garbage_in_the_stride_padding():
    """x and W handed over as views with padded row strides whose padding holds large finite garbage: the
    result must be bit-identical to the dense call (the kernels never let the padding reach a valid output)."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("strided inputs", flush=True)
    N, H, V = 700, 200, 3000
    x, y, w = make_inputs(N, H, V, torch.bfloat16, seed=5, ignore_frac=0.1, device="cuda")
    xs = torch.full((N, H + 24), 1e30, dtype=x.dtype, device="cuda")
    ws = torch.full((H, V + 40), -1e30, dtype=w.dtype, device="cuda")
    xs[:, :H] = x
    ws[:, :V] = w
    res = []
    for xi, wi in ((x, w), (xs[:, :H], ws[:, :V])):
        xi = xi.detach().requires_grad_(True)
        wi = wi.detach().requires_grad_(True)
        out = linear_cross_entropy(xi, y, wi, -1, 1e-4, 1.0, 256, True)
        out[0].backward()
        res.append((torch.stack(out).detach(), xi.grad[:, :H].clone(), wi.grad[:, :V].clone()))
    for a, b in zip(res[0], res[1]):
        assert torch.equal(a, b)


def test_nothing_is_read_past_the_last_row_of_the_inputs():
    """x and W whose memory ends with the last element of their last row (row length not a multiple of 8, so the
    row stride has padding): what would be the stride padding of the LAST row lies outside the matrices and holds
    NaN here.  The results must be those of the dense call, bit for bit, with and without packed rows."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("last row ends the matrix", flush=True)
    N, H, V = 600, 100, 1004
    x, y, w = make_inputs(N, H, V, torch.float16, seed=15, ignore_frac=0.25, device="cuda")
    y[N - 1] = 3  # the last token is kept, so its row is gathered when rows are packed
    ldx, ldw = 104, 1008
    xbuf = torch.zeros(N * ldx, dtype=x.dtype, device="cuda")
    wbuf = torch.zeros(H * ldw, dtype=w.dtype, device="cuda")
    xs = xbuf.as_strided((N, H), (ldx, 1))
    ws = wbuf.as_strided((H, V), (ldw, 1))
    xs.copy_(x)
    ws.copy_(w)
    xbuf[(N - 1) * ldx + H:] = float("nan")
    wbuf[(H - 1) * ldw + V:] = float("nan")
    res = []
    for xi, wi in ((x, w), (xs, ws)):
        xi = xi.detach().requires_grad_(True)
        wi = wi.detach().requires_grad_(True)
        out = linear_cross_entropy(xi, y, wi, -1, 1e-4, 1.0, 256, True)
        out[0].backward()
        res.append((torch.stack(out).detach(), xi.grad.clone(), wi.grad.clone()))
    assert torch.isfinite(res[1][0]).all()
    for a, b in zip(res[0], res[1]):
        assert torch.equal(a, b)


def test_gpt2_vocabulary_matches_fp64_oracle_evaluated_on_gpu():
    """V = 50257 (not a multiple of 8), H = 768, N = 3000: oracle in fp64 on the GPU."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy
    from oracle import lce_forward_backward_fp64

    print("gpt2 vocabulary", flush=True)
    N, H, V = 3000, 768, 50257
    x, y, w = make_inputs(N, H, V, torch.bfloat16, seed=50257, ignore_frac=0.05, zipf=True, device="cuda")
    y[1] = V - 1
    xd = x.clone().requires_grad_(True)
    wd = w.clone().requires_grad_(True)
    out = linear_cross_entropy(xd, y, wd, -1, 0.0, 1.0, 1024, True)
    out[0].backward()
    ref = lce_forward_backward_fp64(x, y, w, -1, 0.0, 1.0, chunk=512)
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item())
    assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
    for name, got, want in (("dx", xd.grad, ref.dx), ("dw", wd.grad, ref.dw)):
        d = got.double() - want
        emax = (d.abs().max() / want.abs().max()).item()
        el2 = (d.norm() / want.norm()).item()
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (name, emax, el2)
    assert (xd.grad[y == -1] == 0).all()


def test_randomized_shapes_and_options_match_oracle():
    """Twenty seeded draws over token counts, hidden sizes, vocabularies (tile multiples, off-by-one,
    non-multiples of 8), dtypes, fp32 master weight, ignore fraction, z-regularisation, scale, N_chunk_size
    (forcing one or many slabs, split-K or not) and monitoring -- each against the fp64 oracle."""
    import random

    rng = random.Random(1234)
    for it in range(20):
        N = rng.choice([1, 7, 100, 255, 256, 257, 600, 1024, 1500, 3000])
        H = rng.choice([8, 24, 100, 128, 136, 256, 264, 520, 777, 1024])
        V = rng.choice([8, 9, 255, 256, 263, 1000, 1001, 4096, 5000, 10008, 12000])
        dt = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        wdt = rng.choice([None, torch.float32]) if dt != torch.float32 else None
        ign, zreg, scale = rng.choice([0.0, 0.1, 0.5]), rng.choice([0.0, 1e-4, 1e-2]), rng.choice([1.0, 0.5, 2.0])
        nc, mon = rng.choice([16, 64, 512, 4096]), rng.choice([False, True])
        print(f"random case {it}: N={N} H={H} V={V} {dt} w={wdt} ign={ign} zreg={zreg} scale={scale} chunk={nc} "
              f"mon={mon}", flush=True)
        x, y, w = make_inputs(N, H, V, dt, seed=100 + it, ignore_frac=ign, w_dtype=wdt)
        if (y != -1).sum() == 0:
            y[0] = 0
        out, dx, dw = _run(x, y, w, -1, zreg, scale, nc, mon, grad_output=1.3)
        ref = _oracle(x, y, w, -1, zreg, scale, grad_output=1.3)
        loss_tol, grad_tol = _tols(dt)
        assert abs(out[0].item() - ref.loss.item()) <= loss_tol * abs(ref.loss.item()), it
        if mon:
            assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item()) + 1e-5, it
            assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item()) + 1e-4, it
            assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item()), it
        for got, want in ((dx, ref.dx), (dw, ref.dw)):
            emax, el2 = rel_errors(got, want)
            assert emax <= grad_tol and el2 <= grad_tol, (it, emax, el2)
        assert (dx.cpu()[y == -1] == 0).all(), it


@pytest.mark.parametrize("mon", [False, True])
def test_many_tokens_go_through_the_forward_in_chunks(mon):
    """More tokens than one forward chunk holds (chunks of max(N_chunk_size, 16384) rows: here 16384 + 16384 +
    7232, the last one not a multiple of the tile size): per-token lse, the loss, the monitoring values and both
    gradients against the oracle, and lse of every kept token individually."""
    from linear_cross_entropy_loss_amd import _lib, linear_cross_entropy
    from oracle import lce_forward_backward_fp64

    N, H, V = 40000, 72, 1000
    print(f"chunked forward N={N} H={H} V={V} monitoring={mon}", flush=True)
    x, y, w = make_inputs(N, H, V, torch.bfloat16, seed=77, ignore_frac=0.2, device="cuda")
    y[N - 1] = V - 1
    out, dx, dw = _run(x, y, w, -1, 1e-4, 1.0, 512, mon)
    ref = lce_forward_backward_fp64(x, y, w, -1, 1e-4, 1.0, chunk=4096)
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item())
    assert abs(out[1].item() - ref.z_reg.item()) <= LOSS_RTOL * abs(ref.z_reg.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    for got, want in ((dx, ref.dx), (dw, ref.dw)):
        emax, el2 = rel_errors(got, want)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (emax, el2)
    assert (dx[y == -1] == 0).all()
    # lse of every kept token, through the C ABI (the autograd path keeps it to itself)
    import ctypes

    from linear_cross_entropy_loss_amd import ops

    lib = _lib.load()
    p = _lib.make_problem(N, H, V, H, V, H, V, x.dtype, w.dtype, x.dtype, w.dtype, -1, 1.0, 1e-4, 512, mon, 0,
                          ops.pack_rows.get())
    fwd_b, _ = _lib.workspace_bytes(p)
    assert fwd_b < (V // 128 + 1) * 16384 * 4 * (4 if mon else 1) + N * (H * 2 + 64)  # partials one chunk wide
    ws = torch.empty(fwd_b, dtype=torch.uint8, device="cuda")
    lse = torch.empty(N, device="cuda")
    out5 = torch.empty(5, device="cuda")
    nv = torch.empty(1, dtype=torch.int64, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.lce_forward(ctypes.byref(p), P(x), P(w), P(y), P(lse), P(out5), P(nv), P(ws), fwd_b,
                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    keep = y != -1
    assert nv.item() == int(keep.sum().item())
    assert torch.allclose(lse[keep].double(), ref.lse[keep], rtol=2e-4, atol=2e-4)
    # a token with an ignored label has lse == 0, whether its row was computed (rows not packed) or not
    assert (lse[~keep].view(torch.int32) == 0).all()
    assert torch.equal(out5[0], out[0])


@pytest.mark.parametrize("z_reg", [0.03125, 0.5])
def test_fp16_with_a_large_z_regularisation(z_reg):
    """fp16 stages dz times 2^10 to keep small probabilities normal; the factor 1 + 2 * z_reg * lse rides on top
    of that, so from z_reg > 1/32 on the staging is left unscaled instead.  Either side of the switch against
    the oracle, with logits large enough for lse to be of order 10."""
    print(f"fp16 z_reg={z_reg}", flush=True)
    x, y, w = make_inputs(512, 256, 4096, torch.float16, seed=91, ignore_frac=0.1, w_std=0.2)
    out, dx, dw = _run(x, y, w, -1, z_reg, 1.0, 512, False, grad_output=64.0)
    ref = _oracle(x, y, w, -1, z_reg, 1.0, grad_output=64.0)
    assert torch.isfinite(dx).all() and torch.isfinite(dw).all()
    assert ref.lse.abs().max().item() > 8
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item())
    for got, want in ((dx, ref.dx), (dw, ref.dw)):
        emax, el2 = rel_errors(got, want)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (emax, el2)


def test_fp16_z_regularisation_with_lse_near_a_thousand_stays_finite():
    """fp16 stages dz times 2^10 with the factor 1 + 2 * z_reg * lse on top: at z_reg = 0.03 and logits around 1e3
    that factor is about 60, the staged values reach 6e4 -- inside fp16's range (the kernel clamps the factor to
    63, which lse < 1033 does not reach here), so the gradients stay finite and match the fp64 oracle."""
    print("fp16 z_reg=0.03, lse near 1000", flush=True)
    x, y, w = make_inputs(512, 256, 4096, torch.float16, seed=93, ignore_frac=0.1)
    scale = 205.0
    out, dx, dw = _run(x, y, w, -1, 0.03, scale, 512, False, grad_output=1.0 / 64)
    ref = _oracle(x, y, w, -1, 0.03, scale, grad_output=1.0 / 64)
    assert 800 < ref.lse.abs().max().item() < 1030
    assert torch.isfinite(out[0]) and torch.isfinite(dx).all() and torch.isfinite(dw).all()
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item())
    for got, want in ((dx, ref.dx), (dw, ref.dw)):
        emax, el2 = rel_errors(got, want)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (emax, el2)


@pytest.mark.parametrize("dtype,w_std,scale", [(torch.bfloat16, 5.0, 1.0), (torch.float16, 1.0, 8.0),
                                               (torch.float32, 5.0, 1.0)])
def test_saturated_softmax_with_logits_in_the_hundreds(dtype, w_std, scale):
    """Logits of standard deviation 80 or more (max beyond 300): exp(logit) alone would overflow fp32, most
    probabilities underflow to zero and every row's softmax is close to one-hot.  The running-maximum form of
    lse must keep loss and gradients finite and equal to the fp64 oracle's, to the tolerances of the dtype."""
    print(f"saturated softmax {dtype}", flush=True)
    x, y, w = make_inputs(512, 256, 4096, dtype, seed=77, ignore_frac=0.1, w_std=w_std)
    out, dx, dw = _run(x, y, w, -1, 0.0, scale, 512, False)
    ref = _oracle(x, y, w, -1, 0.0, scale)
    assert ref.lse.abs().max().item() > 300
    assert torch.isfinite(out[0]) and torch.isfinite(dx).all() and torch.isfinite(dw).all()
    loss_rtol, grad_tol = _tols(dtype)
    assert abs(out[0].item() - ref.loss.item()) <= loss_rtol * abs(ref.loss.item())
    for got, want in ((dx, ref.dx), (dw, ref.dw)):
        emax, el2 = rel_errors(got, want)
        assert emax <= grad_tol and el2 <= grad_tol, (emax, el2)


@pytest.mark.pack_auto  # (run once: every draw picks its own packing mode)
def test_two_hundred_draws_over_layouts_packing_and_sizes_around_a_round_of_tiles():
    """Seeded draws over everything a call can vary at once: both weight layouts, the three packing modes, 16-bit and
    fp32 tensors, fp32 master weights, ignore fractions up to 95 %, and sizes up to 12000 tokens x 2056 hidden units,
    where the dx / dW tile counts pass through one round of 256 workgroups (whole tiles only, split tails only, both).
    Inputs and the fp64 oracle live on the GPU.  A gradient is allowed, on top of its tolerance, what rounding the
    exact result to the output type costs (the fp16 dx of a mean over 12000 tokens lies in fp16's subnormal range)."""
    import random

    from linear_cross_entropy_loss_amd import linear_cross_entropy, ops
    from oracle import lce_forward_backward_fp64

    rng = random.Random(20)
    for it in range(200):
        N = rng.choice([1, 7, 100, 255, 256, 257, 600, 1024, 1500, 3000, 4096, 5000, 8192, 8200, 12000])
        H = rng.choice([8, 24, 104, 128, 136, 256, 264, 520, 776, 1024, 2048, 2056])
        V = rng.choice([8, 9, 255, 256, 263, 1000, 1001, 2048, 4096, 5000, 8192, 10008, 12000, 16384, 20000, 32768])
        dt = rng.choice([torch.bfloat16, torch.float16, torch.bfloat16, torch.float16, torch.float32])
        wdt = None if dt == torch.float32 else rng.choice([None, None, torch.float32])
        vh = dt != torch.float32 and rng.random() < 0.5
        ign, zreg, scale = rng.choice([0.0, 0.1, 0.5, 0.95]), rng.choice([0.0, 1e-4, 1e-2]), rng.choice([1.0, 0.5, 2.0])
        nc, mon, pack = rng.choice([16, 64, 512, 4096, 4096]), rng.choice([False, True]), rng.choice([0, 1, 2])
        if N * V > 2.2e8:  # keeps the fp64 oracle's N x V matrices below 2 GiB
            V = max(8, int(2.2e8 // N) // 8 * 8)
        print(f"draw {it}: N={N} H={H} V={V} {dt} w={wdt} vh={vh} ign={ign} zreg={zreg} scale={scale} chunk={nc} "
              f"mon={mon} pack={pack}", flush=True)
        x, y, w = make_inputs(N, H, V, dt, seed=7000 + it, ignore_frac=ign, w_dtype=wdt, device="cuda")
        if (y != -1).sum() == 0:
            y[0] = 0
        wt = (w.t().contiguous() if vh else w.clone()).requires_grad_(True)
        xd = x.clone().requires_grad_(True)
        token = ops.pack_rows.set(pack)
        try:
            out = linear_cross_entropy(xd, y, wt.t() if vh else wt, -1, zreg, scale, nc, mon)
            (out[0] * 0.7).backward()
            torch.cuda.synchronize()
        finally:
            ops.pack_rows.reset(token)
        ref = lce_forward_backward_fp64(x, y, w, -1, zreg, scale, grad_output=0.7, chunk=512)
        loss_tol, grad_tol = _tols(dt)
        # (relative to max(loss, 1): with one or a few tokens the loss can be a fraction of the logits it is made of,
        # which carry the rounding of the 16-bit operands)
        assert abs(out[0].item() - ref.loss.item()) <= loss_tol * max(abs(ref.loss.item()), 1.0), it
        for name, got, want in (("dx", xd.grad, ref.dx), ("dw", wt.grad.t() if vh else wt.grad, ref.dw)):
            assert torch.isfinite(got).all(), (it, name)
            emax, el2 = rel_errors(got, want)
            rmax, rl2 = rel_errors(want.to(got.dtype), want)
            assert emax <= grad_tol + rmax and el2 <= grad_tol + rl2, (it, name, emax, el2)
        assert (xd.grad[y == -1] == 0).all(), it
        del x, y, w, wt, xd, out, ref

"""A weight stored with the vocabulary as its row index, (V, H) row-major -- a tied embedding matrix or an
``nn.Linear(H, V)`` weight -- handed over as its transposed view ``weight.T`` of shape (H, V).

The reference reads At through its strides (linear_cross_entropy/ops.py:733-734) and returns a gradient with
At's strides (``zeros_like(At)``, ops.py:693), so such a weight costs it no copy.  Here the kernels have a
second layout (``lce_problem.w_layout = LCE_W_VH``); every case is checked against the fp64 oracle and against
the same call on a row-major (H, V) copy of the weight.
"""
import pytest
import torch

from helpers import make_inputs, rel_errors

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-3
GRAD_TOL = 2e-2

CASES = [
    # N, H, V, dtype, w_dtype, ignore_frac, z_reg, scale, n_chunk, monitoring
    (512, 256, 4096, torch.bfloat16, None, 0.1, 0.0, 1.0, 4096, False),
    (1024, 512, 8192, torch.float16, None, 0.05, 1e-4, 0.5, 512, True),       # several vocabulary slabs
    (1000, 520, 5000, torch.bfloat16, None, 0.1, 1e-3, 1.0, 64, True),        # nothing a multiple of a tile; K mask
    (300, 104, 1001, torch.float16, None, 0.0, 0.0, 2.0, 4096, False),
    (33, 8, 9, torch.bfloat16, None, 0.2, 0.0, 1.0, 16, True),
    (768, 384, 6000, torch.float16, torch.float32, 0.1, 1e-4, 1.0, 256, False),  # fp32 master weight, fp32 dW
    (2048, 1024, 32768, torch.bfloat16, torch.float32, 0.05, 0.0, 1.0, 1024, True),
    (4096, 2048, 16384, torch.bfloat16, None, 0.05, 0.0, 1.0, 4096, False),   # split tails in dx and dW
]


def _run(x, y, At, z_reg, scale, n_chunk, mon, g=1.3):
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    out = linear_cross_entropy(x, y, At, -1, z_reg, scale, n_chunk, mon)
    (out[0] * g).backward()
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("N,H,V,dtype,w_dtype,ign,z_reg,scale,n_chunk,mon", CASES)
def test_vocabulary_major_weight_matches_oracle_and_the_row_major_call(N, H, V, dtype, w_dtype, ign, z_reg, scale,
                                                                         n_chunk, mon):
    from linear_cross_entropy_loss_amd import _lib, ops
    from oracle import lce_forward_backward_fp64

    print(f"(V, H) weight: N={N} H={H} V={V} {dtype} w={w_dtype} ign={ign} zreg={z_reg} scale={scale} chunk={n_chunk}",
          flush=True)
    x, y, w = make_inputs(N, H, V, dtype, seed=N + 3 * H + V, ignore_frac=ign, w_dtype=w_dtype, device="cuda")
    y[0] = V - 1
    wt = w.t().contiguous().requires_grad_(True)  # the parameter as a model holds it: (V, H)
    assert ops._weight_layout(wt.t(), dtype) == _lib.W_VH
    xd = x.clone().requires_grad_(True)
    out = _run(xd, y, wt.t(), z_reg, scale, n_chunk, mon)
    assert wt.grad.shape == (V, H) and wt.grad.is_contiguous() and wt.grad.dtype == wt.dtype

    ref = lce_forward_backward_fp64(x, y, w, -1, z_reg, scale, grad_output=1.3, chunk=512)
    assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item())
    if mon:
        assert abs(out[2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
        assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item()) + 1e-4
        assert abs(out[4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())
    for name, got, want in (("dx", xd.grad, ref.dx), ("dw", wt.grad.t(), ref.dw)):
        d = got.double() - want
        emax, el2 = (d.abs().max() / want.abs().max()).item(), (d.norm() / want.norm()).item()
        print(f"  {name}: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (name, emax, el2)
    assert (xd.grad[y == -1] == 0).all()

    # The row-major call does the same arithmetic in the same order on another memory layout: logits, and
    # with them the loss and dx, agree bit for bit; dW exchanges the two operands of its contraction.
    x2 = x.clone().requires_grad_(True)
    w2 = w.clone().requires_grad_(True)
    out2 = _run(x2, y, w2, z_reg, scale, n_chunk, mon)
    for a, b in zip(out, out2):
        assert torch.equal(a, b)
    assert torch.equal(xd.grad, x2.grad)
    emax, el2 = rel_errors(wt.grad.t(), w2.grad)
    assert emax <= 1e-6 and el2 <= 1e-6, (emax, el2)


def test_randomized_shapes_with_a_vocabulary_major_weight():
    """Twenty seeded draws over token counts, hidden sizes (multiples of 8), vocabularies, dtypes, fp32 master
    weight, ignore fraction, z-regularisation, scale, N_chunk_size and monitoring, each against the fp64 oracle."""
    import random

    from linear_cross_entropy_loss_amd import _lib, ops
    from oracle import lce_forward_backward_fp64

    rng = random.Random(4321)
    for it in range(20):
        N = rng.choice([1, 7, 100, 255, 256, 257, 600, 1024, 1500, 3000])
        H = rng.choice([8, 24, 104, 128, 136, 256, 264, 520, 776, 1024])
        V = rng.choice([8, 9, 255, 256, 263, 1000, 1001, 4096, 5000, 10008, 12000])
        dt = rng.choice([torch.bfloat16, torch.float16])
        wdt = rng.choice([None, torch.float32])
        ign, zreg, scale = rng.choice([0.0, 0.1, 0.5]), rng.choice([0.0, 1e-4, 1e-2]), rng.choice([1.0, 0.5, 2.0])
        n_chunk, mon = rng.choice([16, 64, 512, 4096]), rng.choice([False, True])
        print(f"draw {it}: N={N} H={H} V={V} {dt} w={wdt} ign={ign} zreg={zreg} scale={scale} chunk={n_chunk} mon={mon}",
              flush=True)
        x, y, w = make_inputs(N, H, V, dt, seed=1000 + it, ignore_frac=ign, w_dtype=wdt, device="cuda")
        if (y != -1).sum() == 0:
            y[0] = 0
        wt = w.t().contiguous().requires_grad_(True)
        assert ops._weight_layout(wt.t(), dt) == _lib.W_VH
        xd = x.clone().requires_grad_(True)
        out = _run(xd, y, wt.t(), zreg, scale, n_chunk, mon, g=0.7)
        ref = lce_forward_backward_fp64(x, y, w, -1, zreg, scale, grad_output=0.7, chunk=512)
        assert abs(out[0].item() - ref.loss.item()) <= LOSS_RTOL * abs(ref.loss.item()), (it, out[0].item(), ref.loss.item())
        for name, got, want in (("dx", xd.grad, ref.dx), ("dw", wt.grad.t(), ref.dw)):
            emax, el2 = rel_errors(got, want)
            assert emax <= GRAD_TOL and el2 <= GRAD_TOL, (it, name, emax, el2)
        assert (xd.grad[y == -1] == 0).all()


def test_weights_the_kernels_cannot_read_in_place_are_copied():
    """fp32 tensors (computed as bf16 pairs, which have no (V, H) form) and a hidden size that is not a multiple
    of 8: the transposed view is copied into a row-major (H, V) matrix and everything else stays the same."""
    from oracle import lce_forward_backward_fp64

    for dtype, H, loss_tol, grad_tol in ((torch.float32, 256, 1e-5, 1e-3), (torch.bfloat16, 100, LOSS_RTOL, GRAD_TOL)):
        print(f"(V, H) weight, copied: {dtype} H={H}", flush=True)
        N, V = 300, 1000
        x, y, w = make_inputs(N, H, V, dtype, seed=17, ignore_frac=0.1, device="cuda")
        wt = w.t().contiguous().requires_grad_(True)
        xd = x.clone().requires_grad_(True)
        out = _run(xd, y, wt.t(), 1e-4, 1.0, 512, False, g=1.0)
        ref = lce_forward_backward_fp64(x, y, w, -1, 1e-4, 1.0, chunk=512)
        assert abs(out[0].item() - ref.loss.item()) <= loss_tol * abs(ref.loss.item())
        assert wt.grad.shape == (V, H)
        for got, want in ((xd.grad, ref.dx), (wt.grad.t(), ref.dw)):
            emax, el2 = rel_errors(got, want)
            assert emax <= grad_tol and el2 <= grad_tol, (emax, el2)


def test_strided_vocabulary_major_weight_with_garbage_in_the_padding():
    """(V, H) rows with a stride longer than H whose padding holds large finite garbage: same bits as dense."""
    print("(V, H) weight, padded rows", flush=True)
    N, H, V = 700, 200, 3000
    x, y, w = make_inputs(N, H, V, torch.bfloat16, seed=11, ignore_frac=0.1, device="cuda")
    dense = w.t().contiguous()
    padded = torch.full((V, H + 24), -1e30, dtype=w.dtype, device="cuda")
    padded[:, :H] = dense
    res = []
    for wt in (dense, padded[:, :H]):
        wt = wt.detach().requires_grad_(True)
        xd = x.clone().requires_grad_(True)
        out = _run(xd, y, wt.t(), 1e-4, 1.0, 512, True)
        res.append((out, xd.grad, wt.grad))
    for a, b in zip(res[0][0], res[1][0]):
        assert torch.equal(a, b)
    assert torch.equal(res[0][1], res[1][1]) and torch.equal(res[0][2], res[1][2])


def test_vocabulary_major_weight_is_not_copied():
    """A (V, H) matrix used as the output weight: forward + backward allocate its gradient, the dz stage and
    small change -- not the row-major copy of the transposed view that any other striding costs (and that would
    stay alive from forward to backward)."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("(V, H) weight: no copy", flush=True)
    N, H, V = 1024, 1024, 65536
    g = torch.Generator(device="cuda").manual_seed(3)
    wt = (torch.randn(V, H, device="cuda", generator=g) / 32).to(torch.bfloat16).requires_grad_(True)
    x = torch.randn(N, H, device="cuda", generator=g).to(torch.bfloat16).requires_grad_(True)
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    w_bytes = wt.numel() * 2

    def peak(At):
        x.grad = wt.grad = None
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        loss = linear_cross_entropy(x, y, At, -100, 0.0, 1.0, 65536, False)[0]
        loss.backward()
        torch.cuda.synchronize()
        assert torch.isfinite(loss) and wt.grad.shape == (V, H)
        return torch.cuda.max_memory_allocated() - base

    in_place = peak(wt.T)
    # the gradient (one w_bytes), the dz stage (N x V x 2 bytes), 64 MiB of split-K partial sums and small change
    assert in_place < w_bytes + N * V * 2 + (80 << 20), (in_place, w_bytes)
    assert wt.grad.is_contiguous()
    # for contrast, a striding the kernels do not read in place (every other column of a wider matrix) is copied
    wide = torch.zeros(V, 2 * H, device="cuda", dtype=torch.bfloat16)
    wide[:, ::2] = wt.detach()
    wide.requires_grad_(True)
    x.grad = None
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    linear_cross_entropy(x, y, wide[:, ::2].T, -100, 0.0, 1.0, 65536, False)[0].backward()
    torch.cuda.synchronize()
    copied = torch.cuda.max_memory_allocated() - base
    assert copied >= in_place + w_bytes, (copied, in_place)


def test_compiled_model_with_a_tied_output_weight():
    """torch.compile (aot_eager) of embedding -> linear -> loss with the embedding as output weight: matches eager."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("compiled tied model", flush=True)
    torch._dynamo.reset()
    N, H, V = 512, 256, 4096

    class Tied(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = torch.nn.Embedding(V, H)
            self.mix = torch.nn.Linear(H, H)

        def forward(self, ids, y):
            return linear_cross_entropy(self.mix(self.emb(ids)), y, self.emb.weight.T, -100, 1e-4)[0]

    torch.manual_seed(0)
    model = Tied().to(device="cuda", dtype=torch.bfloat16)
    g = torch.Generator(device="cuda").manual_seed(5)
    ids = torch.randint(0, V, (N,), device="cuda", generator=g)
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    model(ids, y).backward()
    eager = [p.grad.clone() for p in model.parameters()]
    for p in model.parameters():
        p.grad = None
    compiled = torch.compile(model, backend="aot_eager", fullgraph=True)
    compiled(ids, y).backward()
    for p, e in zip(model.parameters(), eager):
        emax, el2 = rel_errors(p.grad, e)
        assert emax <= 1e-2 and el2 <= 1e-2, (emax, el2)
    torch._dynamo.reset()


def test_registered_operators_pass_opcheck_with_a_vocabulary_major_weight():
    import linear_cross_entropy_loss_amd  # noqa: F401  (registers the operators)

    print("opcheck, (V, H) weight", flush=True)
    x, y, w = make_inputs(256, 64, 512, torch.bfloat16, seed=9, ignore_frac=0.1, device="cuda")
    wt = w.t().contiguous()
    torch.library.opcheck(torch.ops.lce_amd.forward.default, (x, y, wt.t(), -1, 0.0, 1.0, 4096, False, 0))
    out5, lse, n_valid = torch.ops.lce_amd.forward(x, y, wt.t(), -1, 0.0, 1.0, 4096, False, 0)
    g = torch.ones(1, device="cuda")
    torch.library.opcheck(torch.ops.lce_amd.backward.default,
                          (x, y, wt.t(), lse, n_valid, g, -1, 0.0, 1.0, 4096, True, True, 0))

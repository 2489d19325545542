"""GPU tests of masking, determinism, API behaviour and full-size properties of the HIP path."""
import ctypes
import math

import pytest
import torch

from helpers import make_inputs, rel_errors

pytestmark = pytest.mark.gpu


def _fb(x, y, w, ignore_index=-1, z_reg=0.0, scale=1.0, n_chunk=512, mon=False, g=1.0):
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    xd = x.detach().clone().requires_grad_(True)
    wd = w.detach().clone().requires_grad_(True)
    out = linear_cross_entropy(xd, y, wd, ignore_index, z_reg, scale, n_chunk, mon)
    (out[0] * g).backward()
    torch.cuda.synchronize()
    return out, xd.grad, wd.grad


def test_masking_is_bit_exact_under_garbage_in_ignored_rows():
    print("masking bit-exact", flush=True)
    x, y, w = make_inputs(1024, 256, 8192, torch.bfloat16, seed=21, ignore_frac=0.3, device="cuda")
    out_a, dx_a, dw_a = _fb(x, y, w, z_reg=1e-3)
    xg = x.clone()
    xg[y == -1] = 3.0e4  # finite garbage
    out_b, dx_b, dw_b = _fb(xg, y, w, z_reg=1e-3)
    assert torch.equal(out_a[0], out_b[0]) and torch.equal(out_a[1], out_b[1])
    assert torch.equal(dx_a, dx_b)
    assert torch.equal(dw_a, dw_b)
    assert (dx_a[y == -1].view(torch.int16) == 0).all()  # +0.0 bit pattern


def test_ignored_rows_are_never_read_so_nan_in_them_is_harmless():
    """Tokens with an ignored label are dropped before the tile kernels, so even NaN / Inf in their rows of
    x leaves loss, dx and dW bit-identical (the reference's x^T dz would give NaN * 0 = NaN, ops.py:424).
    With monitoring on, logit_max and logit_norm are taken over all rows (ops.py:15, 17) and do see them."""
    from linear_cross_entropy_loss_amd import _lib, ops

    print("NaN in ignored rows", flush=True)
    ops.pack_rows.set(_lib.PACK_ALWAYS)  # (the fixture restores it)
    x, y, w = make_inputs(1500, 264, 5000, torch.bfloat16, seed=31, ignore_frac=0.4, device="cuda")
    out_a, dx_a, dw_a = _fb(x, y, w, z_reg=1e-3, n_chunk=64)
    xg = x.clone()
    xg[y == -1] = float("nan")
    xg[(y == -1).nonzero()[::2, 0]] = float("inf")
    out_b, dx_b, dw_b = _fb(xg, y, w, z_reg=1e-3, n_chunk=64)
    assert torch.isfinite(out_b[0]) and torch.equal(out_a[0], out_b[0]) and torch.equal(out_a[1], out_b[1])
    assert torch.equal(dx_a, dx_b) and torch.equal(dw_a, dw_b)
    assert (dx_b[y == -1].view(torch.int16) == 0).all()
    out_m, dx_m, dw_m = _fb(xg, y, w, z_reg=1e-3, n_chunk=64, mon=True)
    assert torch.equal(out_m[0], out_a[0]) and torch.equal(dx_m, dx_a) and torch.equal(dw_m, dw_a)
    assert not torch.isfinite(out_m[4])  # the norm over all rows meets the NaN rows


@pytest.mark.parametrize("keep_every", [1, 2, 7, 300, 5000])
def test_results_do_not_depend_on_where_the_ignored_tokens_sit(keep_every):
    """Dropping ignored tokens packs the others to the front in their order: the kept tokens of a sparse
    batch must give the loss, dW and dx rows of the dense batch made of those tokens alone."""
    from oracle import lce_forward_backward_fp64

    from linear_cross_entropy_loss_amd import _lib, ops

    print(f"packed rows keep_every={keep_every}", flush=True)
    ops.pack_rows.set(_lib.PACK_ALWAYS)  # (the fixture restores it)
    N, H, V = 3000, 136, 3003
    x, y, w = make_inputs(N, H, V, torch.float16, seed=40 + keep_every, ignore_frac=0.0, device="cuda")
    keep = torch.zeros(N, dtype=torch.bool, device="cuda")
    keep[::keep_every] = True
    y = torch.where(keep, y, torch.full_like(y, -1))
    # (a scratch bound wide enough for one vocabulary slab either way: the split depends on N, and with it
    # the order in which dx is summed)
    out, dx, dw = _fb(x, y, w, z_reg=1e-4, scale=0.5, n_chunk=4096, g=1.7)
    dense, dxd, dwd = _fb(x[keep], y[keep], w, z_reg=1e-4, scale=0.5, n_chunk=4096, g=1.7)
    # same rows in the same order through the same kernels: bit-identical
    assert torch.equal(out[0], dense[0]) and torch.equal(dw, dwd) and torch.equal(dx[keep], dxd)
    assert (dx[~keep].view(torch.int16) == 0).all()
    ref = lce_forward_backward_fp64(x.cpu().double(), y.cpu(), w.cpu().double(), -1, 1e-4, 0.5, 1.7)
    assert abs(out[0].item() - ref.loss.item()) <= 1e-3 * abs(ref.loss.item())
    assert max(rel_errors(dx, ref.dx)) <= 2e-2 and max(rel_errors(dw, ref.dw)) <= 2e-2


def test_dx_of_2_gib_is_staged_packed_and_moved(pack_mode):
    """Packed dx rows normally go straight to their tokens through 32-bit store offsets; a dx of 2 GiB or
    more is staged packed and moved by a copy kernel.  Same rows through the same kernels either way."""
    from linear_cross_entropy_loss_amd import _lib, ops

    if pack_mode != "pack":
        pytest.skip("one run is enough")
    print("staged dx", flush=True)
    N, H, V = 131072, 8192, 512
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(N, H, device="cuda", dtype=torch.bfloat16, generator=g)
    w = (torch.randn(H, V, device="cuda", generator=g) / math.sqrt(H)).to(torch.bfloat16)
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    y[torch.rand(N, device="cuda", generator=g) < 0.3] = -1
    res = {}
    for mode in (_lib.PACK_ALWAYS, _lib.PACK_NEVER):
        ops.pack_rows.set(mode)
        out, dx, dw = _fb(x, y, w, n_chunk=65536)
        res[mode] = (out[0].item(), dx, dw)
        del out
    a, b = res[_lib.PACK_ALWAYS], res[_lib.PACK_NEVER]
    assert abs(a[0] - b[0]) <= 1e-6 * abs(b[0])
    assert torch.equal(a[1], b[1])          # dx rows do not depend on which other rows share their tile
    assert (a[1][y == -1] == 0).all()
    e_max, e_l2 = rel_errors(a[2], b[2])         # dW: another summation order over the tokens, then bf16 rounding
    assert e_max <= 1e-2 and e_l2 <= 1e-3


def test_valid_count_is_exact_and_nonnegative_ignore_index_is_honoured():
    from linear_cross_entropy_loss_amd import _lib

    print("n_valid exact", flush=True)
    N, H, V = 2048, 256, 4096
    x, y, w = make_inputs(N, H, V, torch.float16, seed=22, ignore_frac=0.0, device="cuda")
    y[::3] = 7  # ignore_index = 7 is a legal column: those rows are ignored, never matched
    lib = _lib.load()
    from linear_cross_entropy_loss_amd import ops

    p = _lib.make_problem(N, H, V, H, V, H, V, x.dtype, w.dtype, x.dtype, w.dtype, 7, 1.0, 0.0, 512, False, 0,
                          ops.pack_rows.get())
    fwd_b, _ = _lib.workspace_bytes(p)
    ws = torch.empty(fwd_b, dtype=torch.uint8, device="cuda")
    lse = torch.empty(N, device="cuda")
    out5 = torch.empty(5, device="cuda")
    nv = torch.zeros(1, dtype=torch.int64, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.lce_forward(ctypes.byref(p), P(x), P(w), P(y), P(lse), P(out5), P(nv), P(ws), fwd_b,
                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert nv.item() == int((y != 7).sum().item())
    from oracle import lce_forward_fp64

    ref = lce_forward_fp64(x.cpu().double(), y.cpu(), w.cpu().double(), 7, 0.0, 1.0)
    assert abs(out5[0].item() - ref.loss.item()) <= 1e-3 * abs(ref.loss.item())
    keep = (y != 7).cpu()
    assert torch.allclose(lse.cpu().double()[keep], ref.lse[keep], rtol=2e-4, atol=2e-4)
    # a row with the ignored label has lse == 0 in either packing mode: packed away it is not computed at all, and
    # where it is computed (rows not packed) the value is not handed out
    assert bool((lse.cpu()[~keep].view(torch.int32) == 0).all())
    _, dx, _ = _fb(x, y, w, ignore_index=7)
    assert (dx[y == 7] == 0).all()


def test_all_labels_ignored_gives_nan_loss():
    print("all ignored", flush=True)
    x, y, w = make_inputs(512, 256, 4096, torch.bfloat16, seed=23, device="cuda")
    y[:] = -1
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    out = linear_cross_entropy(x, y, w, -1)
    assert math.isnan(out[0].item())
    # ... and both gradients are exact zeros (every dz is zero; F.cross_entropy's backward gives zeros as well),
    # whether or not the ignored rows were packed away
    xd, wd = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    linear_cross_entropy(xd, y, wd, -1, 1e-4)[0].backward()
    assert (xd.grad == 0).all() and (wd.grad == 0).all()


def test_runs_are_deterministic_and_backward_can_repeat():
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("determinism", flush=True)
    x, y, w = make_inputs(1024, 512, 8192, torch.bfloat16, seed=24, ignore_frac=0.1, device="cuda")
    a = _fb(x, y, w, z_reg=1e-4, scale=0.5, mon=True)
    b = _fb(x, y, w, z_reg=1e-4, scale=0.5, mon=True)
    for t, u in zip(a[0], b[0]):
        assert torch.equal(t, u)
    assert torch.equal(a[1], b[1]) and torch.equal(a[2], b[2])
    # backward twice on one graph: each call recomputes, nothing is scaled in place
    xd = x.clone().requires_grad_(True)
    wd = w.clone().requires_grad_(True)
    loss = linear_cross_entropy(xd, y, wd, -1, 1e-4, 0.5, 512, False)[0]
    g1 = torch.autograd.grad(loss, (xd, wd), retain_graph=True)
    g2 = torch.autograd.grad(loss, (xd, wd))
    assert torch.equal(g1[0], g2[0]) and torch.equal(g1[1], g2[1])
    assert torch.equal(g1[0], a[1])


def test_two_threads_on_two_streams_do_not_disturb_each_other():
    """The library keeps no state between calls and none that two calls share (lce.h): two host threads, each
    with a stream, inputs and scratch of its own, run forward + backward at the same time, several times over;
    every result is bit-identical to the same call made alone."""
    import contextvars
    import threading

    print("two threads, two streams", flush=True)
    cases = [make_inputs(1024, 512, 8192, torch.bfloat16, seed=61, ignore_frac=0.1, device="cuda") + (1e-4, 0.5),
             make_inputs(768, 256, 12288, torch.float16, seed=62, ignore_frac=0.3, device="cuda") + (0.0, 1.0)]
    alone = [_fb(x, y, w, z_reg=z, scale=s, mon=True) for x, y, w, z, s in cases]
    torch.cuda.synchronize()
    failures = []

    def worker(k):
        try:
            x, y, w, z, s = cases[k]
            stream = torch.cuda.Stream()  # (default priority)
            for _ in range(5):
                with torch.cuda.stream(stream):
                    out, dx, dw = _fb(x, y, w, z_reg=z, scale=s, mon=True)
                stream.synchronize()
                for t, u in zip(out, alone[k][0]):
                    if not torch.equal(t, u):
                        failures.append((k, "output"))
                if not (torch.equal(dx, alone[k][1]) and torch.equal(dw, alone[k][2])):
                    failures.append((k, "gradient"))
        except Exception as exc:  # surfaced below: an exception in a thread would otherwise pass silently
            failures.append((k, repr(exc)))

    # (each thread runs in a copy of this context, so that it packs ignored tokens, or not, as the calls above did)
    threads = [threading.Thread(target=contextvars.copy_context().run, args=(worker, k)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads)
    assert not failures, failures


def test_upstream_gradient_scales_linearly():
    print("grad_output linearity", flush=True)
    # bf16 on purpose: gradients of order 1/N are subnormal in fp16, where scaling by 4 is not exact
    x, y, w = make_inputs(512, 256, 4096, torch.bfloat16, seed=25, ignore_frac=0.1, device="cuda")
    _, dx1, dw1 = _fb(x, y, w, g=1.0)
    _, dx2, dw2 = _fb(x, y, w, g=4.0)  # power of two: exact scaling
    assert torch.equal(dx2, dx1 * 4) and torch.equal(dw2, dw1 * 4)


def test_n_chunk_size_only_changes_scratch_not_results():
    print("chunk invariance", flush=True)
    x, y, w = make_inputs(2048, 256, 16384, torch.bfloat16, seed=26, ignore_frac=0.1, device="cuda")
    ref = _fb(x, y, w, n_chunk=4096)
    for nc in (512, 1024):
        got = _fb(x, y, w, n_chunk=nc)
        assert torch.equal(got[0][0], ref[0][0])
        # dx is summed over vocabulary slabs in fp32, so a different slab count may move the last bit
        assert rel_errors(got[1], ref[1])[0] < 1e-2
        # dW: a tile's sum over the tokens is cut into segments when its slab has few tiles, and a tight bound
        # can switch that (and the packing of ignored tokens) off: the order of an fp32 sum, one bf16 rounding
        emax, el2 = rel_errors(got[2], ref[2])
        assert emax < 1e-2 and el2 < 2e-3


def test_module_api_3d_input_monitoring_and_no_grad():
    from linear_cross_entropy_loss_amd import LinearCrossEntropyLoss
    from oracle import lce_forward_fp64

    print("module api", flush=True)
    torch.manual_seed(3)
    m = LinearCrossEntropyLoss(256, 4096, device="cuda", dtype=torch.float16, ignore_index=-1, logit_scale=0.5,
                               z_regularization=1e-4, N_chunk_size=512)
    x = torch.randn(4, 128, 256, device="cuda", dtype=torch.float16, requires_grad=True)
    y = torch.randint(0, 4096, (4, 128), device="cuda")
    y[0, :10] = -1
    loss = m(x, y)
    assert m.latest_metrics == {}
    assert loss.dtype == torch.float32 and loss.dim() == 0
    loss.backward()
    assert x.grad.shape == x.shape and m.weight.grad.shape == m.weight.shape
    assert x.grad.dtype == torch.float16 and m.weight.grad.dtype == torch.float16
    m.monitoring = True
    with torch.no_grad():
        loss2 = m(x, y)
    assert torch.equal(loss2, loss.detach())
    assert set(m.latest_metrics) == {"logit_norm", "logit_max", "logit_entropy", "z_value"}
    ref = lce_forward_fp64(x.detach().cpu().double(), y.cpu(), m.weight.detach().cpu().double(), -1, 1e-4, 0.5)
    assert abs(m.latest_metrics["logit_max"].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
    assert abs(m.latest_metrics["logit_entropy"].item() - ref.logit_entropy.item()) <= 2e-3 * ref.logit_entropy.item()
    assert abs(m.latest_metrics["logit_norm"].item() - ref.logit_norm.item()) <= 2e-3 * ref.logit_norm.item()
    assert abs(m.latest_metrics["z_value"].item() - ref.z_reg.item()) <= 1e-3 * ref.z_reg.item()
    # only dx wanted: weight frozen
    m.weight.requires_grad_(False)
    x.grad = None
    m(x, y).backward()
    assert x.grad is not None


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_gradient_of_one_input_alone_equals_that_of_the_full_call(dtype):
    """dx without dW (frozen weight) and dW without dx (frozen activations) skip the other contraction and,
    with packed rows, the zeroing of dropped dx rows; what they return is bit-identical to the full call."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("partial gradients", flush=True)
    x, y, w = make_inputs(1300, 264, 5000, dtype, seed=77, ignore_frac=0.35, device="cuda")
    _, dx_full, dw_full = _fb(x, y, w, z_reg=1e-4, scale=0.5, n_chunk=64)
    xo = x.clone().requires_grad_(True)
    linear_cross_entropy(xo, y, w, -1, 1e-4, 0.5, 64)[0].backward()
    assert torch.equal(xo.grad, dx_full) and (xo.grad[y == -1] == 0).all()
    wo = w.clone().requires_grad_(True)
    linear_cross_entropy(x, y, wo, -1, 1e-4, 0.5, 64)[0].backward()
    assert torch.equal(wo.grad, dw_full)


def test_shape_errors_raise_value_error():
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("shape errors", flush=True)
    x = torch.randn(500, 256, device="cuda", dtype=torch.bfloat16)
    w = torch.randn(256, 4096, device="cuda", dtype=torch.bfloat16)
    y = torch.randint(0, 4096, (500,), device="cuda")
    # the reference's error for an unsupported shape (ops.py:43-44); here only degenerate sizes are unsupported
    with pytest.raises(ValueError, match="Provided shape outside the range of valid configs"):
        linear_cross_entropy(x[:0], y[:0], w)
    with pytest.raises(ValueError):
        linear_cross_entropy(torch.randn(512, 256, device="cuda", dtype=torch.bfloat16), y[:12], w)
    with pytest.raises(ValueError):
        linear_cross_entropy(x, y, w[:128])            # in_features mismatch
    with pytest.raises(ValueError):
        linear_cross_entropy(x, y.to(torch.int32), w)  # labels must be int64


def test_out_of_range_labels_poison_the_loss():
    """A label outside [0, V) that is not ignore_index has no column to match.  The reference lets it through
    silently (it then contributes lse alone); F.cross_entropy raises a device assert.  Here the loss is NaN."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("out-of-range labels", flush=True)
    x, y, w = make_inputs(512, 256, 4096, torch.bfloat16, seed=6, ignore_frac=0.1, device="cuda")
    assert torch.isfinite(linear_cross_entropy(x, y, w, -1)[0])
    for bad in (4096, 10**12, -7):
        yb = y.clone()
        yb[3] = bad
        assert torch.isnan(linear_cross_entropy(x, yb, w, -1)[0]), bad
    yb = torch.where(y == -1, torch.full_like(y, -7), y)
    assert torch.isfinite(linear_cross_entropy(x, yb, w, -7)[0])   # ... unless it is the ignore_index
    assert torch.isnan(linear_cross_entropy(x, y, w, -7)[0])       # the -1 labels are now out of range


def test_autocast_keeps_fp32_master_weight_and_returns_fp32_dw():
    from linear_cross_entropy_loss_amd import LinearCrossEntropyLoss
    from oracle import lce_forward_backward_fp64

    print("autocast / fp32 master weight", flush=True)
    torch.manual_seed(4)
    m = LinearCrossEntropyLoss(256, 4096, device="cuda", ignore_index=-1, N_chunk_size=512)  # fp32 parameter
    x = torch.randn(512, 256, device="cuda", requires_grad=True)
    y = torch.randint(0, 4096, (512,), device="cuda")
    with torch.autocast("cuda", dtype=torch.float16):
        loss = m(x, y)
    loss.backward()
    assert m.weight.grad.dtype == torch.float32 and x.grad.dtype == torch.float32
    ref = lce_forward_backward_fp64(x.detach().cpu().double(), y.cpu(), m.weight.detach().cpu().double(), -1)
    assert abs(loss.item() - ref.loss.item()) <= 1e-3 * ref.loss.item()
    assert rel_errors(m.weight.grad, ref.dw)[1] <= 2e-2 and rel_errors(x.grad, ref.dx)[1] <= 2e-2


# ---------------------------------------------------------------------------------------------------------
# Full benchmark shape (N=16384, H=2048, V=131072, bf16): size-independent properties plus the fp64 oracle
# evaluated on the GPU in row chunks.
# ---------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def big():
    N, H, V = 16384, 2048, 131072
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(N, H, device="cuda", generator=g).to(torch.bfloat16)
    std = 1 / math.sqrt(H)
    w = torch.empty(H, V, device="cuda")
    torch.nn.init.trunc_normal_(w, std=std, a=-3 * std, b=3 * std, generator=g)
    w = w.to(torch.bfloat16)
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    y[torch.rand(N, device="cuda", generator=g) < 0.05] = -1
    return x, y, w


def test_full_size_matches_fp64_oracle_on_gpu(big):
    from oracle import lce_forward_backward_fp64

    print("full size vs fp64 oracle (GPU-evaluated)", flush=True)
    x, y, w = big
    out, dx, dw = _fb(x, y, w, n_chunk=4096)
    ref = lce_forward_backward_fp64(x, y, w, -1, 0.0, 1.0, chunk=512)
    assert abs(out[0].item() - ref.loss.item()) <= 1e-3 * ref.loss.item()
    assert abs(out[0].item() - (math.log(131072) + 0.5)) < 0.05  # logits ~ N(0,1): loss ~ log V + 1/2
    for name, got, want in (("dx", dx, ref.dx), ("dw", dw, ref.dw)):
        d = got.double() - want
        emax = (d.abs().max() / want.abs().max()).item()
        el2 = (d.norm() / want.norm()).item()
        print(f"  {name}: max-rel {emax:.3e} l2-rel {el2:.3e}", flush=True)
        assert emax <= 2e-2 and el2 <= 2e-2
    assert (dx[y == -1] == 0).all()
    del ref
    torch.cuda.empty_cache()


def test_full_size_properties(big):
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("full size properties", flush=True)
    x, y, w = big
    V = w.shape[1]
    # zero weight: every lse is exactly log V, loss = log V
    out = linear_cross_entropy(x, y, torch.zeros_like(w), -1, 0.0, 1.0, 4096, True)
    assert abs(out[0].item() - math.log(V)) < 1e-5
    assert abs(out[3].item() - math.log(V)) < 1e-4 and out[2].item() == 0 and out[4].item() == 0
    # zero input: dW = 0 exactly
    _, dx0, dw0 = _fb(torch.zeros_like(x), y, w, n_chunk=4096)
    assert (dw0 == 0).all()
    # row-sum invariant (z_reg = 0): sum_v dW[h, v] = 0 up to rounding of the stored 16-bit entries
    _, dx, dw = _fb(x, y, w, n_chunk=4096)
    s = dw.float().sum(1).abs().max().item()
    a = dw.float().abs().sum(1).max().item()
    assert s <= 2e-3 * a, (s, a)


# ---------------------------------------------------------------------------------------------------------
# The reference's own accuracy protocol (bench_fusions.py:480-512, error measures bench_fusions.py:437-444):
# A ~ randn(V, H) with std 1, x = 0.1*A[y] + randn ("simulate low loss"), no ignored labels, errors as
# torch.dist (L2 norm of the difference) against the fp64 evaluation of the same rounded inputs.  Its published
# figures for its fused operator at this shape are  bf16: |dloss| 4.2e-5, (|ddx|+|ddA|)/2 5.3e-4;
# fp16: 6.9e-5, 1.4e-4  (bench-acc/*over N*.csv:8), on other hardware and another random draw, so this is a
# soft cross-check: same order of magnitude, not equality.
# ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,pub_loss,pub_grad", [(torch.bfloat16, 4.2e-5, 5.3e-4), (torch.float16, 6.9e-5, 1.4e-4)])
def test_reference_accuracy_protocol_full_size(dtype, pub_loss, pub_grad):
    from oracle import lce_forward_backward_fp64

    print(f"reference accuracy protocol {dtype}", flush=True)
    N, H, V = 16384, 2048, 131072
    g = torch.Generator(device="cuda").manual_seed(11)
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    A = torch.randn(V, H, device="cuda", generator=g).to(dtype)
    w = A.T.contiguous()
    x = (0.1 * A[y].float() + torch.randn(N, H, device="cuda", generator=g)).to(dtype)
    del A
    out, dx, dw = _fb(x, y, w, n_chunk=4096)
    ref = lce_forward_backward_fp64(x, y, w, -1, 0.0, 1.0, chunk=512)
    loss_err = abs(out[0].float().item() - ref.loss.float().item())
    dx_err = torch.dist(ref.dx.float(), dx.float()).item()
    dw_err = torch.dist(ref.dw.float(), dw.float()).item()
    grad_err = 0.5 * (dx_err + dw_err)
    print(f"  loss {ref.loss.item():.5f} |dloss| {loss_err:.3e} (published {pub_loss:.1e});  "
          f"(|ddx|+|ddW|)/2 {grad_err:.3e} (published {pub_grad:.1e}); dx {dx_err:.3e} dW {dw_err:.3e}", flush=True)
    # hard gates of this build
    assert loss_err <= 1e-3 * abs(ref.loss.item())
    for got, want in ((dx, ref.dx), (dw, ref.dw)):
        d = got.double() - want
        assert (d.abs().max() / want.abs().max()).item() <= 2e-2
        assert (d.norm() / want.norm()).item() <= 2e-2
    # soft cross-check against the published figures: no worse than twice the reference's own error
    # (observed on MI355X: bf16 0 / 5.3e-4, fp16 0 / 1.1e-4)
    assert loss_err <= 2 * pub_loss
    assert grad_err <= 2 * pub_grad
    del ref
    torch.cuda.empty_cache()


def test_fp32_master_weight_equals_its_16_bit_rounding_bitwise():
    """W in fp32 is rounded once per slab to the compute type; loss and dx must equal, bit for bit, the call on
    the weight rounded by torch, and the fp32 dW must round to the 16-bit dW up to double rounding.  (N_chunk_size is large enough for
    both calls to use one vocabulary slab: the order of the fp32 dx sum over slabs depends on the split.)"""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    print("fp32 master weight vs rounded weight", flush=True)
    for dt, (N, H, V, nc) in ((torch.float16, (1024, 520, 9000, 4096)), (torch.bfloat16, (2048, 1024, 32768, 4096))):
        x, y, w32 = make_inputs(N, H, V, dt, seed=21, ignore_frac=0.1, w_dtype=torch.float32, device="cuda")
        res = []
        for w in (w32, w32.to(dt)):
            xi = x.clone().requires_grad_(True)
            wi = w.clone().requires_grad_(True)
            out = linear_cross_entropy(xi, y, wi, -1, 1e-4, 1.0, nc, True)
            out[0].backward()
            res.append((torch.stack([o.detach() for o in out]), xi.grad, wi.grad))
        assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
        # The 16-bit dW is rounded once from acc*coef (a mixed-precision fma), the fp32 dW is that product rounded
        # to fp32: rounding it again to 16 bits differs on the rare near-ties (double rounding), by one ulp.
        assert res[0][2].dtype == torch.float32
        a, b = res[0][2].to(dt), res[1][2]
        assert (a != b).float().mean().item() < 1e-4
        assert torch.allclose(a.float(), b.float(), rtol=2e-3 if dt == torch.float16 else 1.6e-2, atol=1e-7)


# ---------------------------------------------------------------------------------------------------------
# torch.library registration: operator checks and torch.compile (the reference leaves compile support open:
# `_dynamo.disable` commented out at ops.py:664).  Backend "aot_eager" traces forward and backward through
# fake tensors and the registered autograd formula without generating any device code of its own.
# ---------------------------------------------------------------------------------------------------------
def test_registered_operator_passes_opcheck():
    import linear_cross_entropy_loss_amd  # noqa: F401  (registers torch.ops.lce_amd)

    print("opcheck", flush=True)
    x, y, w = make_inputs(512, 256, 4096, torch.bfloat16, seed=9, ignore_frac=0.1, device="cuda")
    args = (x.requires_grad_(True), y, w.requires_grad_(True), -1, 1e-4, 1.0, 512, True)
    torch.library.opcheck(torch.ops.lce_amd.forward.default, args,
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))


def _head_model(H, V, dtype, hidden=None):
    from linear_cross_entropy_loss_amd import LinearCrossEntropyLoss

    # a fresh trace per test: the packing mode in force while tracing is baked into the graph, and graphs of an
    # earlier test (same shapes, other mode) would otherwise be reused
    torch._dynamo.reset()
    torch.manual_seed(3)
    head = LinearCrossEntropyLoss(H, V, device="cuda", dtype=dtype, ignore_index=-1, z_regularization=1e-4,
                                  logit_scale=0.5)
    body = torch.nn.Linear(hidden or H, H, device="cuda", dtype=dtype)

    def model(x, y):
        return head(torch.nn.functional.gelu(body(x)), y)

    return head, body, model


def _fp64_model_grads(head, body, x, y):
    """Loss and weight gradients of gelu(body(x)) -> scaled logits -> cross-entropy + z-regularisation, by
    autograd in fp64 from library routines only (the definition the oracle itself is pinned against)."""
    F = torch.nn.functional
    wb = body.weight.detach().double().requires_grad_(True)
    bb = body.bias.detach().double().requires_grad_(True)
    wh = head.weight.detach().double().requires_grad_(True)
    h = F.gelu(F.linear(x.double(), wb, bb)).reshape(-1, wh.shape[0])
    z = (h @ wh) * head.logit_scale
    yy = y.reshape(-1)
    loss = F.cross_entropy(z, yy, ignore_index=-1) + head.z_regularization * z.logsumexp(-1)[yy != -1].pow(2).mean()
    loss.backward()
    return loss.detach(), wh.grad, wb.grad


def _run_compiled_and_check(model, compiled, head, body, x, y, eager_bitwise, one_pass=False):
    # (`one_pass` off: the operator that a traced call goes through computes the loss alone in its forward and
    # recomputes the logits in its backward; "always": loss and gradients come from lce_amd.forward_grads and the
    # upstream gradient is multiplied in by lce_amd.scale.  Eager calls make the same device calls under the same
    # setting, and the two are compared bit for bit.  The setting in force while tracing is baked into the graph; the
    # autouse fixture of conftest.py puts the default back.)
    from linear_cross_entropy_loss_amd import ops

    ops.one_pass.set(one_pass)
    loss = model(x, y)
    loss.backward()
    ref = (loss.detach().clone(), head.weight.grad.clone(), body.weight.grad.clone())
    want_loss, want_wh, want_wb = _fp64_model_grads(head, body, x, y)
    for _ in range(2):
        head.weight.grad = None
        body.weight.grad = None
        loss_c = compiled(x, y)
        loss_c.backward()
        torch.cuda.synchronize()
        if eager_bitwise:
            assert torch.equal(loss_c.detach(), ref[0])
            assert torch.equal(head.weight.grad, ref[1])
            assert torch.equal(body.weight.grad, ref[2])
        # the compiled path against fp64 (16-bit activations and parameters: 1e-3 on the loss, 2e-2 on gradients)
        assert abs(loss_c.item() - want_loss.item()) <= 2e-3 * abs(want_loss.item())
        assert max(rel_errors(head.weight.grad, want_wh)) <= 2e-2
        assert max(rel_errors(body.weight.grad, want_wb)) <= 3e-2
    head.weight.grad = None
    body.weight.grad = None


@pytest.mark.parametrize("one_pass", [False, "always", True])
def test_torch_compile_matches_eager_and_fp64(one_pass):
    print(f"torch.compile aot_eager, one_pass={one_pass}", flush=True)
    head, body, model = _head_model(256, 5000, torch.bfloat16)
    x = torch.randn(4, 150, 256, device="cuda", dtype=torch.bfloat16)
    y = torch.randint(0, 5000, (4, 150), device="cuda")
    y[0, :7] = -1
    compiled = torch.compile(model, backend="aot_eager", fullgraph=True)
    _run_compiled_and_check(model, compiled, head, body, x, y, eager_bitwise=True, one_pass=one_pass)


@pytest.mark.parametrize("one_pass", [False, "always"])
def test_torch_compile_odd_shapes_and_strided_weight(one_pass):
    """in_features and out_features that are not multiples of 8 (the host makes padded copies for the kernels)
    and a head weight that is a strided view: the fake kernels of the registered operator must describe what
    the real ones return (shapes, dtypes, contiguity), or the traced backward would not line up."""
    print(f"torch.compile aot_eager, odd shapes, one_pass={one_pass}", flush=True)
    head, body, model = _head_model(100, 1001, torch.float16, hidden=72)
    x = torch.randn(3, 50, 72, device="cuda", dtype=torch.float16)
    y = torch.randint(0, 1001, (3, 50), device="cuda")
    y[1, :5] = -1
    compiled = torch.compile(model, backend="aot_eager", fullgraph=True)
    _run_compiled_and_check(model, compiled, head, body, x, y, eager_bitwise=True, one_pass=one_pass)
    # the functional form on a transposed (V, H) -> (H, V) view of a weight, compiled, against the oracle
    from linear_cross_entropy_loss_amd import linear_cross_entropy
    from oracle import lce_forward_backward_fp64

    A = (torch.randn(1001, 100, device="cuda") * 0.1).to(torch.float16).requires_grad_(True)
    xin = torch.randn(150, 100, device="cuda", dtype=torch.float16, requires_grad=True)
    yy = y.reshape(-1)

    def fn(xi, Ai):
        return linear_cross_entropy(xi, yy, Ai.t(), -1, 1e-4, 0.5, 512, True)

    out = torch.compile(fn, backend="aot_eager", fullgraph=True)(xin, A)
    out[0].backward()
    ref = lce_forward_backward_fp64(xin.detach().double(), yy, A.detach().t().double(), -1, 1e-4, 0.5)
    assert abs(out[0].item() - ref.loss.item()) <= 1e-3 * abs(ref.loss.item())
    assert abs(out[3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
    assert max(rel_errors(xin.grad, ref.dx)) <= 2e-2 and max(rel_errors(A.grad.t(), ref.dw)) <= 2e-2
    assert A.grad.shape == A.shape


@pytest.mark.parametrize("one_pass", [False, "always"])
def test_torch_compile_inductor_around_the_operator(one_pass):
    """The default backend (inductor, what the reference's own probe uses: variants/compile_tests_NV5.py:535
    compiles with mode="max-autotune") generates the kernels of the surrounding Linear + gelu; the fused loss
    stays an opaque registered operator inside the compiled graph, forward and backward."""
    print(f"torch.compile inductor, one_pass={one_pass}", flush=True)
    head, body, model = _head_model(256, 4096, torch.bfloat16)
    x = torch.randn(2, 256, 256, device="cuda", dtype=torch.bfloat16)
    y = torch.randint(0, 4096, (2, 256), device="cuda")
    y[0, :9] = -1
    compiled = torch.compile(model, fullgraph=True)
    # inductor fuses bias + gelu its own way, so the activations handed to the loss differ from eager's in the
    # last bit: checked against fp64, not bitwise against eager
    _run_compiled_and_check(model, compiled, head, body, x, y, eager_bitwise=False, one_pass=one_pass)


def test_registered_backward_operator_passes_opcheck():
    import linear_cross_entropy_loss_amd  # noqa: F401

    print("opcheck backward", flush=True)
    x, y, w = make_inputs(300, 100, 1001, torch.bfloat16, seed=12, ignore_frac=0.1, device="cuda")
    out5, lse, n_valid = torch.ops.lce_amd.forward(x, y, w, -1, 1e-4, 1.0, 512, False)
    g = torch.ones(1, device="cuda")
    for need_dx, need_dw in ((True, True), (True, False), (False, True)):
        torch.library.opcheck(torch.ops.lce_amd.backward.default,
                              (x, y, w, lse, n_valid, g, -1, 1e-4, 1.0, 512, need_dx, need_dw),
                              test_utils=("test_schema", "test_faketensor"))


def test_operators_of_the_one_pass_route_pass_opcheck_and_equal_the_eager_function():
    """lce_amd.forward_grads (loss and gradients in one call) and lce_amd.scale: schema, fake kernels and autograd
    registration; and, taken wherever the route fits, bit for bit what LinearXentImplementation gives in eager mode,
    also for an upstream gradient other than 1, a weight stored (V, H) and a second backward over the same graph."""
    from linear_cross_entropy_loss_amd import LinearXentImplementation, ops

    print("opcheck forward_grads / scale", flush=True)
    x, y, w = make_inputs(600, 104, 3001, torch.bfloat16, seed=13, ignore_frac=0.1, device="cuda")
    for need_dx, need_dw in ((True, True), (True, False), (False, True)):
        args = (x.clone().requires_grad_(need_dx), y, w.clone().requires_grad_(need_dw), -1, 1e-4, 0.5, 512, True,
                need_dx, need_dw, 0, True)
        torch.library.opcheck(torch.ops.lce_amd.forward_grads.default, args,
                              test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
    f = torch.full((1,), 0.37, device="cuda")
    torch.library.opcheck(torch.ops.lce_amd.scale.default, (w, f), test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(torch.ops.lce_amd.scale.default, (w.t(), f), test_utils=("test_schema", "test_faketensor"))
    assert torch.equal(torch.ops.lce_amd.scale(w.t(), f), (w.t().float() * 0.37).to(w.dtype))
    assert torch.equal(torch.ops.lce_amd.scale(x[:7, :3].contiguous(), f), (x[:7, :3].float() * 0.37).to(x.dtype))

    ops.one_pass.set("always")
    for dt in (torch.bfloat16, torch.float16):
        for vh in (False, True):
            # (a problem that the one-pass route covers: on others the eager function folds the upstream gradient into
            # its backward kernels, while the operator rounds twice)
            x, y, w = make_inputs(2000, 256, 5000, dt, seed=14, ignore_frac=0.1, device="cuda")
            res = []
            for via_op in (False, True):
                xi = x.clone().requires_grad_(True)
                wi = (w.t().contiguous() if vh else w.clone()).requires_grad_(True)
                wv = wi.t() if vh else wi
                if via_op:
                    out = torch.ops.lce_amd.forward_grads(xi, y, wv, -1, 1e-4, 0.5, 1024, True, True, True,
                                                          int(ops.pack_rows.get()), True)[0].unbind(0)
                else:
                    out = LinearXentImplementation.apply(xi, y, wv, -1, 1e-4, 0.5, 1024, True)
                (out[0] * 3.0).backward(retain_graph=True)
                first = (xi.grad.clone(), wi.grad.clone())
                xi.grad = wi.grad = None
                (out[0] * 3.0).backward()  # the eager function recomputes here; the operator scales its saved gradients again
                res.append((torch.stack([o.detach() for o in out]), first, (xi.grad, wi.grad)))
            assert torch.equal(res[0][0], res[1][0])
            for a, b in zip(res[0][1], res[1][1]):
                assert torch.equal(a, b), (dt, vh)
            for a, b in zip(res[0][2], res[1][2]):  # (recomputed against saved: rounding only)
                assert max(rel_errors(b, a)) <= 1.5e-2, (dt, vh)


def test_autocast_follows_a_16_bit_weight_and_mismatched_dtypes_are_named():
    """Under autocast the activations take the weight's own 16-bit type (bf16 parameters under the default fp16
    autocast: the input is cast to bf16, nothing is copied); without autocast a dtype mismatch is an error that
    says so."""
    from linear_cross_entropy_loss_amd import LinearCrossEntropyLoss, linear_cross_entropy
    from oracle import lce_forward_backward_fp64

    print("autocast with 16-bit parameters", flush=True)
    torch.manual_seed(5)
    m = LinearCrossEntropyLoss(256, 4096, device="cuda", dtype=torch.bfloat16, ignore_index=-1, N_chunk_size=512)
    x = torch.randn(300, 256, device="cuda", requires_grad=True)  # fp32 activations
    y = torch.randint(0, 4096, (300,), device="cuda")
    with torch.autocast("cuda", dtype=torch.float16):
        loss = m(x, y)
    loss.backward()
    assert x.grad.dtype == torch.float32 and m.weight.grad.dtype == torch.bfloat16
    ref = lce_forward_backward_fp64(x.detach().bfloat16().double(), y, m.weight.detach().double(), -1)
    assert abs(loss.item() - ref.loss.item()) <= 1e-3 * ref.loss.item()
    assert max(rel_errors(x.grad, ref.dx)) <= 2e-2 and max(rel_errors(m.weight.grad, ref.dw)) <= 2e-2
    with pytest.raises(ValueError, match="share a dtype"):
        linear_cross_entropy(x.detach().half(), y, m.weight.detach(), -1)


def test_function_and_registered_operator_agree_bitwise():
    from linear_cross_entropy_loss_amd import LinearXentImplementation, linear_cross_entropy, ops

    print("Function vs operator", flush=True)
    x, y, w = make_inputs(777, 264, 10008, torch.float16, seed=10, ignore_frac=0.1, device="cuda")
    res = []

    def via_operator(x, y, w, *cfg):  # what linear_cross_entropy calls while torch.compile traces
        return torch.ops.lce_amd.forward(x, y, w, *cfg, ops.pack_rows.get())[0].unbind(0)

    for fn in (LinearXentImplementation.apply, linear_cross_entropy, via_operator):
        xi = x.clone().requires_grad_(True)
        wi = w.clone().requires_grad_(True)
        out = fn(xi, y, wi, -1, 1e-4, 0.5, 512, True)
        out[0].backward()
        res.append((torch.stack([o.detach() for o in out]), xi.grad, wi.grad))
    for other in res[1:]:
        for a, b in zip(res[0], other):
            assert torch.equal(a, b)


@pytest.mark.parametrize("one_pass", [False, True])
def test_forward_backward_can_be_captured_in_a_hip_graph(one_pass):
    """The library only enqueues kernels on the caller's stream (no synchronisation, no memset nodes, no
    allocation of its own), so a whole loss + backward step can be captured once and replayed; every replay,
    with eager work and synchronisations in between, must equal the eager result bit for bit.  On both routes:
    two passes (here with the monitoring values), and loss and gradients from one evaluation of the logits in
    several chunks of token rows, whose row counts the kernels also take from device memory."""
    from linear_cross_entropy_loss_amd import _lib, linear_cross_entropy, ops

    print(f"hip graph capture, one pass: {one_pass}", flush=True)
    N, H, V = (4096 if one_pass else 1024), 512, 10000
    x, y, w = make_inputs(N, H, V, torch.bfloat16, seed=3, ignore_frac=0.1, device="cuda")
    xs, ws, ys = x.clone().requires_grad_(True), w.clone().requires_grad_(True), y.clone()
    if one_pass:
        ops.one_pass.set("always")  # (the autouse fixtures of conftest.py put the default back)
        prob = _lib.make_problem(N, H, V, H, V, H, V, torch.bfloat16, torch.bfloat16, torch.bfloat16, torch.bfloat16, -1,
                                 1.0, 1e-4, 1500, False, 0, int(ops.pack_rows.get()), 0, 0, _lib.ROUTE_ONE_PASS)
        assert _lib.forward_backward_plan(prob)[0] > 1

    def step(xi, yi, wi):
        out = linear_cross_entropy(xi, yi, wi, -1, 1e-4, 1.0, 1500 if one_pass else 512, not one_pass)
        out[0].backward()
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            xs.grad = None
            ws.grad = None
            step(xs, ys, ws)
    torch.cuda.current_stream().wait_stream(side)
    xs.grad = None
    ws.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = step(xs, ys, ws)
    for trial in range(3):
        # other labels on every replay, with another number of ignored ones: the kernels take the number of
        # rows they work on from device memory (0 ignored: nothing is packed and dx is written in place)
        x2, y2, w2 = make_inputs(N, H, V, torch.bfloat16, seed=10 + trial, ignore_frac=(0.0, 0.1, 0.6)[trial],
                                 device="cuda")
        with torch.no_grad():
            xs.copy_(x2)
            ws.copy_(w2)
            ys.copy_(y2)
        graph.replay()
        torch.cuda.synchronize()
        got = (torch.stack([o.detach() for o in out_g]).clone(), xs.grad.clone(), ws.grad.clone())
        xe, we = x2.clone().requires_grad_(True), w2.clone().requires_grad_(True)
        oe = step(xe, y2, we)
        torch.cuda.synchronize()
        assert torch.equal(got[0], torch.stack([o.detach() for o in oe]))
        assert torch.equal(got[1], xe.grad) and torch.equal(got[2], we.grad)

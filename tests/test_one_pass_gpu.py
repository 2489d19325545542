"""lce_forward_backward: loss and gradients from one evaluation of the logits, through the C ABI.

Checked against the fp64 oracle to the operator's tolerances (loss 1e-3, gradients 2e-2) and against lce_forward +
lce_backward on the same inputs: lse and loss to fp32 rounding (both sum the same fp32 logits, in another order),
the gradients to the second rounding of the staged dz (16-bit: 2^-8 relative per element before the contraction).
"""
import ctypes

import pytest
import torch

from helpers import make_inputs, rel_errors

pytestmark = pytest.mark.gpu


def P(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _problem(N, H, V, x, w, dt, dw_dt, z_reg, scale, n_chunk, pack, layout, phases=0, mon=False, exact=False):
    from linear_cross_entropy_loss_amd import _lib

    hp, cols = H + (-H) % 8, (H if layout else V)
    return _lib.make_problem(N, H, V, x.stride(0), w.stride(0), hp, cols + (-cols) % 8, dt, w.dtype, dt, dw_dt, -1, scale,
                             z_reg, n_chunk, mon, phases, pack, 0, layout,
                             _lib.ROUTE_ONE_PASS | (_lib.ROUTE_EXACT_SUMS if exact else 0))


def _both_routes(N, H, V, dt, n_chunk, ignore, z_reg=0.0, scale=1.0, pack=0, layout=0, dw_dt=None, grad_out=1.0,
                 seed=7, want_chunks=None, w_dt=None, mon=False, exact=False):
    """Runs the two routes on the same inputs; returns (inputs on the CPU, two-pass outputs, one-pass outputs)."""
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    x, y, w = make_inputs(N, H, V, dt, seed, ignore_frac=ignore, w_dtype=w_dt)
    xd, yd, wd = x.cuda(), y.cuda(), (w.t().contiguous() if layout else w).cuda()
    if w_dt is not None:
        dw_dt = w_dt  # (the gradient of an fp32 master weight is fp32)
    if wd.stride(0) % 8:  # rows of the weight on 16-byte boundaries
        pad = torch.zeros(wd.shape[0], wd.shape[1] + (-wd.shape[1]) % 8, dtype=wd.dtype, device="cuda")
        pad[:, :wd.shape[1]] = wd
        wd = pad[:, :wd.shape[1]]
    if xd.stride(0) % 8:
        pad = torch.zeros(N, H + (-H) % 8, dtype=xd.dtype, device="cuda")
        pad[:, :H] = xd
        xd = pad[:, :H]
    dw_dt = dw_dt or dt
    prob = _problem(N, H, V, xd, wd, dt, dw_dt, z_reg, scale, n_chunk, pack, layout, mon=mon, exact=exact)
    chunks, rows = _lib.forward_backward_plan(prob)
    print(f"N={N} H={H} V={V} {dt} n_chunk={n_chunk} pack={pack} layout={layout}: {chunks} chunks of {rows} rows", flush=True)
    assert chunks > 0, "this case is meant to take the one-pass route"
    if want_chunks is not None:
        assert chunks >= want_chunks
    fb, bb = _lib.workspace_bytes(prob)
    ub = _lib.forward_backward_workspace_bytes(prob)
    ws = torch.empty(max(fb, bb, ub), dtype=torch.uint8, device="cuda")
    g = torch.full((1,), grad_out, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    hp = H + (-H) % 8

    def outs():
        shape = (V, hp) if layout else (H, V + (-V) % 8)
        return dict(lse=torch.full((N,), 7.0, device="cuda"), out5=torch.zeros(5, device="cuda"),
                    nv=torch.zeros(1, dtype=torch.int64, device="cuda"),
                    dx=torch.full((N, hp), 3.0, dtype=dt, device="cuda"), dw=torch.full(shape, 3.0, dtype=dw_dt, device="cuda"))

    a, b = outs(), outs()
    rc = lib.lce_forward(ctypes.byref(prob), P(xd), P(wd), P(yd), P(a["lse"]), P(a["out5"]), P(a["nv"]), P(ws), ws.numel(), st)
    assert rc == 0
    rc = lib.lce_backward(ctypes.byref(prob), P(xd), P(wd), P(yd), P(a["lse"]), P(a["nv"]), P(g), P(a["dx"]), P(a["dw"]),
                          P(ws), ws.numel(), st)
    assert rc == 0
    torch.cuda.synchronize()
    ws.fill_(0x5a)  # nothing in the workspace has to start at any value
    rc = lib.lce_forward_backward(ctypes.byref(prob), P(xd), P(wd), P(yd), P(g), P(b["lse"]), P(b["out5"]), P(b["nv"]),
                                  P(b["dx"]), P(b["dw"]), P(ws), ub, st)
    assert rc == 0, (rc, lib.lce_last_hip_error())
    torch.cuda.synchronize()
    b["chunks"], b["rows"], b["workspace"] = chunks, rows, ub
    for o in (a, b):
        o["dx"] = o["dx"][:, :H]
        o["dw"] = o["dw"][:, :H].t() if layout else o["dw"][:, :V]
    return (x, y, w), a, b


def _check(inputs, a, b, z_reg, scale, grad_out=1.0, fp64=True):
    x, y, w = inputs
    assert a["nv"].item() == b["nv"].item() == int((y != -1).sum())
    # the same fp32 logits summed in another order
    assert abs(a["out5"][0].item() - b["out5"][0].item()) <= 2e-6 * abs(a["out5"][0].item())
    assert abs(a["out5"][1].item() - b["out5"][1].item()) <= 4e-6 * abs(a["out5"][1].item()) + 1e-12
    assert rel_errors(b["lse"], a["lse"])[0] <= 1e-6
    assert (b["lse"].cpu()[y == -1] == 0).all()
    # ignored tokens: exact zeros
    assert (b["dx"].cpu()[y == -1] == 0).all()
    for name in ("dx", "dw"):
        emax, el2 = rel_errors(b[name], a[name])
        print(f"  {name} one-pass vs two-pass: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert emax <= 1.5e-2 and el2 <= 3e-3, (name, emax, el2)
    if fp64:
        from oracle import lce_forward_backward_fp64

        ref = lce_forward_backward_fp64(x.double(), y, w.double(), -1, z_reg, scale, grad_out)
        assert abs(b["out5"][0].item() - ref.loss.item()) <= 1e-3 * abs(ref.loss.item())
        for name, want in (("dx", ref.dx), ("dw", ref.dw)):
            emax, el2 = rel_errors(b[name], want)
            print(f"  {name} one-pass vs fp64: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
            assert emax <= 2e-2 and el2 <= 2e-2, (name, emax, el2)


CASES = [
    # N, H, V, dtype, n_chunk, ignored, z_reg, scale, pack, layout, dW dtype, grad_out
    (4096, 512, 4096, torch.bfloat16, 1024, 0.1, 0.0, 1.0, 2, 0, None, 1.0),        # 16 chunks, all rows computed
    (4096, 512, 4096, torch.bfloat16, 2048, 0.1, 0.0, 1.0, 1, 0, None, 1.0),        # packed rows, several chunks
    (4000, 520, 5000, torch.float16, 2048, 0.1, 1e-3, 0.7, 1, 0, None, 0.37),       # ragged shapes, fp16, z-reg
    (4000, 520, 5000, torch.bfloat16, 1200, 0.1, 0.0, 1.0, 2, 1, None, 1.0),        # weight stored (V, H)
    (4000, 520, 5000, torch.bfloat16, 2048, 0.1, 1e-4, 1.0, 1, 1, None, 2.5),       # (V, H), packed
    (4000, 520, 5000, torch.bfloat16, 2048, 0.7, 0.0, 1.0, 1, 0, torch.float32, 1.0),   # chunks without a row; fp32 dW
    (2048, 1024, 8192, torch.bfloat16, 4096, 0.0, 0.0, 1.0, 0, 0, torch.float32, 1.0),  # a single chunk: no plane
    (1000, 300, 777, torch.float16, 4096, 0.2, 0.0, 2.0, 1, 0, None, 1.0),          # single chunk, nothing a multiple of 8
    (8192, 1024, 32768, torch.bfloat16, 4096, 0.05, 0.0, 1.0, 0, 0, None, 1.0),     # mid size: 3 chunks
]

# fp32 master weight under 16-bit activations: N, H, V, dtype of x, n_chunk, ignored, z_reg, scale, pack, layout
MASTER_CASES = [
    (4096, 512, 4096, torch.bfloat16, 2048, 0.1, 0.0, 1.0, 1, 0),
    (4000, 520, 5000, torch.float16, 2048, 0.1, 1e-3, 0.7, 1, 0),
    (4000, 520, 5000, torch.bfloat16, 2048, 0.3, 0.0, 1.0, 2, 1),
    (1000, 304, 777, torch.float16, 4096, 0.2, 0.0, 2.0, 1, 0),      # a single chunk
]


@pytest.mark.pack_auto
@pytest.mark.parametrize("N,H,V,dt,n_chunk,ign,z_reg,scale,pack,layout", MASTER_CASES)
def test_one_pass_with_an_fp32_master_weight(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout):
    inputs, a, b = _both_routes(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout, w_dt=torch.float32)
    assert b["dw"].dtype == torch.float32
    _check(inputs, a, b, z_reg, scale, 1.0, fp64=True)


@pytest.mark.pack_auto
@pytest.mark.parametrize("N,H,V,dt,n_chunk,ign,z_reg,scale,pack,layout,dw_dt,grad_out", CASES)
def test_one_pass_matches_two_pass_and_the_fp64_oracle(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout, dw_dt, grad_out):
    inputs, a, b = _both_routes(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout, dw_dt, grad_out)
    _check(inputs, a, b, z_reg, scale, grad_out, fp64=N * V <= 4096 * 8192)


# the monitoring values on the one-pass route (the forward then runs on all rows): N, H, V, dtype, n_chunk, ignored, z_reg,
# scale, pack, layout
MON_CASES = [
    (4096, 512, 4096, torch.bfloat16, 2048, 0.1, 1e-4, 1.0, 1, 0),
    (4000, 512, 5000, torch.float16, 2048, 0.3, 1e-3, 0.5, 2, 0),    # the tile column that straddles V
    (4000, 640, 5000, torch.bfloat16, 2048, 0.1, 0.0, 2.0, 1, 1),    # weight stored (V, H)
    (1000, 384, 777, torch.float16, 4096, 0.2, 0.0, 1.0, 0, 0),      # a single chunk
    # packed (1 = always): the dropped tokens follow the kept ones; 8 chunks of 512 rows, the last five without a kept row
    (4096, 512, 4096, torch.bfloat16, 1024, 0.7, 1e-4, 1.0, 1, 0),
    (6000, 256, 3000, torch.float16, 1024, 0.45, 0.0, 0.5, 1, 1),    # 6 chunks, the edge of dW cuts tiles, (V, H)
    (4096, 512, 4096, torch.float16, 1024, 0.97, 0.0, 1.0, 1, 0),    # kept rows in the first chunk only
    # hidden sizes that are no multiple of 128: the K mask and the monitoring sums together
    (3000, 520, 5000, torch.bfloat16, 1024, 0.1, 1e-4, 1.0, 1, 0),
    (3000, 200, 4096, torch.float16, 1024, 0.3, 0.0, 0.5, 2, 1),
    (700, 72, 777, torch.bfloat16, 4096, 0.0, 1e-3, 2.0, 0, 0),
]


@pytest.mark.pack_auto
@pytest.mark.parametrize("N,H,V,dt,n_chunk,ign,z_reg,scale,pack,layout", MON_CASES)
def test_one_pass_with_the_monitoring_values(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout):
    inputs, a, b = _both_routes(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout, mon=True)
    _check(inputs, a, b, z_reg, scale, 1.0, fp64=True)
    # logit_max exactly, entropy and norm to fp32 summation order
    assert a["out5"][2].item() == b["out5"][2].item()
    for i in (3, 4):
        assert abs(a["out5"][i].item() - b["out5"][i].item()) <= 2e-5 * abs(a["out5"][i].item()), (i, a["out5"], b["out5"])
    from oracle import lce_forward_backward_fp64

    x, y, w = inputs
    ref = lce_forward_backward_fp64(x.double(), y, w.double(), -1, z_reg, scale, 1.0)
    assert abs(b["out5"][2].item() - ref.logit_max.item()) <= 1e-3 * abs(ref.logit_max.item())
    assert abs(b["out5"][3].item() - ref.logit_entropy.item()) <= 2e-3 * abs(ref.logit_entropy.item())
    assert abs(b["out5"][4].item() - ref.logit_norm.item()) <= 2e-3 * abs(ref.logit_norm.item())


# Hidden sizes near twice N_chunk_size and above: the lower halves of the sums of a 16-bit dW do not fit the bound, and
# the route keeps a byte of each (sums of 24 bits, rounded to nearest each time they go back to memory).
# N, H, V, dtype, n_chunk, ignored, z_reg, scale, pack, layout
LO8_CASES = [
    (2048, 1536, 12288, torch.bfloat16, 1024, 0.1, 0.0, 1.0, 1, 0),
    (2048, 2048, 12288, torch.float16, 1024, 0.3, 1e-4, 0.5, 2, 1),
    (4096, 1536, 20000, torch.bfloat16, 1024, 0.1, 1e-3, 2.0, 0, 0),   # 16 chunks; the edge of dW cuts tiles
    (4096, 1400, 16000, torch.float16, 1024, 0.6, 0.0, 1.0, 1, 1),     # both edges; chunks without a kept row
]


@pytest.mark.pack_auto
@pytest.mark.parametrize("N,H,V,dt,n_chunk,ign,z_reg,scale,pack,layout", LO8_CASES)
def test_sums_of_dw_with_a_byte_of_each_lower_half(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout):
    from linear_cross_entropy_loss_amd import _lib

    inputs, a, b = _both_routes(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout, want_chunks=4)
    # (this is such a problem: the workspace is smaller than the chunk's stage plus two bytes per element of dW)
    hp, vp = H + (-H) % 256, V + (-V) % 256
    assert b["workspace"] < hp * vp * 2 + b["rows"] * vp * 2
    _check(inputs, a, b, z_reg, scale, 1.0, fp64=True)
    # against the two-pass route, whose sums never leave fp32 registers: what the 24 bits cost is far below the rounding
    # of the 16-bit result (2^-9 in bf16, 2^-12 in fp16); the gradients differ by the staged dz's second rounding
    emax, el2 = rel_errors(b["dw"], a["dw"])
    assert el2 <= 3e-3


@pytest.mark.pack_auto
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_exact_sums_flag_keeps_the_halves_and_changes_only_the_rounding(dt):
    """N=8192, H=2048, V=16384 at N_chunk_size 2048 (H = N_chunk_size: the lower halves take half of the bound): the
    library's plan keeps a byte per sum and runs longer chunks; with LCE_ROUTE_EXACT_SUMS it keeps both halves, in more
    and shorter chunks.  Both agree with the two-pass route and with fp64, and with each other to the rounding of dz
    and of the 24 bits."""
    a_inputs, a2, fast = _both_routes(8192, 2048, 16384, dt, 2048, 0.1, 1e-4, 1.0, 1, 0, seed=21)
    b_inputs, b2, exact = _both_routes(8192, 2048, 16384, dt, 2048, 0.1, 1e-4, 1.0, 1, 0, seed=21, exact=True)
    assert fast["chunks"] > 1 and exact["chunks"] > fast["chunks"]
    _check(a_inputs, a2, fast, 1e-4, 1.0, 1.0, fp64=True)
    _check(b_inputs, b2, exact, 1e-4, 1.0, 1.0, fp64=True)
    assert torch.equal(fast["lse"], exact["lse"]) or rel_errors(fast["lse"], exact["lse"])[0] <= 1e-6
    for name in ("dx", "dw"):
        emax, el2 = rel_errors(fast[name], exact[name])
        print(f"  {name} bytes vs halves: max-rel {emax:.3e}  l2-rel {el2:.3e}", flush=True)
        assert el2 <= 3e-3


@pytest.mark.pack_auto
def test_fp16_z_regularisation_with_lse_near_a_thousand_on_the_one_pass_route():
    from linear_cross_entropy_loss_amd import linear_cross_entropy, ops

    ops.one_pass.set("always")  # (the autouse fixtures of conftest.py put the default back)

    N, H, V = 1024, 256, 4096
    x, y, w = make_inputs(N, H, V, torch.float16, seed=11, ignore_frac=0.1)
    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    out = linear_cross_entropy(xd, y.cuda(), wd, -1, 0.03, 205.0, 4096, False)
    out[0].backward()
    torch.cuda.synchronize()
    assert torch.isfinite(out[0]) and torch.isfinite(xd.grad).all() and torch.isfinite(wd.grad).all()
    from oracle import lce_forward_backward_fp64

    ref = lce_forward_backward_fp64(x.double(), y, w.double(), -1, 0.03, 205.0, 1.0)
    assert abs(out[0].item() - ref.loss.item()) <= 1e-3 * abs(ref.loss.item())
    assert max(rel_errors(xd.grad, ref.dx)) <= 2e-2 and max(rel_errors(wd.grad, ref.dw)) <= 2e-2


@pytest.mark.pack_auto
def test_a_second_backward_recomputes_and_the_upstream_gradient_is_multiplied_in_fp32():
    from linear_cross_entropy_loss_amd import linear_cross_entropy, ops

    ops.one_pass.set("always")

    N, H, V = 2048, 512, 8192
    x, y, w = make_inputs(N, H, V, torch.bfloat16, seed=5, ignore_frac=0.1)
    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    loss = linear_cross_entropy(xd, y.cuda(), wd, -1, 0.0, 1.0, 4096, False)[0]
    g = 1.0 / 3.0
    (loss * g).backward(retain_graph=True)
    first = (xd.grad.clone(), wd.grad.clone())
    xd.grad = wd.grad = None
    (loss * g).backward()  # nothing is left from the forward: the logit tiles are recomputed
    torch.cuda.synchronize()
    from oracle import lce_forward_backward_fp64

    ref = lce_forward_backward_fp64(x.double(), y, w.double(), -1, 0.0, 1.0, g)
    for got in (first, (xd.grad, wd.grad)):
        assert max(rel_errors(got[0], ref.dx)) <= 2e-2 and max(rel_errors(got[1], ref.dw)) <= 2e-2
    assert max(rel_errors(first[0], xd.grad)) <= 1.5e-2 and max(rel_errors(first[1], wd.grad)) <= 1.5e-2
    # the factor is not rounded to 16 bits before it is applied: the sum of dW follows it to 1e-3
    ones = lce_forward_backward_fp64(x.double(), y, w.double(), -1, 0.0, 1.0, 1.0)
    ratio = (first[1].double().cpu() * ones.dw).sum() / (ones.dw * ones.dw).sum()
    assert abs(ratio.item() - g) <= 1e-3 * g


@pytest.mark.pack_auto
def test_scale_with_a_factor_of_one_touches_nothing_and_other_factors_round_once():
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        m = 4 if dt == torch.float32 else 8
        t = torch.randn(37, 104 + m, device="cuda").to(dt)
        view = t[:, :101]  # the last piece of a row is cut
        before = t.clone()
        one = torch.ones(1, device="cuda")
        assert lib.lce_scale(P(view), _lib.dtype_code(dt), 37, 101, t.stride(0), P(one), st) == 0
        torch.cuda.synchronize()
        assert torch.equal(t, before)
        f = torch.full((1,), 1.0 / 3.0, device="cuda")
        assert lib.lce_scale(P(view), _lib.dtype_code(dt), 37, 101, t.stride(0), P(f), st) == 0
        torch.cuda.synchronize()
        assert torch.equal(t[:, :101], (before[:, :101].float() * f).to(dt))
        assert torch.equal(t[:, 101:], before[:, 101:])  # nothing past the columns
    assert lib.lce_scale(P(view), 7, 37, 101, t.stride(0), P(one), st) == _lib.LCE_EINVAL_DTYPE
    assert lib.lce_scale(P(view), _lib.LCE_F32, 37, 101, 50, P(one), st) == _lib.LCE_EINVAL_ARG


@pytest.mark.pack_auto
def test_problems_outside_the_one_pass_route_take_the_two_calls_inside_the_entry_point():
    """fp32 activations: lce_forward_backward runs lce_forward and lce_backward itself, bit for bit."""
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    N, H, V = 512, 256, 4096
    x, y, w = make_inputs(N, H, V, torch.float32, seed=3, ignore_frac=0.1, device="cuda")
    prob = _lib.make_problem(N, H, V, H, V, H, V, torch.float32, torch.float32, torch.float32, torch.float32, -1, 1.0, 0.0,
                             512, False)
    assert _lib.forward_backward_plan(prob) == (0, 0)
    fb, bb = _lib.workspace_bytes(prob)
    ub = _lib.forward_backward_workspace_bytes(prob)
    assert ub == max(fb, bb)
    ws = torch.empty(ub, dtype=torch.uint8, device="cuda")
    g = torch.ones(1, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = lambda: dict(lse=torch.zeros(N, device="cuda"), out5=torch.zeros(5, device="cuda"),
                        nv=torch.zeros(1, dtype=torch.int64, device="cuda"), dx=torch.zeros(N, H, device="cuda"),
                        dw=torch.zeros(H, V, device="cuda"))
    a, b = outs(), outs()
    assert lib.lce_forward(ctypes.byref(prob), P(x), P(w), P(y), P(a["lse"]), P(a["out5"]), P(a["nv"]), P(ws), ub, st) == 0
    assert lib.lce_backward(ctypes.byref(prob), P(x), P(w), P(y), P(a["lse"]), P(a["nv"]), P(g), P(a["dx"]), P(a["dw"]),
                            P(ws), ub, st) == 0
    assert lib.lce_forward_backward(ctypes.byref(prob), P(x), P(w), P(y), P(g), P(b["lse"]), P(b["out5"]), P(b["nv"]),
                                    P(b["dx"]), P(b["dw"]), P(ws), ub, st) == 0
    torch.cuda.synchronize()
    for k in a:
        assert torch.equal(a[k], b[k]), k


@pytest.mark.pack_auto
@pytest.mark.parametrize("layout", [0, 1])
def test_sums_over_chunks_kept_in_dw_stay_inside_dw(layout):
    """A 16-bit dW summed over several chunks holds the upper halves of its fp32 sums while the call runs: with dW a
    view of a wider buffer (rows 72 elements longer than they need to be), nothing beyond the 8 elements of stride
    padding that the stores of a row may touch is written, the rows behind the last one included, and the result is
    the one a dense dW gets, bit for bit."""
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    N, H, V, dt = 3000, 520, 5000, torch.bfloat16   # the edge of dW cuts tiles in both directions
    x, y, w = make_inputs(N, H, V, dt, seed=11, ignore_frac=0.1, device="cuda")
    hp, vp = H + (-H) % 8, V + (-V) % 8
    xd = torch.zeros(N, hp, dtype=dt, device="cuda")
    xd[:, :H] = x
    rows, cols = (V, H) if layout else (H, V)
    cp = cols + (-cols) % 8
    wd = torch.zeros(rows, cp, dtype=dt, device="cuda")
    wd[:, :cols] = w.t() if layout else w
    g = torch.ones(1, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    results = []
    for extra in (0, 72):
        ld = cp + extra
        prob = _lib.make_problem(N, H, V, hp, cp, hp, ld, dt, dt, dt, dt, -1, 1.0, 0.0, 1024, False, 0, 1, 0, layout,
                                 _lib.ROUTE_ONE_PASS)
        chunks, _ = _lib.forward_backward_plan(prob)
        assert chunks >= 3
        ub = _lib.forward_backward_workspace_bytes(prob)
        ws = torch.empty(ub, dtype=torch.uint8, device="cuda")
        buf = torch.full((rows + 4, ld), 7.0, dtype=dt, device="cuda")   # four more rows behind dW
        lse, out5 = torch.zeros(N, device="cuda"), torch.zeros(5, device="cuda")
        nv, dx = torch.zeros(1, dtype=torch.int64, device="cuda"), torch.zeros(N, hp, dtype=dt, device="cuda")
        print(f"layout={layout} ld={ld}: {chunks} chunks", flush=True)
        rc = lib.lce_forward_backward(ctypes.byref(prob), P(xd), P(wd), P(y), P(g), P(lse), P(out5), P(nv), P(dx), P(buf),
                                      P(ws), ub, st)
        assert rc == 0, (rc, lib.lce_last_hip_error())
        torch.cuda.synchronize()
        assert (buf[rows:] == 7.0).all()
        assert (buf[:rows, cp:] == 7.0).all()
        results.append(buf[:rows, :cols].clone())
    assert torch.equal(results[0], results[1])


@pytest.mark.pack_auto
def test_forty_draws_over_chunks_packing_monitoring_and_layouts():
    """Seeded draws over what the one-pass route varies at once -- the number of chunks (1 to 20), the three packing
    modes with none to nine tenths of the labels ignored, the monitoring values, both weight layouts, a 16-bit or fp32
    dW, z-regularisation and scale, shapes that the tiles do not divide -- each against the two-pass route and, where
    the fp64 oracle is quick, against that."""
    import random

    rng = random.Random(9)
    ran = several = 0
    for it in range(40):
        mon = rng.random() < 0.5
        H = rng.choice([64, 200, 256, 520, 768, 128, 384, 640])
        N = rng.choice([1500, 3000, 4096, 5000, 9000])
        V = rng.choice([2048, 3000, 4096, 5000, 8200])
        dt = rng.choice([torch.bfloat16, torch.float16])
        n_chunk = rng.choice([512, 1024, 2048])
        ign = rng.choice([0.0, 0.1, 0.5, 0.9])
        z_reg = rng.choice([0.0, 1e-4, 1e-2])
        scale = rng.choice([1.0, 0.5, 2.0])
        pack, layout = rng.choice([0, 1, 2]), rng.choice([0, 1])
        dw_dt = rng.choice([None, None, torch.float32])
        print(f"draw {it}: N={N} H={H} V={V} {dt} n_chunk={n_chunk} ignored={ign} z_reg={z_reg} scale={scale} pack={pack} "
              f"layout={layout} monitoring={mon} dW={dw_dt}", flush=True)
        try:
            inputs, a, b = _both_routes(N, H, V, dt, n_chunk, ign, z_reg, scale, pack, layout, dw_dt=dw_dt, mon=mon,
                                        seed=100 + it)
        except AssertionError as e:
            if "meant to take the one-pass route" not in str(e):
                raise
            continue  # (the bound of this draw leaves no room for the route)
        ran += 1
        several += b["chunks"] > 1
        _check(inputs, a, b, z_reg, scale, 1.0, fp64=N * V <= 4096 * 8192)
        if mon:
            assert a["out5"][2].item() == b["out5"][2].item()
            for i in (3, 4):
                assert abs(a["out5"][i].item() - b["out5"][i].item()) <= 5e-5 * abs(a["out5"][i].item()) + 1e-7, (i, a["out5"], b["out5"])
    assert ran >= 25 and several >= 20, (ran, several)


@pytest.mark.pack_auto
@pytest.mark.parametrize("layout", [0, 1])
def test_one_pass_is_deterministic_at_the_headline_shape(layout):
    """N=16384, H=2048, V=131072, bf16, four chunks on all compute units: three calls on a workspace that is overwritten
    in between give the same loss, lse, dx and dW bit for bit (the sums of dW over the chunks are added in chunk order,
    dx's K segments in segment order, and dW's upper halves are replaced in place by the results of the last chunk)."""
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    N, H, V, dt = 16384, 2048, 131072, torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(N, H, device="cuda", generator=g).to(dt)
    w = (torch.randn((V, H) if layout else (H, V), device="cuda", generator=g) / H ** 0.5).to(dt)
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    y[torch.rand(N, device="cuda", generator=g) < 0.05] = -1
    ldw = H if layout else V
    prob = _lib.make_problem(N, H, V, H, ldw, H, ldw, dt, dt, dt, dt, -1, 1.0, 1e-4, 4096, False, 0, 0, 0, layout,
                             _lib.ROUTE_ONE_PASS)
    chunks, rows = _lib.forward_backward_plan(prob)
    print(f"layout={layout}: {chunks} chunks of {rows} rows", flush=True)
    assert chunks >= 3
    ub = _lib.forward_backward_workspace_bytes(prob)
    ws = torch.empty(ub, dtype=torch.uint8, device="cuda")
    one = torch.ones(1, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    runs = []
    for fill in (0x00, 0x5a, 0xff):
        ws.fill_(fill)
        o = dict(lse=torch.empty(N, device="cuda"), out5=torch.empty(5, device="cuda"),
                 nv=torch.empty(1, dtype=torch.int64, device="cuda"), dx=torch.full((N, H), 3.0, dtype=dt, device="cuda"),
                 dw=torch.full(w.shape, float(fill), dtype=dt, device="cuda"))
        rc = lib.lce_forward_backward(ctypes.byref(prob), P(x), P(w), P(y), P(one), P(o["lse"]), P(o["out5"]), P(o["nv"]),
                                      P(o["dx"]), P(o["dw"]), P(ws), ub, st)
        assert rc == 0, (rc, lib.lce_last_hip_error())
        torch.cuda.synchronize()
        runs.append(o)
    assert torch.isfinite(runs[0]["dw"]).all() and torch.isfinite(runs[0]["dx"]).all()
    for o in runs[1:]:
        for k in o:
            assert torch.equal(o[k], runs[0][k]), k

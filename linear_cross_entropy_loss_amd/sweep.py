"""Sweep harness writing CSV files with the reference's schema.

The reference publishes its results as CSV files written by `bench_fusions.py`
(one per precision mode and swept variable, under `bench/`, `bench-mem/` and
`bench-acc/`): first column the swept variable, one column per provider.  This
module runs the same three protocols on one MI355X and writes files with the
same names, the same first column, the same units and the same FLOP convention
for the speed files (`3 * (2*N*H*V + 3*N*V)` for fwd+bwd, bench_fusions.py:287-291),
so that a curve from here can be laid over the reference's curve.

  speed   fwd+bwd TFLOP/s, median of event timings      bench_fusions.py:210-297
  mem     peak GiB beyond the inputs                    bench_fusions.py:304-394
  acc     torch.dist to an fp64 evaluation              bench_fusions.py:399-519

Providers: `torch-baseline` (eager `F.linear` + `F.cross_entropy` on the GPU, the
reference's first column, bench_fusions.py:31-33) and `hip-gfx950` (this
package).  A point a provider cannot run is left empty, as in the reference's
files.  Sweep ranges are the reference's: H 2^8..2^13, V 2^8..2^17, N 2^8..2^16
(bench_fusions.py:113; accuracy N up to 2^15, bench_fusions.py:446).

Usage:  python -m linear_cross_entropy_loss_amd.sweep --out DIR
            [--kind speed mem acc] [--acc bf16 fp16 fp16-mixed] [--vars N V H] [--quick]
        python -m linear_cross_entropy_loss_amd.sweep --out DIR --heads
            (not one of the reference's protocols: output layers of the sizes of public language models, bf16,
            time and peak memory of a fwd+bwd step beside eager, and the route the library takes; writes DIR/heads.txt)
        python -m linear_cross_entropy_loss_amd.sweep --out DIR --routes
            (lce_forward_backward at 25 shapes with the library's choice of route, with exact sums, forced onto one pass
            and onto two; writes DIR/routes.txt)
"""
from __future__ import annotations

import argparse
import math
import os
import sys

DEFAULTS = dict(N=16384, H=2048, V=131072)
RANGES = {"H": range(8, 14), "V": range(8, 18), "N": range(8, 17)}
ACC_RANGES = {"H": range(8, 14), "V": range(8, 18), "N": range(8, 16)}
PROVIDERS = ["torch-baseline", "hip-gfx950"]
TITLE_DEFAULTS = "Defaults: N=B*S=16384, H=2048, V=131072"
# The eager baseline materialises N x V fp32 logits and their gradient; skip it beyond this many elements.
BASELINE_MAX_LOGITS = 65536 * 131072


def _dtype(torch, acc):
    return {"fp16": torch.float16, "bf16": torch.bfloat16}.get(acc, torch.float32)


def _inputs(torch, N, H, V, acc, low_loss=False, seed=0):
    """Inputs of the reference's sweeps: A ~ randn(V, H), y uniform, x ~ randn (or 0.1*A[y] + randn for accuracy)."""
    dt = _dtype(torch, acc)
    g = torch.Generator(device="cuda").manual_seed(seed)
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    A = torch.randn(V, H, device="cuda", generator=g).to(dt)
    if low_loss:
        x = (0.1 * A[y].float() + torch.randn(N, H, device="cuda", generator=g)).to(dt)
    else:
        x = torch.randn(N, H, device="cuda", generator=g).to(dt)
    At = A.T.contiguous()
    return x.requires_grad_(), y, A.requires_grad_(), At.requires_grad_()


def _make_fn(torch, provider, x, y, A, At, acc):
    import torch.nn.functional as F

    mixed = "mixed" in acc
    amp_dtype = torch.bfloat16 if "bf16" in acc else torch.float16
    if provider == "torch-baseline":
        def loss_fn():
            return F.cross_entropy(F.linear(x, A).float(), y)
        grads = (x, A)
    else:
        from linear_cross_entropy_loss_amd import linear_cross_entropy

        def loss_fn():
            return linear_cross_entropy(x, y, At)[0]
        grads = (x, At)

    def step():
        for t in grads:
            t.grad = None
        with torch.autocast("cuda", dtype=amp_dtype, enabled=mixed):
            loss = loss_fn()
        loss.backward()
        return loss

    return step, grads


def _median_ms(torch, step, warmup, reps):
    cache = torch.empty(256 << 20, dtype=torch.int8, device="cuda")  # flushed before every repetition
    for _ in range(warmup):
        step()
    ts = []
    for _ in range(reps):
        cache.zero_()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        step()
        e.record()
        torch.cuda.synchronize()
        ts.append(s.elapsed_time(e))
    ts.sort()
    return ts[len(ts) // 2]


def _skip_baseline(provider, N, V):
    return provider == "torch-baseline" and N * V > BASELINE_MAX_LOGITS


def point_speed(torch, provider, N, H, V, acc, quick):
    if _skip_baseline(provider, N, V):
        return float("nan")
    x, y, A, At = _inputs(torch, N, H, V, acc)
    step, _ = _make_fn(torch, provider, x, y, A, At, acc)
    ms = _median_ms(torch, step, 2 if quick else 5, 5 if quick else 20)
    flop = 3 * (2 * N * H * V + 3 * N * V)
    return flop * 1e-12 / (ms * 1e-3)


def point_mem(torch, provider, N, H, V, acc, quick):
    if _skip_baseline(provider, N, V):
        return float("nan")
    x, y, A, At = _inputs(torch, N, H, V, acc)
    if provider == "torch-baseline":
        del At
        At = None
    else:
        A = A.detach()
    step, grads = _make_fn(torch, provider, x, y, A, At, acc)
    step()  # warm-up (allocator pools, lazy initialisation)
    for t in grads:
        t.grad = None
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    initial = torch.cuda.memory_allocated()
    step()
    torch.cuda.synchronize()
    return (torch.cuda.max_memory_allocated() - initial) / 1024**3


def _fp64_reference(torch, x, y, A, chunk=512):
    """Loss and gradients in fp64, row-chunked (the reference's torch_checkpoint in double, bench_fusions.py:408)."""
    import torch.nn.functional as F

    N = x.shape[0]
    Ad = A.detach().double().requires_grad_()
    dx = torch.empty(x.shape, dtype=torch.float64, device=x.device)
    loss = torch.zeros((), dtype=torch.float64, device=x.device)
    for i in range(0, N, chunk):
        xb = x[i:i + chunk].detach().double().requires_grad_()
        part = F.cross_entropy(F.linear(xb, Ad), y[i:i + chunk], reduction="sum") / N
        part.backward()
        dx[i:i + chunk] = xb.grad
        loss += part.detach()
    return loss.float(), Ad.grad.float(), dx.float()


def point_acc(torch, provider, N, H, V, acc, mode):
    if _skip_baseline(provider, N, V):
        return float("nan")
    x, y, A, At = _inputs(torch, N, H, V, acc, low_loss=True, seed=1)
    ref_loss, ref_dA, ref_dx = _fp64_reference(torch, x, y, A)
    step, grads = _make_fn(torch, provider, x, y, A, At, acc)
    loss = step()
    if mode == "fwd":
        return torch.dist(loss.float(), ref_loss).item()
    if provider == "torch-baseline":
        a_err = torch.dist(ref_dA, A.grad.float()).item()
    else:
        a_err = torch.dist(ref_dA.T, At.grad.float()).item()
    x_err = torch.dist(ref_dx, x.grad.float()).item()
    return 0.5 * (x_err + a_err)


def _write_csv(path, var, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write(",".join([var] + PROVIDERS) + "\n")
        for xval, vals in rows:
            cells = ["%f" % xval] + ["" if (v is None or math.isnan(v)) else "%f" % v for v in vals]
            f.write(",".join(cells) + "\n")


def run(out, kinds, accs, variables, quick=False, log=print):
    import torch

    if not torch.cuda.is_available():
        raise RuntimeError("the sweep needs an AMD GPU")
    written = []
    for kind in kinds:
        modes = ["fwd", "bwd"] if kind == "acc" else ["fwd-bwd"]
        for mode in modes:
            for acc in accs:
                if kind == "acc" and "mixed" in acc:
                    continue  # the reference's accuracy sweep covers fp16 and bf16 only (bench_fusions.py:448)
                for var in variables:
                    rng = (ACC_RANGES if kind == "acc" else RANGES)[var]
                    xs = [2**i for i in rng]
                    if quick:
                        xs = xs[::3]
                    rows = []
                    for xv in xs:
                        shape = dict(DEFAULTS)
                        shape[var] = xv
                        vals = []
                        for prov in PROVIDERS:
                            try:
                                torch.cuda.empty_cache()
                                if kind == "speed":
                                    v = point_speed(torch, prov, shape["N"], shape["H"], shape["V"], acc, quick)
                                elif kind == "mem":
                                    v = point_mem(torch, prov, shape["N"], shape["H"], shape["V"], acc, quick)
                                else:
                                    v = point_acc(torch, prov, shape["N"], shape["H"], shape["V"], acc, mode)
                            except (ValueError, RuntimeError, torch.OutOfMemoryError) as exc:
                                log(f"  {prov} N={shape['N']} H={shape['H']} V={shape['V']} {acc}: {type(exc).__name__}: "
                                    f"{str(exc).splitlines()[0][:120]}")
                                v = float("nan")
                            vals.append(v)
                        log(f"{kind} {mode} {acc} {var}={xv}: " + ", ".join(f"{p}={v:.4g}" for p, v in zip(PROVIDERS, vals)))
                        rows.append((float(xv), vals))
                    if kind == "speed":
                        name = f"bench/{acc} {mode}-Linear+Loss Performance over {var}. {TITLE_DEFAULTS}.csv"
                    elif kind == "mem":
                        name = f"bench-mem/{acc} {mode}-Linear+Loss Memory Peak over {var}. {TITLE_DEFAULTS}.csv"
                    else:
                        name = f"bench-acc/ {mode} {acc} Linear+Loss Accuracy over {var}. {TITLE_DEFAULTS}.csv"
                    path = os.path.join(out, name)
                    _write_csv(path, var, rows)
                    written.append(path)
    return written


# Output layers (hidden size, vocabulary) of the sizes of some public language models, with a token count per step.
HEADS = [
    ("gpt2-small", 8192, 768, 50257), ("gpt2-xl", 8192, 1600, 50257), ("llama-2-7b", 16384, 4096, 32000),
    ("mistral-7b", 16384, 4096, 32768), ("phi-3-mini", 8192, 3072, 32064), ("llama-3-8b", 16384, 4096, 128256),
    ("llama-3-70b", 8192, 8192, 128256), ("qwen-2.5-7b", 8192, 3584, 152064), ("gemma-2b", 8192, 2048, 256000),
    ("gemma-2-9b", 8192, 3584, 256000),
]


def run_heads(out, chunk_sizes=(4096, 8192), log=print):
    """fwd+bwd of each output layer in HEADS, bf16, 5 % of the labels ignored: this package at each N_chunk_size
    (route, ms, peak GiB beyond the inputs) beside eager F.linear + F.cross_entropy (bench_fusions.py:31-33)."""
    import torch
    import torch.nn.functional as F

    from . import _lib, linear_cross_entropy

    lines = [f"{'head':<13}{'N':>7}{'H':>6}{'V':>8} | {'eager ms':>9}{'GiB':>7} | "
             + " | ".join(f"{'N_chunk ' + str(c):>13}{'ms':>8}{'GiB':>7}{'x eager':>8}" for c in chunk_sizes)]
    for name, N, H, V in HEADS:
        torch.manual_seed(0)
        dt = torch.bfloat16
        x = torch.randn(N, H, device="cuda", dtype=dt).requires_grad_(True)
        w = (torch.randn(H, V, device="cuda") / math.sqrt(H)).to(dt).requires_grad_(True)
        y = torch.randint(0, V, (N,), device="cuda")
        y[torch.rand(N, device="cuda") < 0.05] = -100

        def measure(step):
            def run():
                x.grad = w.grad = None
                step()
            ms = _median_ms(torch, run, 3, 10)
            x.grad = w.grad = None
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            torch.cuda.reset_peak_memory_stats()
            initial = torch.cuda.memory_allocated()
            step()
            torch.cuda.synchronize()
            return ms, (torch.cuda.max_memory_allocated() - initial) / 1024**3

        try:
            e_ms, e_gib = measure(lambda: F.cross_entropy(F.linear(x, w.t()).float(), y).backward())
        except (RuntimeError, torch.OutOfMemoryError):
            e_ms = e_gib = float("nan")
        cells = []
        for c in chunk_sizes:
            ldw = V + (-V) % 8
            prob = _lib.make_problem(N, H, V, H, ldw, H, ldw, dt, dt, dt, dt, -100, 1.0, 0.0, c, False)
            chunks, rows = _lib.forward_backward_plan(prob)
            route = f"one, {chunks}x{rows}" if chunks else "two passes"
            ms, gib = measure(lambda: linear_cross_entropy(x, y, w, N_chunk_size=c)[0].backward())
            cells.append(f"{route:>13}{ms:>8.2f}{gib:>7.2f}{e_ms / ms:>8.2f}")
        lines.append(f"{name:<13}{N:>7}{H:>6}{V:>8} | {e_ms:>9.2f}{e_gib:>7.2f} | " + " | ".join(cells))
        log(lines[-1])
        del x, w, y
        torch.cuda.empty_cache()
    os.makedirs(out, exist_ok=True)
    path = os.path.join(out, "heads.txt")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")
    return path


# Shapes (N, H, V, N_chunk_size) on which the library's choice of route is timed against the alternatives.
ROUTE_SHAPES = [
    ("headline", 16384, 2048, 131072, 4096), ("config 3's", 16384, 4096, 131072, 4096),
    ("llama-3-8b", 16384, 4096, 128256, 4096), ("llama-2-7b", 16384, 4096, 32000, 4096),
    ("qwen-2.5-7b", 8192, 3584, 152064, 4096), ("phi-3-mini", 8192, 3072, 32064, 4096),
    ("config 4", 16384, 2048, 32768, 2048), ("config 4", 16384, 2048, 65536, 2048), ("config 4", 16384, 2048, 131072, 2048),
    ("config 4", 16384, 2048, 262144, 2048), ("config 4", 16384, 2048, 32768, 4096), ("config 4", 16384, 2048, 262144, 8192),
    ("H = 8192", 16384, 8192, 131072, 4096), ("H = 1024", 16384, 1024, 131072, 4096), ("H = 512", 16384, 512, 131072, 4096),
    ("H = 256", 16384, 256, 131072, 4096), ("V = 16384", 16384, 2048, 16384, 4096), ("V = 8192", 16384, 2048, 8192, 4096),
    ("V = 4096", 16384, 2048, 4096, 4096), ("N = 65536", 65536, 2048, 131072, 4096), ("N = 4096", 4096, 2048, 131072, 4096),
    ("N = 1024", 1024, 2048, 131072, 4096), ("small", 8192, 1024, 32768, 4096), ("small", 4096, 512, 4096, 1024),
    ("small", 2048, 2048, 16384, 4096),
]


def run_routes(out, log=print):
    """lce_forward_backward through the C ABI, bf16, 5 % of the labels ignored, at each shape of ROUTE_SHAPES with
    lce_problem.route = LCE_ROUTE_AUTO (the library's choice), the same with LCE_ROUTE_EXACT_SUMS, LCE_ROUTE_ONE_PASS and
    LCE_ROUTE_TWO_PASS: (chunks, rows per chunk) of the plan -- (0, 0) = two passes -- and ms per call."""
    import ctypes
    import time

    import torch

    from . import _lib

    lib = _lib.load()
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    dt = torch.bfloat16
    routes = (("library", _lib.ROUTE_AUTO), ("exact sums", _lib.ROUTE_AUTO | _lib.ROUTE_EXACT_SUMS),
              ("one pass", _lib.ROUTE_ONE_PASS), ("two passes", _lib.ROUTE_TWO_PASS))
    lines = [f"{'shape':<12}{'N':>7}{'H':>6}{'V':>8}{'N_chunk':>8} | "
             + " | ".join(f"{name:>12}{'ms':>9}" for name, _ in routes) + " | library / fastest"]
    for name, N, H, V, n_chunk in ROUTE_SHAPES:
        g = torch.Generator(device="cuda").manual_seed(1)
        x = torch.randn(N, H, device="cuda", generator=g).to(dt)
        w = (torch.randn(H, V, device="cuda", generator=g) / math.sqrt(H)).to(dt)
        y = torch.randint(0, V, (N,), device="cuda", generator=g)
        y[torch.rand(N, device="cuda", generator=g) < 0.05] = -1
        lse, out5 = torch.empty(N, device="cuda"), torch.empty(5, device="cuda")
        nv = torch.empty(1, dtype=torch.int64, device="cuda")
        dx, dw = torch.empty(N, H, dtype=dt, device="cuda"), torch.empty(H, V, dtype=dt, device="cuda")
        one = torch.ones(1, device="cuda")
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        cells, times = [], []
        for _, route in routes:
            prob = _lib.make_problem(N, H, V, H, V, H, V, dt, dt, dt, dt, -1, 1.0, 0.0, n_chunk, False, route=route)
            plan = _lib.forward_backward_plan(prob)
            nbytes = _lib.forward_backward_workspace_bytes(prob)
            ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")

            def call():
                rc = lib.lce_forward_backward(ctypes.byref(prob), ptr(x), ptr(w), ptr(y), ptr(one), ptr(lse), ptr(out5), ptr(nv),
                                              ptr(dx), ptr(dw), ptr(ws), nbytes, stream)
                _lib.raise_for_status(rc, "lce_forward_backward")

            for _ in range(3):
                call()
            torch.cuda.synchronize()
            reps = 10 if N * H * V < 3e13 else 4
            t0 = time.perf_counter()
            for _ in range(reps):
                call()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) / reps * 1e3
            times.append(ms)
            cells.append(f"{str(plan):>12}{ms:>9.3f}")
            del ws
        lines.append(f"{name:<12}{N:>7}{H:>6}{V:>8}{n_chunk:>8} | " + " | ".join(cells) + f" | {times[0] / min(times):.3f}")
        log(lines[-1])
        del x, w, dx, dw
        torch.cuda.empty_cache()
    os.makedirs(out, exist_ok=True)
    path = os.path.join(out, "routes.txt")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")
    return path


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--out", required=True)
    ap.add_argument("--kind", nargs="+", default=["speed", "mem", "acc"], choices=["speed", "mem", "acc"])
    ap.add_argument("--acc", nargs="+", default=["fp16", "bf16", "fp16-mixed"], choices=["fp16", "bf16", "fp16-mixed"])
    ap.add_argument("--vars", nargs="+", default=["H", "N", "V"], choices=["H", "N", "V"])
    ap.add_argument("--quick", action="store_true", help="every third point, fewer repetitions")
    ap.add_argument("--heads", action="store_true", help="output layers of the sizes of public language models instead")
    ap.add_argument("--routes", action="store_true", help="the library's choice of route against the alternatives instead")
    args = ap.parse_args(argv)
    if args.routes:
        print("wrote", run_routes(args.out, log=lambda m: print(m, flush=True)), flush=True)
        return 0
    if args.heads:
        print("wrote", run_heads(args.out, log=lambda m: print(m, flush=True)), flush=True)
        return 0
    for p in run(args.out, args.kind, args.acc, args.vars, args.quick, log=lambda m: print(m, flush=True)):
        print("wrote", p, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

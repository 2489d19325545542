#!/usr/bin/env python3
"""Benchmark of the fused linear + cross-entropy operator on one MI355X.

One step = one forward + backward (dx and dW) of the operator over one batch of synthetic input already
resident in HBM.  Prints ONE JSON line.  Default workload: N = B*S = 16384, H = 2048, V = 131072 in bf16,
5 % of the labels ignored, N_chunk_size = 4096.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published dense peaks used as roofline denominators.  fp32 tensors are computed as bf16 pairs, three
# bf16 MFMA products per fp32 product, so the bound of that path in fp32-equivalent FLOPs is a third of the bf16 peak.
PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 2500.0 / 3.0}
# The reference's own published fwd+bwd figure for this shape in bf16 (unnamed 48 GB NVIDIA GPU),
# 86.75 TFLOP/s on its 6*N*H*V convention = 304.4 ms = 115.6 TFLOP/s on the 8*N*H*V convention used here.
REFERENCE_PUBLISHED_TFLOPS_8NHV = 115.6

WORKLOADS = {
    "c2_bf16_N16384_H2048_V131072": dict(N=16384, H=2048, V=131072, dtype="bf16", ignore=0.05, n_chunk=4096,
                                          z_reg=0.0, scale=1.0, monitoring=False, seed=2),
    # the headline shape with the weight stored (V, H) -- a tied embedding handed over as weight.T, read in place
    "c2_bf16_N16384_H2048_V131072_weight_VH": dict(N=16384, H=2048, V=131072, dtype="bf16", ignore=0.05, n_chunk=4096,
                                                    z_reg=0.0, scale=1.0, monitoring=False, seed=2, w_vh=True),
    # the small fp32 case (fp32 tensors, computed as bf16 pairs)
    "c1_f32_N2048_H2048_V16384": dict(N=2048, H=2048, V=16384, dtype="f32", ignore=0.0, n_chunk=4096,
                                       z_reg=0.0, scale=1.0, monitoring=False, seed=1),
    # fp16 with every loss feature on, Zipf(1.1) labels, 10 % ignored
    "c3_f16_N16384_H4096_V131072_all_features": dict(N=16384, H=4096, V=131072, dtype="f16", ignore=0.10, n_chunk=4096,
                                                      z_reg=1e-4, scale=0.5, monitoring=True, seed=3, zipf=True),
    # long sequence, fp16 activations, fp32 master weight (fp32 dW), Zipf(1.1) labels, 10 % ignored
    "c5_f16_w32_N65536_H8192_V262144": dict(N=65536, H=8192, V=262144, dtype="f16", w_dtype="f32", ignore=0.10,
                                             n_chunk=8192, z_reg=0.0, scale=1.0, monitoring=False, seed=5, zipf=True),
}


def make_gpu_inputs(cfg, torch):
    dt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[cfg["dtype"]]
    g = torch.Generator(device="cuda").manual_seed(cfg["seed"])
    N, H, V = cfg["N"], cfg["H"], cfg["V"]
    x = torch.randn(N, H, device="cuda", generator=g, dtype=torch.float32).to(dt)
    std = 1.0 / math.sqrt(H)
    w = torch.empty(H, V, device="cuda", dtype=torch.float32)
    torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-3 * std, b=3 * std, generator=g)
    if cfg.get("w_dtype") != "f32":
        w = w.to(dt)
    if cfg.get("zipf"):
        p = torch.arange(1, V + 1, dtype=torch.float64, device="cuda") ** -1.1
        cdf = torch.cumsum(p, 0) / p.sum()
        u = torch.rand(N, device="cuda", generator=g, dtype=torch.float64)
        y = torch.searchsorted(cdf, u).clamp_(max=V - 1)
    else:
        y = torch.randint(0, V, (N,), device="cuda", generator=g)
    if cfg["ignore"] > 0:
        y[torch.rand(N, device="cuda", generator=g) < cfg["ignore"]] = -1
    if cfg.get("w_vh"):
        w = w.t().contiguous().t()  # shape (H, V), stored (V, H) row-major
    return x, y, w


def time_phases_one_pass(cfg, x, y, w, prob, chunks, torch, reps):
    """time_phases for lce_forward_backward's single pass over the logits (`w`: the rows the kernels read)."""
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    N, H, V = cfg["N"], cfg["H"], cfg["V"]
    dev = x.device
    ws = torch.empty(_lib.forward_backward_workspace_bytes(prob(0)), dtype=torch.uint8, device=dev)
    lse = torch.empty(N, dtype=torch.float32, device=dev)
    out5 = torch.empty(5, dtype=torch.float32, device=dev)
    nv = torch.empty(1, dtype=torch.int64, device=dev)
    g = torch.ones(1, dtype=torch.float32, device=dev)
    dx = torch.empty_like(x)
    dw = torch.empty_like(w)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def call(ph):
        p = prob(ph)
        rc = lib.lce_forward_backward(ctypes.byref(p), P(x), P(w), P(y), P(g), P(lse), P(out5), P(nv), P(dx), P(dw),
                                      P(ws), ws.numel(), stream)
        _lib.raise_for_status(rc, "lce_forward_backward")

    call(0)
    torch.cuda.synchronize()
    rows = int(nv.item()) if 8.0 * N * H * V >= 2.0 ** 41 else N
    out = {}
    for name, ph, flops, nbytes in (
        ("fwd_stage", _lib.PHASE_FWD_TILES, 2.0 * (N if cfg["monitoring"] else rows) * H * V / chunks, 0.0),
        # 2 bytes read and 2 written per logit: bound by memory traffic, not by matrix instructions
        ("stage_scale", _lib.PHASE_BWD_DZ, 0.0, 4.0 * rows * V / chunks),
        ("bwd_dx", _lib.PHASE_BWD_DX, 2.0 * rows * H * V / chunks, 0.0),
        # (with more than one chunk: the tile kernel adds into the fp32 sums of dW that are kept over the chunks; the last chunk's launch stores dW)
        ("bwd_dw", _lib.PHASE_BWD_DW, 2.0 * rows * H * V / chunks, 0.0),
        ("pack", _lib.PHASE_PACK, 0.0, 0.0),
    ):
        call(ph)
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            call(ph)
        e.record()
        torch.cuda.synchronize()
        launches = 1 if name == "pack" else chunks
        per_launch_ms = s.elapsed_time(e) / reps / launches
        out[name] = dict(ms_per_launch=per_launch_ms, launches_per_step=launches, flops_per_launch=flops,
                         tflops=flops / per_launch_ms / 1e9)
        if nbytes:
            out[name].update(bytes_per_launch=nbytes, gb_per_s=nbytes / per_launch_ms / 1e6)
    return out


def time_phases(cfg, x, y, w, torch, reps=5, one_pass=True):
    """Average duration (ms) of each heavy kernel, bracketed by events on the launch stream, through the C ABI."""
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    N, H, V = cfg["N"], cfg["H"], cfg["V"]
    dev = x.device

    vh = bool(cfg.get("w_vh"))
    w = w.t() if vh else w  # the rows the kernels read
    ldw = w.stride(0)

    def prob(phases):
        return _lib.make_problem(N, H, V, x.stride(0), ldw, H, ldw, x.dtype, w.dtype, x.dtype, w.dtype,
                                 -1, cfg["scale"], cfg["z_reg"], cfg["n_chunk"], cfg["monitoring"], phases, 0, 0,
                                 _lib.W_VH if vh else _lib.W_HV)

    chunks, _ = _lib.forward_backward_plan(prob(0))
    if chunks > 0 and one_pass:
        return time_phases_one_pass(cfg, x, y, w, prob, chunks, torch, reps)
    fwd_b, bwd_b = _lib.workspace_bytes(prob(0))
    # one workspace per call: a call restricted to one kernel relies on what the full call left in it
    ws_f = torch.empty(fwd_b, dtype=torch.uint8, device=dev)
    ws_b = torch.empty(bwd_b, dtype=torch.uint8, device=dev)
    lse = torch.empty(N, dtype=torch.float32, device=dev)
    out5 = torch.empty(5, dtype=torch.float32, device=dev)
    nv = torch.empty(1, dtype=torch.int64, device=dev)
    g = torch.ones(1, dtype=torch.float32, device=dev)
    dx = torch.empty_like(x)
    dw = torch.empty_like(w)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def fwd(ph):
        p = prob(ph)
        rc = lib.lce_forward(ctypes.byref(p), P(x), P(w), P(y), P(lse), P(out5), P(nv), P(ws_f), ws_f.numel(), stream)
        _lib.raise_for_status(rc, "lce_forward")

    def bwd(ph):
        p = prob(ph)
        rc = lib.lce_backward(ctypes.byref(p), P(x), P(w), P(y), P(lse), P(nv), P(g), P(dx), P(dw), P(ws_b),
                              ws_b.numel(), stream)
        _lib.raise_for_status(rc, "lce_backward")

    fwd(0)
    bwd(0)
    torch.cuda.synchronize()
    # tokens with an ignored label are dropped before the tile kernels (from 8*N*H*V = 2^41 FLOPs on, the
    # library's default rule): FLOPs are counted on the others only
    rows = int(nv.item()) if 8.0 * N * H * V >= 2.0 ** 41 else N
    # launches per call: the backward runs once per vocabulary slab
    slabs, _ = _lib.backward_plan(prob(0))
    out = {}
    for name, fn, ph, launches, flops in (
        ("fwd_tiles", fwd, _lib.PHASE_FWD_TILES, 1, 2.0 * (N if cfg["monitoring"] else rows) * H * V),
        ("bwd_dz", bwd, _lib.PHASE_BWD_DZ, slabs, 2.0 * rows * H * V / slabs),
        ("bwd_dx", bwd, _lib.PHASE_BWD_DX, slabs, 2.0 * rows * H * V / slabs),
        ("bwd_dw", bwd, _lib.PHASE_BWD_DW, slabs, 2.0 * rows * H * V / slabs),
        # the packing pre-pass of the backward (labels, packed x and lse); the forward runs the same without lse
        ("bwd_pack", bwd, _lib.PHASE_PACK, 1, 0.0),
    ):
        fn(ph)
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            fn(ph)
        e.record()
        torch.cuda.synchronize()
        per_launch_ms = s.elapsed_time(e) / reps / launches
        out[name] = dict(ms_per_launch=per_launch_ms, launches_per_step=launches, flops_per_launch=flops,
                         tflops=flops / per_launch_ms / 1e9)
    return out


def median_step_ms(step, torch, reps=20, flush=False):
    """Median of per-step event timings; with `flush`, a 256 MiB buffer is zeroed before every step so that
    no operand starts in L2 / Infinity Cache (the protocol of triton.testing.do_bench, which the reference's
    bench_fusions.py:280-281 uses)."""
    cache = torch.empty(256 << 20, dtype=torch.int8, device="cuda") if flush else None
    ts = []
    for _ in range(reps):
        if flush:
            cache.zero_()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        step()
        e.record()
        torch.cuda.synchronize()
        ts.append(s.elapsed_time(e))
    ts.sort()
    return 0.5 * (ts[(reps - 1) // 2] + ts[reps // 2])


def host_cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(cfg, torch, chunk=2048, budget_s=75.0):
    """Eager fp32 linear + F.cross_entropy fwd+bwd on all host cores over the WHOLE workload, as an N-chunked eager
    loop: `chunk` rows at a time (the N x V fp32 logits and their gradient, 16 GiB at the default shape, never exist
    at once), every chunk's gradients accumulated -- the same mathematics as one unchunked step.

    Inputs by the workload's own recipe (x ~ N(0,1), W truncated normal with std 1/sqrt(H), the workload's labels and
    ignored fraction) in fp32; a warm-up over one chunk, then up to three timed steps (median), fewer when a step
    takes so long that three would exceed `budget_s` seconds; a workload whose single step would exceed it (config
    5: about 600 s) is timed on its first chunks only and says so.
    """
    from oracle import eager_fp32_step_chunked

    N, H, V = cfg["N"], cfg["H"], cfg["V"]
    # all host cores of this job: the box's share (OMP_NUM_THREADS there) where that is smaller than what the OS shows
    torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS") or (os.cpu_count() or 1))))
    g = torch.Generator().manual_seed(cfg["seed"])
    std = 1.0 / math.sqrt(H)
    w = torch.empty(H, V)
    torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-3 * std, b=3 * std, generator=g)
    threads = torch.get_num_threads()

    def inputs(n):
        x = torch.randn(n, H, generator=g)
        if cfg.get("zipf"):
            p = torch.arange(1, V + 1, dtype=torch.float64) ** -1.1
            y = torch.searchsorted(torch.cumsum(p, 0) / p.sum(), torch.rand(n, generator=g, dtype=torch.float64)).clamp_(max=V - 1)
        else:
            y = torch.randint(0, V, (n,), generator=g)
        if cfg["ignore"] > 0:
            y[torch.rand(n, generator=g) < cfg["ignore"]] = -1
        return x, y

    def timed(x, y):
        t0 = time.perf_counter()
        eager_fp32_step_chunked(x, y, w, -1, cfg["z_reg"], cfg["scale"], chunk=chunk)
        return time.perf_counter() - t0

    xw, yw = inputs(min(N, chunk))
    t_chunk = timed(xw, yw)  # warm-up (one chunk), also the estimate of a step
    est = t_chunk * math.ceil(N / chunk)
    if est <= budget_s:
        Ns = N
        x, y = inputs(N)
        reps = max(1, min(3, int(budget_s / est)))
    else:  # bounded sample: as many whole chunks as fit about a third of the budget
        Ns = min(N, chunk * max(1, int(budget_s / 3 / t_chunk)))
        x, y = inputs(Ns)
        reps = 1
    ts = sorted(timed(x, y) for _ in range(reps))
    t = ts[(reps - 1) // 2]
    whole = Ns == N
    return dict(value=8.0 * Ns * H * V / t / 1e12, unit="TFLOP/s",
                cores=threads, kind="port", host_cpu=host_cpu_model(), os_cpu_count=os.cpu_count(),
                torch_num_threads=threads,
                sample=(f"the whole workload: all {N} tokens at H={H}, V={V} in {math.ceil(N / chunk)} chunks of {chunk} rows"
                        if whole else
                        f"the first {Ns} of {N} tokens at full H={H}, V={V} in chunks of {chunk} rows (one step of the "
                        f"whole workload would take about {est:.0f} s)") +
                       f", inputs by the workload's recipe; eager fp32 matmul + F.cross_entropy fwd+bwd with gradients "
                       f"accumulated over the chunks; warm-up over one chunk, {reps} timed step(s), median; "
                       f"8*N*H*V FLOP convention",
                ms_per_step=t * 1e3 * (N / Ns), ms_per_step_is_measured=whole, timed_steps=reps,
                tokens_timed=Ns)


def sources_sha16():
    """Hash of the operator's kernel sources: profiles/hbm_traffic.json carries the one its counters were collected on."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "linear_cross_entropy_loss_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


C4_POINTS = [(V, nc) for V in (32768, 65536, 131072, 262144) for nc in (2048, 4096, 8192)]


def c4_sweep(args, torch):
    """Vocabulary sweep in bf16 at N=16384, H=2048 (no ignored labels): time and peak memory at each of the
    12 (V, N_chunk_size) points, as the reference's bench_fusions.py:304-315 measures them."""
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    N, H = 16384, 2048
    points = []
    cur = {}
    for V, nc in C4_POINTS:
        if cur.get("V") != V:
            cur.clear()
            torch.cuda.empty_cache()
            x, y, w = make_gpu_inputs(dict(N=N, H=H, V=V, dtype="bf16", ignore=0.0, seed=4), torch)
            cur.update(V=V, x=x.requires_grad_(True), y=y, w=w.requires_grad_(True))
        x, y, w = cur["x"], cur["y"], cur["w"]

        def step():
            x.grad = None
            w.grad = None
            out = linear_cross_entropy(x, y, w, -1, 0.0, 1.0, nc, False)
            out[0].backward()
            return out[0]

        for _ in range(3):
            loss = step()
        x.grad = None
        w.grad = None
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        loss = step()
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() - base
        grads = x.numel() * x.element_size() + w.numel() * w.element_size()
        ms = median_step_ms(step, torch, reps=max(5, args.steps // 10), flush=False)
        from linear_cross_entropy_loss_amd import _lib, ops

        plan = (0, 0)
        if ops.one_pass.get():
            plan = _lib.forward_backward_plan(_lib.make_problem(N, H, V, H, V, H, V, x.dtype, w.dtype, x.dtype, w.dtype, -1,
                                                                1.0, 0.0, nc, False))
        points.append(dict(V=V, N_chunk_size=nc, ms=ms, route="one_pass" if plan[0] else "two_pass",
                           chunks=plan[0], chunk_rows=plan[1], tflops_8NHV=8.0 * N * H * V / ms / 1e9,
                           pct_mfma_peak=100.0 * 8.0 * N * H * V / ms / 1e9 / PEAK_TFLOPS["bf16"],
                           peak_hbm_bytes_incl_grads=int(peak), peak_hbm_bytes_extra=int(peak - grads),
                           scratch_budget_bytes=int(nc * V * 4), within_budget=bool(peak - grads <= nc * V * 4),
                           loss=float(loss.item())))
    total_flops = sum(8.0 * N * H * p["V"] for p in points)
    total_ms = sum(p["ms"] for p in points)
    return {
        "metric": "fwd+bwd TFLOP/s (8*N*H*V) over the 12 points of the vocabulary sweep, N=16384, H=2048, bf16",
        "value": total_flops / total_ms / 1e9, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": total_ms / len(points), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "c4_sweep_bf16_N16384_H2048", "N": N, "H": H,
                   "V": sorted({p["V"] for p in points}), "N_chunk_size": sorted({p["N_chunk_size"] for p in points}),
                   "ignored_label_frac": 0.0},
        "points": points,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2_bf16_N16384_H2048_V131072", choices=sorted(WORKLOADS) + ["c4_sweep"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--two-pass", action="store_true",
                    help="loss-only forward and a backward that recomputes the logit tiles (lce_forward, lce_backward: "
                         "8*H*V FLOPs per token), instead of the default, gradients from the forward's one evaluation of "
                         "the logits where the problem allows it (lce_forward_backward: 6*H*V)")
    ap.add_argument("--library", metavar="SO",
                    help="load this build of liblce_gfx950.so instead of the one in the package (to time two builds "
                         "on the same box)")
    ap.add_argument("--probe", choices=["ceiling", "flush", "overlap"],
                    help="run a measurement probe instead of the benchmark and print its JSON (built on demand, "
                         "linear_cross_entropy_loss_amd/probes): 'ceiling' (register-only MFMA loop, vendor GEMM, half of "
                         "the compute units), 'flush' (partial-sum blocks into memory), 'overlap' (epilogue arithmetic "
                         "behind matrix instructions)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one 1 GiB device-to-device copy (a kernel of known traffic, to scale "
                         "FETCH_SIZE / WRITE_SIZE counters collected with rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this operator is a single-GPU kernel path and this build measures one GPU only; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an AMD GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(1)
    from linear_cross_entropy_loss_amd import _lib, linear_cross_entropy, ops

    if args.two_pass:
        ops.one_pass.set(False)
    if args.library:
        from pathlib import Path

        _lib.LIB_PATH = Path(args.library).resolve()
    if not _lib.LIB_PATH.exists():  # normally built beforehand and shipped with the tree
        from linear_cross_entropy_loss_amd.build import build

        build(force=True)

    if args.probe:
        from linear_cross_entropy_loss_amd import probes

        print(json.dumps(probes.run(args.probe, torch)))
        return
    if args.workload == "c4_sweep":
        print(json.dumps(c4_sweep(args, torch)))
        return
    cfg = WORKLOADS[args.workload]
    N, H, V = cfg["N"], cfg["H"], cfg["V"]
    x, y, w = make_gpu_inputs(cfg, torch)
    x.requires_grad_(True)
    w.requires_grad_(True)

    def step():
        x.grad = None
        w.grad = None
        out = linear_cross_entropy(x, y, w, -1, cfg["z_reg"], cfg["scale"], cfg["n_chunk"], cfg["monitoring"])
        out[0].backward()
        return out[0]

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        loss = step()
    torch.cuda.synchronize()
    x.grad = None
    w.grad = None
    torch.cuda.reset_peak_memory_stats()
    base_mem = torch.cuda.memory_allocated()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms = elapsed * 1e3 / args.steps
    peak_bytes = torch.cuda.max_memory_allocated() - base_mem
    out_bytes = x.numel() * x.element_size() + w.numel() * w.element_size()
    # Tokens whose label is ignored are dropped before the tile kernels (their rows of the four GEMMs are
    # not computed), so the rate counts the computed rows only; with monitoring on the forward keeps all rows.
    rows = int((y != -1).sum().item()) if 8.0 * N * H * V >= 2.0 ** 41 else N
    flops = (2.0 * (N if cfg["monitoring"] else rows) + 6.0 * rows) * H * V
    tflops = flops / ms / 1e9
    peak = PEAK_TFLOPS[cfg["dtype"]]
    # which route the steps above took (ops.LinearXentImplementation.forward decides the same way)
    route = "two_pass"
    if not args.two_pass and cfg["dtype"] != "f32":
        wr = w.detach().t() if cfg.get("w_vh") else w.detach()
        pr = _lib.make_problem(N, H, V, x.stride(0), wr.stride(0), H, wr.stride(0), x.dtype, wr.dtype, x.dtype, wr.dtype, -1,
                               cfg["scale"], cfg["z_reg"], cfg["n_chunk"], cfg["monitoring"], 0, 0, 0,
                               _lib.W_VH if cfg.get("w_vh") else _lib.W_HV)
        if _lib.forward_backward_plan(pr)[0] > 0:
            route = "one_pass"
    flops_executed = flops if route == "two_pass" else (2.0 * (N if cfg["monitoring"] else rows) + 4.0 * rows) * H * V

    ms_median = median_step_ms(step, torch, reps=20, flush=False)
    ms_median_flushed = median_step_ms(step, torch, reps=20, flush=True)
    x.grad = None
    w.grad = None

    phases = time_phases(cfg, x.detach(), y, w.detach(), torch, one_pass=route == "one_pass")
    dom = max(phases, key=lambda k: phases[k]["ms_per_launch"] * phases[k]["launches_per_step"])
    d = phases[dom]
    roofline = dict(bound="mfma", kernel=dom, achieved=d["tflops"], peak=peak, unit="TFLOP/s",
                    frac=d["tflops"] / peak, traffic=None, ms_per_launch=d["ms_per_launch"],
                    flops_per_launch=d["flops_per_launch"])
    traffic_file = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(traffic_file):
        with open(traffic_file) as f:
            tr = json.load(f)
        # counters collected on other kernel sources say nothing about this build
        if tr.get("sources_sha16") == sources_sha16():
            roofline["traffic"] = tr.get(args.workload, {}).get(route, {}).get(dom)
            roofline["traffic_note"] = tr.get("note")
        else:
            roofline["traffic_note"] = "profiles/hbm_traffic.json was collected on other kernel sources: dropped"

    line = {
        "metric": "fwd+bwd TFLOP/s (8*H*V FLOPs per token computed) at N=16384,H=2048,V=131072 bf16"
        if args.workload.startswith("c2") else f"fwd+bwd TFLOP/s (8*H*V FLOPs per token computed) {args.workload}",
        "value": tflops,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "ms_per_step_median_events": ms_median,
        "ms_per_step_median_events_cache_flushed": ms_median_flushed,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": tflops / REFERENCE_PUBLISHED_TFLOPS_8NHV if args.workload.startswith("c2") else None,
        "baseline_note": "reference's published bf16 fwd+bwd at this shape on an unnamed 48 GB NVIDIA GPU: "
                         "304.4 ms = 115.6 TFLOP/s on the 8NHV convention",
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "flops_note": "value is on the metric's convention, 8*H*V FLOPs per token (logits, logits again, dx, dW), times the "
                      "tokens computed: tokens with an ignored label are dropped before the tile kernels.  On the "
                      "one_pass route the logits are evaluated once and 6*H*V FLOPs per token are executed "
                      "(tflops_executed, pct_mfma_peak_executed); on the two_pass route value is what is executed",
        "route": route,
        "tflops_executed": flops_executed / ms / 1e9,
        "pct_mfma_peak_executed": 100.0 * flops_executed / ms / 1e9 / peak,
        "tokens_computed": rows,
        "tflops_8NHV_convention": 8.0 * N * H * V / ms / 1e9,
        "pct_mfma_peak_8NHV_convention": 100.0 * 8.0 * N * H * V / ms / 1e9 / PEAK_TFLOPS[cfg["dtype"]],
        "config": {"workload": args.workload, "N": N, "H": H, "V": V, "ignored_label_frac": cfg["ignore"],
                   "N_chunk_size": cfg["n_chunk"], "z_regularization": cfg["z_reg"], "logit_scale": cfg["scale"],
                   "outputs": "loss, dx, dW"},
        "pct_mfma_peak": 100.0 * tflops / peak,
        "mfma_peak_tflops_used": peak,
        "loss": float(loss.item()),
        "loss_expected_approx": math.log(V) + 0.5 * cfg["scale"] ** 2,
        "peak_hbm_bytes_incl_grads": int(peak_bytes),
        "peak_hbm_bytes_extra": int(peak_bytes - out_bytes),
        "scratch_budget_bytes": int(cfg["n_chunk"] * V * 4),
        # device memory the library's code object holds on every GPU it runs on, outside the allocator's statistics:
        # the fixed scratch array of lce_forward_static (not used by this benchmark)
        "static_scratch_bytes_per_gpu": int(_lib.STATIC_SCRATCH_BYTES),
        "kernels": phases,
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(cfg, torch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()

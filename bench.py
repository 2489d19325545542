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


def time_phases(cfg, x, y, w, torch, reps=5):
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


def cpu_baseline(cfg, torch, rows=2048):
    """Eager fp32 linear + F.cross_entropy fwd+bwd on all host cores, on a bounded row sample of the same workload.

    Inputs by the workload's own recipe (x ~ N(0,1), W truncated normal with std 1/sqrt(H), the workload's labels
    and ignored fraction) upcast to fp32; 1 warm-up + 3 timed steps, median.  The whole workload would need the
    N x V fp32 logits and their gradient on the host (16 GiB at the default shape), so the first `rows` tokens
    are timed at full H and V and the rate is what is reported: the cost per token does not depend on N.
    """
    from oracle import eager_fp32_step

    H, V = cfg["H"], cfg["V"]
    Ns = min(cfg["N"], rows)
    # all host cores of this job: the box's share (OMP_NUM_THREADS there) where that is smaller than what the OS shows
    torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS") or (os.cpu_count() or 1))))
    g = torch.Generator().manual_seed(cfg["seed"])
    x = torch.randn(Ns, H, generator=g)
    std = 1.0 / math.sqrt(H)
    w = torch.empty(H, V)
    torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-3 * std, b=3 * std, generator=g)
    if cfg.get("zipf"):
        p = torch.arange(1, V + 1, dtype=torch.float64) ** -1.1
        y = torch.searchsorted(torch.cumsum(p, 0) / p.sum(), torch.rand(Ns, generator=g, dtype=torch.float64)).clamp_(max=V - 1)
    else:
        y = torch.randint(0, V, (Ns,), generator=g)
    if cfg["ignore"] > 0:
        y[torch.rand(Ns, generator=g) < cfg["ignore"]] = -1
    threads = torch.get_num_threads()
    eager_fp32_step(x, y, w, -1, cfg["z_reg"], cfg["scale"])  # warm-up
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        eager_fp32_step(x, y, w, -1, cfg["z_reg"], cfg["scale"])
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[1]
    return dict(value=8.0 * Ns * H * V / t / 1e12, unit=f"TFLOP/s (8*N*H*V convention, on a {Ns}-token sample)",
                cores=threads, kind="port", host_cpu=host_cpu_model(), os_cpu_count=os.cpu_count(),
                torch_num_threads=threads,
                sample=f"first {Ns} of {cfg['N']} tokens at full H={H}, V={V}, inputs by the workload's recipe; eager "
                       f"fp32 matmul + F.cross_entropy fwd+bwd; 1 warm-up + 3 timed, median; {t * 1e3:.0f} ms per "
                       f"sample step",
                ms_per_sample_step=t * 1e3)


def sources_sha16():
    """Hash of the operator's kernel sources (the measurement probes are a library of their own and do not count):
    profiles/hbm_traffic.json carries the one its counters were collected on."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "linear_cross_entropy_loss_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")) and name != "lce_probe.hip":
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
        points.append(dict(V=V, N_chunk_size=nc, ms=ms, tflops_8NHV=8.0 * N * H * V / ms / 1e9,
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


def _events_ms(fn, torch, reps):
    fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(reps):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / reps


def _load_probe_lib():
    from linear_cross_entropy_loss_amd.build import PROBE_LIB_PATH

    if not PROBE_LIB_PATH.exists():
        raise RuntimeError(f"{PROBE_LIB_PATH} is missing: run `python -m linear_cross_entropy_loss_amd.build`")
    lib = ctypes.CDLL(str(PROBE_LIB_PATH))
    vp = ctypes.c_void_p
    lib.lce_probe_mfma.restype = ctypes.c_int
    lib.lce_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
    lib.lce_probe_mfma_loads.restype = ctypes.c_int
    lib.lce_probe_mfma_loads.argtypes = [ctypes.c_int, ctypes.c_int, vp, ctypes.c_uint64, ctypes.c_int, ctypes.c_int, vp, vp]
    lib.lce_probe_flush.restype = ctypes.c_int
    lib.lce_probe_flush.argtypes = [ctypes.c_int, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, vp]
    return lib


def probe_ceiling(torch):
    """What bounds the tile kernels on this part: (1) a register-only loop of the same MFMA instruction over
    the same 128 x 128 wave tile, on constant and on random operands, with the tile kernels' LDS reads and
    writes added, with their operand loads from L2 added as well, with their one barrier per K tile, and with a
    quarter of the loads missing L2 (still no epilogues), on all and on half of the compute units;
    (2) the vendor GEMM (torch.matmul -> hipBLASLt) on the four contractions of the default workload; (3) the
    operator's forward tile kernel on all and on half of the compute units (a chip-level power limit shows as a
    higher rate per compute unit when fewer of them run)."""
    from linear_cross_entropy_loss_amd import _lib

    probe = _load_probe_lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = {"probe": "ceiling", "compute_units": cus, "peak_bf16_tflops_published": PEAK_TFLOPS["bf16"], "mfma_loop": [],
           "vendor_gemm": [], "fwd_tiles": []}
    buf = torch.empty(cus * 256 * 4, dtype=torch.float32, device="cuda")
    iters = 200000
    # operand windows of the loads patterns: 2 MiB of random bf16 in [-2, 2) each.  One window walked by all workgroups
    # stays in every L2; with 64 of them (128 MiB: resident in the Infinity Cache, 16 MiB per XCD: not in its L2), one per
    # four workgroups of an XCD, a quarter of the requests goes over the fabric, as in the tile kernels
    window = (torch.rand(64 << 20, device="cuda") * 4 - 2).to(torch.bfloat16)
    for wgs in (cus, cus // 2):
        for pattern, name in ((0, "constant operands"), (1, "random bf16 operands"),
                              (2, "random, fragments re-read from LDS"), (3, "random, LDS reads + LDS writes"),
                              (4, "random, LDS traffic + operand loads"),
                              (5, "random, LDS traffic + loads + barrier"),
                              (6, "same, a quarter of the loads over fabric")):
            def run():
                if pattern >= 4:
                    rc = probe.lce_probe_mfma_loads(wgs, iters, ctypes.c_void_p(window.data_ptr()), 2 << 20,
                                                    64 if pattern == 6 else 1, int(pattern >= 5),
                                                    ctypes.c_void_p(buf.data_ptr()), stream)
                else:
                    rc = probe.lce_probe_mfma(pattern, wgs, iters, ctypes.c_void_p(buf.data_ptr()), stream)
                assert rc == 0
            ms = _events_ms(run, torch, 3)
            flops = wgs * 4.0 * iters * 16 * 32768
            out["mfma_loop"].append(dict(operands=name, workgroups=wgs, waves_per_simd=1, ms=ms,
                                         tflops=flops / ms / 1e9, tflops_per_cu=flops / ms / 1e9 / wgs))
    del window
    N, H, V = 16384, 2048, 131072
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(N, H, device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn(H, V // 4, device="cuda", generator=g) / math.sqrt(H)).to(torch.bfloat16)
    dz = (torch.randn(N, V // 4, device="cuda", generator=g) * 1e-3).to(torch.bfloat16)
    for name, a, b in (("logits of one slab  x[N,H] @ W[H,V/4]", x, w), ("dx of one slab  dz[N,V/4] @ W^T", dz, w.t()),
                       ("dW of one slab  x^T @ dz[N,V/4]", x.t(), dz)):
        ms = _events_ms(lambda: torch.matmul(a, b), torch, 10)
        out["vendor_gemm"].append(dict(gemm=name, ms=ms, tflops=2.0 * N * H * (V // 4) / ms / 1e9))
    del dz
    wf = (torch.randn(H, V, device="cuda", generator=g) / math.sqrt(H)).to(torch.bfloat16)
    ms = _events_ms(lambda: torch.matmul(x, wf), torch, 5)
    out["vendor_gemm"].append(dict(gemm="all logits  x[N,H] @ W[H,V]", ms=ms, tflops=2.0 * N * H * V / ms / 1e9))
    # the operator's own forward tile kernel, all compute units against half of them
    lib = _lib.load()
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    lse = torch.empty(N, device="cuda")
    out5 = torch.empty(5, device="cuda")
    nv = torch.empty(1, dtype=torch.int64, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    for cap in (0, cus // 2):
        p = _lib.make_problem(N, H, V, H, V, H, V, x.dtype, wf.dtype, x.dtype, wf.dtype, -1, 1.0, 0.0, 4096, False,
                              _lib.PHASE_FWD_TILES, _lib.PACK_NEVER, cap)
        fwd_b, _ = _lib.workspace_bytes(p)
        ws = torch.empty(fwd_b, dtype=torch.uint8, device="cuda")

        def run():
            rc = lib.lce_forward(ctypes.byref(p), P(x), P(wf), P(y), P(lse), P(out5), P(nv), P(ws), fwd_b, stream)
            assert rc == 0
        ms = _events_ms(run, torch, 5)
        n = cap or cus
        out["fwd_tiles"].append(dict(workgroups=n, ms=ms, tflops=2.0 * N * H * V / ms / 1e9,
                                     tflops_per_cu=2.0 * N * H * V / ms / 1e9 / n))
    return out


def probe_flush(torch):
    """Cost of flushing 256 x 256 fp32 blocks of partial sums into a matrix in memory, the traffic a backward
    would generate that fed every dz tile straight into the dx and dW contractions: a compute unit cannot hold
    an H-wide accumulator (256 x H fp32 = 2 MiB at H = 2048 against 512 KiB of registers), so each
    256-token x 256-column dz tile would add H/256 blocks to dW and H/256 blocks to dx."""
    probe = _load_probe_lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    H, Vs = 2048, 32768  # one slab of dW in fp32: 256 MiB
    dst = torch.zeros(H, Vs, dtype=torch.float32, device="cuda")
    tiles = 64
    out = {"probe": "flush", "compute_units": cus, "target": f"fp32 [{H}][{Vs}]", "block": "256 x 256 fp32 = 256 KiB",
           "modes": []}
    for atomic, name in ((1, "fp32 atomic add (global_atomic_add_f32)"), (0, "plain 16-byte load + add + store (no other writer)")):
        def run():
            rc = probe.lce_probe_flush(atomic, ctypes.c_void_p(dst.data_ptr()), H, Vs, tiles, cus, stream)
            assert rc == 0
        ms = _events_ms(run, torch, 3)
        payload = cus * tiles * 256 * 256 * 4
        out["modes"].append(dict(mode=name, ms=ms, blocks=cus * tiles, us_per_block_per_cu=ms * 1e3 / tiles,
                                 payload_TB_per_s=payload / ms / 1e9))
    # what the default workload would flush per step: R/256 x V/256 dz tiles, each 2 * H/256 blocks
    N, V = 16384, 131072
    dz_tiles = (N // 256) * (V // 256)
    blocks = dz_tiles * 2 * (H // 256)
    out["fused_backward_at_default_shape"] = dict(
        dz_tiles=dz_tiles, blocks_flushed=blocks, payload_GiB=blocks * 256 * 256 * 4 / 2 ** 30,
        ms_at_measured_rate={m["mode"]: blocks * 256 * 256 * 4 / (m["payload_TB_per_s"] * 1e9) for m in out["modes"]},
        note="to be compared with the 19 ms the whole staged backward takes (dz through a 16-bit buffer in HBM)")
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2_bf16_N16384_H2048_V131072", choices=sorted(WORKLOADS) + ["c4_sweep"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--probe", choices=["ceiling", "flush"],
                    help="run a measurement probe instead of the benchmark and print its JSON: 'ceiling' (register-only "
                         "MFMA loop, vendor GEMM, half of the compute units), 'flush' (partial-sum blocks into memory)")
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
    from linear_cross_entropy_loss_amd import _lib, linear_cross_entropy

    if not _lib.LIB_PATH.exists():  # normally built beforehand and shipped with the tree
        from linear_cross_entropy_loss_amd.build import build

        build(force=True)

    if args.probe:
        print(json.dumps(probe_ceiling(torch) if args.probe == "ceiling" else probe_flush(torch)))
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

    ms_median = median_step_ms(step, torch, reps=20, flush=False)
    ms_median_flushed = median_step_ms(step, torch, reps=20, flush=True)
    x.grad = None
    w.grad = None

    phases = time_phases(cfg, x.detach(), y, w.detach(), torch)
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
            roofline["traffic"] = tr.get(args.workload, {}).get(dom)
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
        "flops_note": "value counts the FLOPs executed: tokens with an ignored label are dropped before the tile "
                      "kernels, so 8*H*V is multiplied by the tokens computed, not by N",
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
        "kernels": phases,
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(cfg, torch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()

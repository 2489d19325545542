"""Measurement probes behind ``bench.py --probe``: what bounds the tile kernels on this part.

Not part of the operator: a HIP source and a library of their own (``lce_probe.hip`` -> ``liblce_probe_gfx950.so``
in this folder), built on demand with ``python -m linear_cross_entropy_loss_amd.build --probes``.
"""
from __future__ import annotations

import ctypes
import math

# MI355X published dense bf16 peak (the denominator of the ceiling probe's fractions)
PEAK_TFLOPS = {"bf16": 2500.0}


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
    from linear_cross_entropy_loss_amd.build import PROBE_LIB_PATH, build_probes

    if not PROBE_LIB_PATH.exists():
        build_probes()
    lib = ctypes.CDLL(str(PROBE_LIB_PATH))
    vp = ctypes.c_void_p
    lib.lce_probe_mfma.restype = ctypes.c_int
    lib.lce_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
    lib.lce_probe_mfma_loads.restype = ctypes.c_int
    lib.lce_probe_mfma_loads.argtypes = [ctypes.c_int, ctypes.c_int, vp, ctypes.c_uint64, ctypes.c_int, ctypes.c_int, vp, vp]
    lib.lce_probe_flush.restype = ctypes.c_int
    lib.lce_probe_flush.argtypes = [ctypes.c_int, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, vp]
    lib.lce_probe_overlap.restype = ctypes.c_int
    lib.lce_probe_overlap.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
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


def probe_overlap(torch):
    """How much of an epilogue's vector ALU work hides behind matrix instructions of the same wave (one wave per
    SIMD, as in the tile kernels): the register-only MFMA loop on random operands with k = 1, 2, 4 (fma, exp2, add)
    triples behind every MFMA, against the MFMAs alone and the triples alone.  The tile kernels' epilogues have
    about 40 such triples per matrix instruction of a K tile (256 logits per lane against 64 MFMAs)."""
    probe = _load_probe_lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    buf = torch.empty(cus * 256, dtype=torch.float32, device="cuda")
    iters = 200000
    out = {"probe": "overlap", "compute_units": cus, "mfma_per_wave": iters * 16, "rows": []}

    def ms_of(mode, k):
        def run():
            assert probe.lce_probe_overlap(mode, k, cus, iters, ctypes.c_void_p(buf.data_ptr()), stream) == 0
        return _events_ms(run, torch, 3)

    m = ms_of(0, 1)
    out["mfma_only_ms"] = m
    out["mfma_only_tflops"] = cus * 4.0 * iters * 16 * 32768 / m / 1e9
    for k in (1, 2, 4):
        v, b = ms_of(1, k), ms_of(2, k)
        out["rows"].append(dict(triples_per_mfma=k, valu_only_ms=v, both_ms=b, sum_ms=m + v, max_ms=max(m, v),
                                hidden_frac_of_the_shorter=(m + v - b) / min(m, v)))
    return out


def run(name, torch):
    return {"ceiling": probe_ceiling, "flush": probe_flush, "overlap": probe_overlap}[name](torch)

"""lce_forward_static (the entry point that allocates nothing) against lce_forward, through the C ABI.

Two calls in a row on the library's static scratch, the second on a smaller problem: every output must equal
lce_forward's bit for bit (same kernels, same order, another scratch address), nothing may be allocated on
the device between the calls, and a problem beyond the static scratch must be refused with LCE_ESTATIC.
"""
import ctypes

import pytest
import torch

from helpers import make_inputs

pytestmark = pytest.mark.gpu


def _P(t):
    return ctypes.c_void_p(t.data_ptr())


def _both_ways(lib, _lib, N, H, V, dtype, seed, ignore_frac, z_reg, scale, monitoring, pack):
    x, y, w = make_inputs(N, H, V, dtype, seed=seed, ignore_frac=ignore_frac, device="cuda")
    p = _lib.make_problem(N, H, V, H, V, H, V, x.dtype, w.dtype, x.dtype, w.dtype, -1, scale, z_reg, 512,
                          monitoring, 0, pack)
    fwd_b, _ = _lib.workspace_bytes(p)
    assert fwd_b <= _lib.STATIC_SCRATCH_BYTES
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for static in (False, True):
        # outputs pre-filled with different garbage so that an unwritten cell cannot compare equal by luck
        lse = torch.full((N,), 7.0 if static else -3.0, device="cuda")
        out5 = torch.full((5,), 11.0 if static else -5.0, device="cuda")
        nv = torch.full((1,), 99 if static else -99, dtype=torch.int64, device="cuda")
        if static:
            torch.cuda.synchronize()
            free0 = torch.cuda.mem_get_info()[0]
            rc = lib.lce_forward_static(ctypes.byref(p), _P(x), _P(w), _P(y), _P(lse), _P(out5), _P(nv), stream)
            torch.cuda.synchronize()
            free1 = torch.cuda.mem_get_info()[0]
        else:
            ws = torch.empty(fwd_b, dtype=torch.uint8, device="cuda")
            rc = lib.lce_forward(ctypes.byref(p), _P(x), _P(w), _P(y), _P(lse), _P(out5), _P(nv), _P(ws), fwd_b, stream)
            torch.cuda.synchronize()
            free0 = free1 = 0
        assert rc == 0, (static, rc, lib.lce_strerror(rc))
        outs.append((lse, out5, nv, free0, free1))
    (lse_a, out_a, nv_a, _, _), (lse_b, out_b, nv_b, free0, free1) = outs
    assert torch.equal(lse_a, lse_b)
    assert torch.equal(out_a.view(torch.int32), out_b.view(torch.int32))  # bit for bit (NaN-safe)
    assert torch.equal(nv_a, nv_b) and nv_a.item() == int((y != -1).sum().item())
    return free0, free1


def test_static_forward_equals_forward_on_two_calls_in_a_row():
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    print("static forward: first call (N=2048, H=520, V=16384, bf16, monitoring, packed rows)", flush=True)
    _both_ways(lib, _lib, 2048, 520, 16384, torch.bfloat16, 71, 0.2, 1e-4, 0.5, True, _lib.PACK_ALWAYS)
    print("static forward: second call, smaller (N=300, H=264, V=5000, f16)", flush=True)
    free0, free1 = _both_ways(lib, _lib, 300, 264, 5000, torch.float16, 72, 0.1, 0.0, 1.0, False, _lib.PACK_ALWAYS)
    # the second call on this device found the scratch address cached: the device's free memory did not move
    # (to within what the runtime's own pools of launch arguments and signals may grow by; that the library
    # imports no allocation routine at all is checked on its symbol table, tests/test_abi_host.py)
    assert abs(free0 - free1) <= 8 << 20, (free0, free1)
    print("static forward: third call, larger again, fp32 master weight", flush=True)
    x, y, w = make_inputs(1024, 256, 8192, torch.float16, seed=73, ignore_frac=0.0, w_dtype=torch.float32, device="cuda")
    p = _lib.make_problem(1024, 256, 8192, 256, 8192, 256, 8192, x.dtype, w.dtype, x.dtype, w.dtype, -1, 1.0, 0.0, 512,
                          False, 0, _lib.PACK_NEVER)
    fwd_b, _ = _lib.workspace_bytes(p)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = []
    for static in (False, True):
        lse = torch.empty(1024, device="cuda")
        out5 = torch.empty(5, device="cuda")
        nv = torch.empty(1, dtype=torch.int64, device="cuda")
        if static:
            rc = lib.lce_forward_static(ctypes.byref(p), _P(x), _P(w), _P(y), _P(lse), _P(out5), _P(nv), stream)
        else:
            ws = torch.empty(fwd_b, dtype=torch.uint8, device="cuda")
            rc = lib.lce_forward(ctypes.byref(p), _P(x), _P(w), _P(y), _P(lse), _P(out5), _P(nv), _P(ws), fwd_b, stream)
        torch.cuda.synchronize()
        assert rc == 0
        res.append((lse, out5, nv))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1]) and torch.equal(res[0][2], res[1][2])


def test_static_forward_refuses_what_does_not_fit():
    from linear_cross_entropy_loss_amd import _lib

    lib = _lib.load()
    print("static forward: oversize problem is refused", flush=True)
    x, y, w = make_inputs(256, 256, 4096, torch.bfloat16, seed=74, device="cuda")
    lse = torch.empty(256, device="cuda")
    out5 = torch.empty(5, device="cuda")
    nv = torch.empty(1, dtype=torch.int64, device="cuda")
    # the benchmark shape needs 64 MiB of partials alone: refused from the problem description, before any
    # pointer is looked at
    big = _lib.make_problem(16384, 2048, 131072, 2048, 131072, 2048, 131072, x.dtype, w.dtype, x.dtype, w.dtype, -1,
                            1.0, 0.0, 4096, False, 0, _lib.PACK_AUTO)
    fwd_b, _ = _lib.workspace_bytes(big)
    assert fwd_b > _lib.STATIC_SCRATCH_BYTES
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.lce_forward_static(ctypes.byref(big), _P(x), _P(w), _P(y), _P(lse), _P(out5), _P(nv), stream)
    assert rc == _lib.LCE_ESTATIC
    assert b"static" in lib.lce_strerror(rc)
    with pytest.raises(RuntimeError, match="static"):
        _lib.raise_for_status(rc, "lce_forward_static")
    # The sizes include/lce.h quotes at V = 131072, H = 2048: 4096 rows fit without the monitoring values (32.1 MiB)
    # and do not with them (four partial buffers instead of one, no packed copy of x: 64.02 MiB); 2048 rows with
    # monitoring fit.
    for rows, mon, fits in ((4096, False, True), (4096, True, False), (2048, True, True)):
        p = _lib.make_problem(rows, 2048, 131072, 2048, 131072, 2048, 131072, x.dtype, w.dtype, x.dtype, w.dtype, -1,
                              1.0, 0.0, 4096, mon, 0, _lib.PACK_AUTO)
        need, _ = _lib.workspace_bytes(p)
        assert (need <= _lib.STATIC_SCRATCH_BYTES) == fits, (rows, mon, need)
        if not fits:  # refused before any pointer is looked at (these buffers are far too small for the problem)
            assert lib.lce_forward_static(ctypes.byref(p), _P(x), _P(w), _P(y), _P(lse), _P(out5), _P(nv), stream) == _lib.LCE_ESTATIC
    sizes = {mon: _lib.workspace_bytes(_lib.make_problem(4096, 2048, 131072, 2048, 131072, 2048, 131072, x.dtype, w.dtype,
                                                         x.dtype, w.dtype, -1, 1.0, 0.0, 4096, mon, 0, _lib.PACK_AUTO))[0]
             for mon in (False, True)}
    assert abs(sizes[False] / 2**20 - 32.1) < 0.1 and abs(sizes[True] / 2**20 - 64.02) < 0.1, sizes

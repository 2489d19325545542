"""CPU-side checks: the C-ABI library loads and exports what include/lce.h declares; argument validation and
scratch planning behave as documented; the Python surface mirrors the reference's.  No compute calls."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from linear_cross_entropy_loss_amd import _lib
    from linear_cross_entropy_loss_amd.build import build

    build(force=False)
    return _lib.load()


def _prob(**kw):
    from linear_cross_entropy_loss_amd import _lib

    d = dict(N=512, H=256, V=4096, ldx=256, ldw=4096, lddx=256, lddw=4096, x_dtype=torch.bfloat16,
             w_dtype=torch.bfloat16, dx_dtype=torch.bfloat16, dw_dtype=torch.bfloat16, ignore_index=-100,
             logit_scale=1.0, z_reg=0.0, n_chunk=4096, monitoring=False)
    d.update(kw)
    return _lib.make_problem(**d)


def test_every_declared_symbol_is_exported(lib):
    from linear_cross_entropy_loss_amd import _lib

    header = open(os.path.join(ROOT, "include", "lce.h")).read()
    declared = set(re.findall(r"^\s*(?:const\s+char\*|int)\s+(lce_\w+)\s*\(", header, flags=re.M))
    assert declared == set(_lib.EXPORTS), (declared, _lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.lce_version() >= 100


def test_struct_layout_matches_header():
    from linear_cross_entropy_loss_amd import _lib

    header = open(os.path.join(ROOT, "include", "lce.h")).read()
    body = re.search(r"typedef struct lce_problem \{(.*?)\} lce_problem;", header, flags=re.S).group(1)
    fields = re.findall(r"^\s*(int64_t|int32_t|float)\s+(\w+);", body, flags=re.M)
    ctype = {"int64_t": ctypes.c_int64, "int32_t": ctypes.c_int32, "float": ctypes.c_float}
    assert [(n, ctype[t]) for t, n in fields] == list(_lib.LceProblem._fields_)
    assert ctypes.sizeof(_lib.LceProblem) == 7 * 8 + 4 * 4 + 8 + 2 * 4 + 8 + 6 * 4


def test_shape_contract(lib):
    """The reference's divisibility rules (ops.py:689-691, 905-907) are lifted: any N, H, V >= 1 is accepted;
    only row strides are constrained (16-byte rows).  Non-positive sizes keep the reference's ValueError."""
    from linear_cross_entropy_loss_amd import _lib

    ok = _prob()
    assert lib.lce_check_problem(ctypes.byref(ok)) == _lib.LCE_OK
    for fine in (dict(N=500), dict(N=1), dict(H=128, ldx=128, lddx=128), dict(H=100, ldx=104, lddx=104),
                 dict(V=4000, ldw=4000, lddw=4000), dict(V=50257, ldw=50264, lddw=50264), dict(n_chunk=100)):
        assert lib.lce_check_problem(ctypes.byref(_prob(**fine))) == _lib.LCE_OK, fine
    for bad in (dict(N=0), dict(H=0, ldx=8), dict(V=-8), dict(n_chunk=0), dict(N=(1 << 30) + 1)):
        assert lib.lce_check_problem(ctypes.byref(_prob(**bad))) == _lib.LCE_EINVAL_SHAPE, bad
    for bad in (dict(H=100, ldx=100, lddx=104), dict(V=50257, ldw=50257, lddw=50264), dict(H=100, ldx=104, lddx=102),
                dict(V=50257, ldw=50264, lddw=50260), dict(ldx=248)):
        assert lib.lce_check_problem(ctypes.byref(_prob(**bad))) == _lib.LCE_EINVAL_ARG, bad
    assert lib.lce_check_problem(ctypes.byref(_prob(logit_scale=0.0))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(ctypes.byref(_prob(z_reg=-1.0))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(ctypes.byref(_prob(ldx=250))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(ctypes.byref(_prob(x_dtype=torch.bfloat16, w_dtype=torch.float16))) == _lib.LCE_EINVAL_DTYPE
    assert lib.lce_check_problem(ctypes.byref(_prob(x_dtype=torch.float32, w_dtype=torch.bfloat16))) == _lib.LCE_EINVAL_DTYPE
    assert lib.lce_check_problem(ctypes.byref(_prob(w_dtype=torch.float32, dw_dtype=torch.float32))) == _lib.LCE_OK
    # 32-bit tile addressing: 256 rows of x, of a 16-bit w and of dx stay below 2 GiB; an fp32 w is exempt
    big = (1 << 22) + 8
    assert lib.lce_check_problem(ctypes.byref(_prob(V=4096, ldw=big, lddw=big))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(ctypes.byref(_prob(V=4096, ldw=1 << 22, lddw=1 << 22))) == _lib.LCE_OK
    assert lib.lce_check_problem(ctypes.byref(_prob(V=4096, ldw=big, lddw=big, w_dtype=torch.float32, dw_dtype=torch.float32))) == _lib.LCE_OK
    assert lib.lce_check_problem(ctypes.byref(_prob(ldx=big))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(ctypes.byref(_prob(lddx=big))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(ctypes.byref(_prob(N=1 << 30, V=1 << 20, ldw=1 << 20, lddw=1 << 20))) == _lib.LCE_EINVAL_SHAPE
    assert lib.lce_check_problem(ctypes.byref(_prob(pack_rows=3))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(None) == _lib.LCE_EINVAL_ARG


def test_status_maps_to_reference_exceptions(lib):
    from linear_cross_entropy_loss_amd import _lib

    with pytest.raises(ValueError, match="Provided shape outside the range of valid configs"):
        _lib.raise_for_status(_lib.LCE_EINVAL_SHAPE, "x")
    with pytest.raises(ValueError):
        _lib.raise_for_status(_lib.LCE_EINVAL_DTYPE, "x")
    with pytest.raises(RuntimeError):
        _lib.raise_for_status(_lib.LCE_EWORKSPACE, "x")
    assert b"HIP" in lib.lce_strerror(_lib.LCE_EHIP)


@pytest.mark.parametrize("N,H,V,n_chunk", [(16384, 2048, 131072, 4096), (16384, 4096, 131072, 4096),
                                           (16384, 2048, 262144, 2048), (16384, 2048, 32768, 8192),
                                           (65536, 8192, 262144, 8192), (512, 256, 4096, 512),
                                           (1000, 520, 50264, 4096), (16384, 768, 50264, 4096)])
def test_backward_scratch_within_n_chunk_bound(N, H, V, n_chunk):
    from linear_cross_entropy_loss_amd import _lib

    p = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=n_chunk)
    fwd, bwd = _lib.workspace_bytes(p)
    assert bwd <= n_chunk * V * 4
    assert fwd >= (V // 128) * N * 4


def _pack_bytes(N, H, es_x=2, es_dx=2, backward=True):
    """Scratch of the packed rows (tokens with an ignored label dropped): segment counts, the row count, the
    row -> token map, packed labels and the packed copy of x; for the backward also the packed lse and -- only
    for a dx of 2 GiB or more, which 32-bit store offsets cannot span -- a packed staging copy of dx."""
    al = lambda v: -(-v // 256) * 256
    pad = lambda v, m: -(-v // m) * m
    b = al(-(-N // 2048) * 4) + 256 + al(4 * N) + al(8 * N) + al(N * pad(H, 16 // es_x) * es_x)
    if backward:
        b += al(4 * N)
        if N * H * es_dx >= 1 << 31:   # (the tests use lddx = H)
            b += al(N * pad(H, 8) * es_dx)
    return b


def test_budget_is_a_target_not_a_refusal():
    """Small vocabulary with many tokens: the strict bound N_chunk*V*4 cannot be met (the fp32 running dx alone
    exceeds it).  The bound is then widened by N*H*4, the fp32 x_grad buffer the reference allocates beside
    its logits chunk (ops.py:693); beyond that the narrowest split is used.  The call is never refused."""
    from linear_cross_entropy_loss_amd import _lib

    N, H, nc = 16384, 2048, 4096
    for V in (256, 4096, 8192):     # one slab fits the widened bound: no running dx at all
        p = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=nc, pack_rows=_lib.PACK_ALWAYS)
        assert _lib.backward_plan(p) == (1, V)
        _, bwd = _lib.workspace_bytes(p)
        # dz for all tokens within the widened bound; on top: the packed rows and at most 64 MiB each of
        # K-split partial sums of dW (few dW tiles) and of dx (room for a split last round of tiles)
        assert nc * V * 4 < N * V * 2 <= nc * V * 4 + N * H * 4 and 0 <= bwd - N * V * 2 - _pack_bytes(N, H) <= 128 << 20
    p = _prob(N=65536, H=256, V=4096, ldx=256, ldw=4096, lddx=256, lddw=4096, n_chunk=64,
              pack_rows=_lib.PACK_ALWAYS)   # nothing fits
    assert _lib.backward_plan(p) == (16, 256)
    _, bwd = _lib.workspace_bytes(p)
    # dz + fp32 running dx (256 dx tiles: no K split) + the split-K partials of the single dW tile
    assert 0 < bwd - (65536 * 256 * 2 + 65536 * 256 * 4) - _pack_bytes(65536, 256) <= 128 << 20


def test_backward_plan_is_consistent_with_workspace():
    from linear_cross_entropy_loss_amd import _lib

    pad = lambda v, m: -(-v // m) * m

    def dx_part_bytes(Np, Hp, vs, last_vs):
        # dx: the tiles of a last, mostly idle round of workgroups are cut along K on the device; room for the
        # most 256 x 256 fp32 blocks that can ask for: (tiles x most segments per tile), capped at 256
        def blocks(w):
            kt, s = w // 64, 1
            while kt // (s * 2) >= 16 and s * 2 <= 256:
                s *= 2
            return 0 if s == 1 else min(256, (Np // 256) * (Hp // 256) * s)
        return max(blocks(vs), blocks(last_vs)) * 256 * 256 * 4

    def dw_part_bytes(Np, Hp, vs, last_vs):
        # the same for dW, whose K runs over the tokens and whose segments need not divide the K tiles evenly
        def blocks(w):
            kt, s = Np // 64, 1
            while kt // (s * 2) >= 16 and s * 2 <= 256:
                s *= 2
            return 0 if s == 1 else min(256, (w // 256) * (Hp // 256) * s)
        return max(blocks(vs), blocks(last_vs)) * 256 * 256 * 4

    for N, H, V, nc in ((16384, 2048, 131072, 4096), (16384, 2048, 131072, 8192), (65536, 8192, 262144, 8192),
                        (512, 256, 4096, 512), (1000, 520, 50264, 512), (300, 104, 1008, 64), (16384, 768, 50264, 4096)):
        p = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=nc, pack_rows=_lib.PACK_ALWAYS)
        slabs, width = _lib.backward_plan(p)
        # slabs of `width` columns (a multiple of 256) cover the vocabulary; the last one may be narrower
        assert width % 256 == 0 and (slabs - 1) * width < V <= slabs * width
        Np, Hp = pad(N, 256), pad(H, 256)
        _, bwd = _lib.workspace_bytes(p)
        part = dx_part_bytes(Np, Hp, width, pad(V, 256) - (slabs - 1) * width)
        partw = dw_part_bytes(Np, Hp, width, pad(V, 256) - (slabs - 1) * width)
        assert part <= 64 << 20 and partw <= 64 << 20
        # (one buffer serves both: the dx kernels are done with it before the dW kernels start)
        assert bwd == _pack_bytes(N, H) + Np * width * 2 + (Np * Hp * 4 if slabs > 1 else 0) + max(part, partw)
        assert Np * width * 2 <= max(1 << 30, Np * 256 * 2)   # dz stage capped at 1 GiB
        # without the packing of ignored tokens: the same minus its buffers, if the split stays the same;
        # by default the library packs from 8*N*H*V = 2^41 FLOPs on
        q = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=nc, pack_rows=_lib.PACK_NEVER)
        if _lib.backward_plan(q) == (slabs, width):
            assert _lib.workspace_bytes(q)[1] == bwd - _pack_bytes(N, H)
        auto = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=nc)
        assert _lib.workspace_bytes(auto) == _lib.workspace_bytes(p if 8 * N * H * V >= 2 ** 41 else q)


def test_fp32_weight_adds_one_16_bit_slab_copy_to_the_scratch():
    """An fp32 (master) weight is rounded to the compute type one vocabulary slab at a time; the scratch of
    both calls grows by that slab copy and stays within the N_chunk bound."""
    from linear_cross_entropy_loss_amd import _lib

    N, H, V, nc = 65536, 8192, 262144, 8192
    p16 = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=nc, x_dtype=torch.float16, w_dtype=torch.float16)
    p32 = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=nc, x_dtype=torch.float16, w_dtype=torch.float32,
                dw_dtype=torch.float32)
    f16, b16 = _lib.workspace_bytes(p16)
    f32, b32 = _lib.workspace_bytes(p32)
    slabs, width = _lib.backward_plan(p32)
    assert b32 - b16 == H * width * 2 and b32 <= nc * V * 4
    # forward: the slab copy (at most 256 MiB), and partial sums for chunks of 65536 tokens instead of 16384
    # (the copies are made once per chunk of tokens, so chunks are longer under an fp32 weight)
    assert f32 - f16 == (256 << 20) + (65536 - 16384) * (V // 128) * 4


def test_forward_scratch_does_not_grow_with_the_partial_sums_of_all_tokens():
    """The forward works through the tokens in chunks (of N_chunk_size rows, at least 16384), so its partial sums
    are one chunk wide however many tokens there are; what still grows with N is 16 bytes per token of packing
    state, 4 + 1/8 bytes of per-token results and, when tokens are packed, the packed copy of x."""
    from linear_cross_entropy_loss_amd import _lib

    H, V = 2048, 131072
    for mon in (False, True):
        sizes = []
        for N in (16384, 65536, 1 << 20):
            p = _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=4096, monitoring=1 if mon else 0,
                      pack_rows=_lib.PACK_NEVER)
            sizes.append(_lib.workspace_bytes(p)[0])
        part = (V // 128) * 16384 * 4 * (4 if mon else 1)
        for N, f in zip((16384, 65536, 1 << 20), sizes):
            assert part <= f <= part + N * 8 + 4096, (N, f)
    # a larger N_chunk_size widens the chunks
    p = _prob(N=1 << 20, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=65536, pack_rows=_lib.PACK_NEVER)
    assert _lib.workspace_bytes(p)[0] >= (V // 128) * 65536 * 4


def test_null_and_small_workspace_are_rejected_without_touching_the_gpu(lib):
    from linear_cross_entropy_loss_amd import _lib

    p = _prob()
    one = ctypes.c_void_p(256)  # never dereferenced: validation fails first
    rc = lib.lce_forward(ctypes.byref(p), one, one, one, one, one, one, None, 0, None)
    assert rc == _lib.LCE_EWORKSPACE
    rc = lib.lce_forward(ctypes.byref(p), None, one, one, one, one, one, one, 1 << 30, None)
    assert rc == _lib.LCE_EINVAL_ARG
    rc = lib.lce_backward(ctypes.byref(p), one, one, one, one, one, one, one, one, one, 16, None)
    assert rc == _lib.LCE_EWORKSPACE
    rc = lib.lce_backward(ctypes.byref(p), one, one, one, one, one, one, ctypes.c_void_p(260), one, one, 1 << 40, None)
    assert rc == _lib.LCE_EINVAL_ARG  # misaligned dx
    # lce_forward_backward, on its one-pass route (a bf16 problem that it covers) and on the two calls it makes otherwise
    f32 = dict(x_dtype=torch.float32, w_dtype=torch.float32, dx_dtype=torch.float32, dw_dtype=torch.float32)
    for kw in (dict(), f32):
        q = _prob(**kw)
        args = lambda ws, n, dx=one: (ctypes.byref(q), one, one, one, one, one, one, one, dx, one, ws, n, None)
        assert lib.lce_forward_backward(*args(None, 0)) == _lib.LCE_EWORKSPACE
        assert lib.lce_forward_backward(*args(one, 16)) == _lib.LCE_EWORKSPACE
        assert lib.lce_forward_backward(*args(one, 1 << 40, ctypes.c_void_p(260))) == _lib.LCE_EINVAL_ARG
        assert lib.lce_forward_backward(ctypes.byref(q), one, one, one, None, one, one, one, one, one, one, 1 << 40,
                                        None) == _lib.LCE_EINVAL_ARG  # no upstream gradient


def test_python_surface_mirrors_reference():
    import linear_cross_entropy_loss_amd as pkg

    assert pkg.fwd_configs == [] and pkg.bwd_configs == []
    sig = inspect.signature(pkg.linear_cross_entropy)
    assert list(sig.parameters) == ["x", "y", "At", "ignore_index", "z_regularization", "logit_scale",
                                    "N_chunk_size", "monitoring"]
    assert sig.parameters["ignore_index"].default == -100
    assert sig.parameters["N_chunk_size"].default == 4096 and sig.parameters["monitoring"].default is False
    msig = inspect.signature(pkg.LinearCrossEntropyLoss.__init__)
    assert list(msig.parameters)[1:] == ["in_features", "out_features", "device", "dtype", "ignore_index",
                                         "logit_scale", "z_regularization", "N_chunk_size", "init_method"]


def test_module_contract_on_cpu():
    from linear_cross_entropy_loss_amd import LinearCrossEntropyLoss

    m = LinearCrossEntropyLoss(256, 4096)
    assert isinstance(m, torch.nn.Linear)
    assert tuple(m.weight.shape) == (256, 4096)          # transposed weight
    assert not hasattr(m, "bias") or m.bias is None or "bias" not in dict(m.named_parameters())
    assert list(dict(m.named_parameters())) == ["weight"]
    assert m.ignore_index == -100 and m.monitoring is False and m.latest_metrics == {}
    std = (1 / 256) ** 0.5
    assert m.weight.abs().max() <= 3 * std + 1e-6 and abs(m.weight.std().item() - std) < 0.1 * std
    assert "bias=False" in repr(m)
    called = []
    LinearCrossEntropyLoss(256, 4096, init_method=lambda w: (called.append(1), w.data.zero_()))
    assert called
    # the reference's divisibility asserts (ops.py:905-907) are lifted; non-positive sizes still assert
    LinearCrossEntropyLoss(100, 1000, N_chunk_size=100)
    for bad in (dict(in_features=0, out_features=4096), dict(in_features=256, out_features=0)):
        with pytest.raises(AssertionError):
            LinearCrossEntropyLoss(**bad)
    with pytest.raises(AssertionError):
        LinearCrossEntropyLoss(256, 4096, N_chunk_size=0)
    with pytest.raises(AssertionError):
        LinearCrossEntropyLoss(256, 4096, logit_scale=0.0)
    sd = m.state_dict()
    assert list(sd) == ["weight"]


def test_cpu_tensors_fail_loudly():
    from linear_cross_entropy_loss_amd import linear_cross_entropy

    x = torch.randn(512, 256)
    w = torch.randn(256, 4096)
    y = torch.randint(0, 4096, (512,))
    with pytest.raises(RuntimeError, match="no CPU path"):
        linear_cross_entropy(x, y, w)


def test_product_does_not_import_the_oracle():
    pkg_dir = os.path.join(ROOT, "linear_cross_entropy_loss_amd")
    for dirpath, _, files in os.walk(pkg_dir):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)


def test_header_is_plain_c_and_links_from_a_c_program(tmp_path):
    """include/lce.h compiles as strict C99 and a C program linked against the library can call the
    host-only entry points (no GPU involved: validation, planning, error strings)."""
    import shutil
    import subprocess

    from linear_cross_entropy_loss_amd import _lib

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "lce.h"
int main(void) {
  lce_problem p;
  size_t fwd = 0, bwd = 0;
  int64_t slabs = 0, width = 0;
  memset(&p, 0, sizeof p);
  p.N = 16384; p.H = 2048; p.V = 131072; p.ldx = 2048; p.ldw = 131072; p.lddx = 2048; p.lddw = 131072;
  p.x_dtype = LCE_BF16; p.w_dtype = LCE_BF16; p.dx_dtype = LCE_BF16; p.dw_dtype = LCE_BF16;
  p.ignore_index = -100; p.logit_scale = 1.0f; p.z_reg = 0.0f; p.n_chunk = 4096;
  if (lce_check_problem(&p) != LCE_OK) return 1;
  if (lce_workspace_bytes(&p, &fwd, &bwd) != LCE_OK) return 2;
  if (lce_backward_plan(&p, &slabs, &width) != LCE_OK) return 3;
  p.N = 0;
  if (lce_check_problem(&p) != LCE_EINVAL_SHAPE) return 4;
  printf("%d %lu %lu %ld %ld %s\n", lce_version(), (unsigned long)fwd, (unsigned long)bwd, (long)slabs, (long)width,
         lce_strerror(LCE_EWORKSPACE));
  return 0;
}
''')
    exe = tmp_path / "abi"
    libdir = str(_lib.LIB_PATH.parent)
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", inc, str(src), "-o", str(exe),
                    "-L", libdir, "-l:" + _lib.LIB_PATH.name, "-Wl,-rpath," + libdir,
                    "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split(None, 5)
    assert int(out[0]) >= 100 and int(out[3]) == 4 and int(out[4]) == 32768
    assert int(out[2]) <= 4096 * 131072 * 4 and "workspace" in out[5]


def test_library_imports_no_allocation_or_synchronisation_routine():
    """The operator's library allocates nothing, frees nothing and never synchronises: its dynamic symbol table
    imports no HIP routine that could (the whole list is device query, launch, error text and the symbol
    lookup of the static scratch)."""
    import subprocess

    from linear_cross_entropy_loss_amd import _lib

    out = subprocess.run(["nm", "-D", "--undefined-only", str(_lib.LIB_PATH)], capture_output=True, text=True, check=True)
    hip = sorted({line.split()[-1].split("@")[0] for line in out.stdout.splitlines() if " hip" in line})
    allowed = {"hipDeviceGetAttribute", "hipFuncSetAttribute", "hipGetDevice", "hipGetErrorString", "hipGetLastError",
               "hipGetSymbolAddress", "hipLaunchKernel", "__hipRegisterFatBinary", "__hipRegisterFunction",
               "__hipRegisterVar", "__hipUnregisterFatBinary", "__hipPushCallConfiguration", "__hipPopCallConfiguration"}
    assert set(hip) <= allowed, set(hip) - allowed
    for banned in ("Malloc", "Free", "Synchronize", "Memcpy", "Memset", "MemPool"):
        assert not any(banned in name for name in hip), (banned, hip)


def test_backward_plan_invariants_on_random_problems():
    """Seeded random problems: the slabs cover the vocabulary, widths are tile multiples, the reported scratch
    is what the bound allows whenever the narrowest split could meet it, a larger bound keeps the slab count
    inside the planner's search window, and forward scratch never depends on more than one chunk of tokens."""
    import random

    from linear_cross_entropy_loss_amd import _lib

    rng = random.Random(7)
    dts = (torch.bfloat16, torch.float16, torch.float32)
    for it in range(300):
        N = rng.choice([1, 100, 255, 256, 1000, 4096, 16384, 40000, 65536, 300000])
        H = rng.choice([8, 64, 264, 768, 2048, 4096, 8192])
        V = rng.choice([8, 1000, 4096, 32000, 50264, 131072, 262144])
        nc = rng.choice([16, 512, 2048, 4096, 8192, 65536])
        xd = rng.choice(dts)
        wd = xd if xd == torch.float32 else rng.choice((xd, torch.float32))
        pack = rng.choice((_lib.PACK_AUTO, _lib.PACK_ALWAYS, _lib.PACK_NEVER))
        mk = lambda n: _prob(N=N, H=H, V=V, ldx=H, ldw=V, lddx=H, lddw=V, n_chunk=n, x_dtype=xd, w_dtype=wd,
                             dx_dtype=xd, dw_dtype=wd, pack_rows=pack)
        p = mk(nc)
        fwd, bwd = _lib.workspace_bytes(p)
        slabs, width = _lib.backward_plan(p)
        Vp = -(-V // 256) * 256
        assert width % 256 == 0 and 1 <= slabs and (slabs - 1) * width < Vp <= slabs * width, (it, slabs, width)
        assert fwd > 0 and bwd > 0
        # The planner takes the fewest slabs that fit or, when its model of the kernels' rounds of workgroups says
        # that more of them run faster, up to 4 * fewest + 8.  A larger bound cannot raise the fewest that fit.
        slabs2, _ = _lib.backward_plan(mk(nc * 4))
        assert slabs2 <= 4 * slabs + 8, (it, slabs, slabs2)
        # forward: partial sums of one chunk of tokens at most, whatever N
        chunk = max(-(-nc // 256) * 256, 65536 if wd == torch.float32 and xd != torch.float32 or xd == torch.float32 else 16384)
        Np = -(-N // 256) * 256
        part = (Vp // 128) * min(Np, chunk) * 4
        split = 3 if xd == torch.float32 else 1
        slab_copy = (256 << 20) + 256 * H * 2 * split if wd == torch.float32 else 0
        assert fwd <= part + Np * 16 + N * (split * H + 8) * 2 + slab_copy + N * 16 + 8192, (it, fwd)


def test_vocabulary_major_weight_layout_is_checked_and_detected():
    """lce_problem.w_layout = LCE_W_VH: row strides are checked against H, fp32 activations and hidden sizes
    that are not multiples of 8 are refused; the Python host picks the layout from the strides alone."""
    from linear_cross_entropy_loss_amd import _lib, ops

    lib = _lib.load()
    ok = dict(N=512, H=256, V=1000, ldx=256, ldw=256, lddx=256, lddw=256, n_chunk=512, w_layout=_lib.W_VH)
    assert lib.lce_check_problem(ctypes.byref(_prob(**ok))) == 0
    assert _lib.workspace_bytes(_prob(**ok)) == _lib.workspace_bytes(_prob(**dict(ok, ldw=1000, lddw=1000, w_layout=_lib.W_HV)))
    assert lib.lce_check_problem(ctypes.byref(_prob(**dict(ok, ldw=248)))) == _lib.LCE_EINVAL_ARG      # shorter than a row
    assert lib.lce_check_problem(ctypes.byref(_prob(**dict(ok, w_layout=2)))) == _lib.LCE_EINVAL_ARG
    assert lib.lce_check_problem(ctypes.byref(_prob(**dict(ok, H=252, ldx=256)))) == _lib.LCE_EINVAL_ARG  # H % 8
    f32 = dict(ok, x_dtype=torch.float32, w_dtype=torch.float32, dx_dtype=torch.float32, dw_dtype=torch.float32)
    assert lib.lce_check_problem(ctypes.byref(_prob(**f32))) == _lib.LCE_EINVAL_DTYPE
    # a row-major (H, V) problem with the same numbers is refused for its strides (1000 columns need ldw >= 1000)
    assert lib.lce_check_problem(ctypes.byref(_prob(**dict(ok, w_layout=_lib.W_HV)))) == _lib.LCE_EINVAL_ARG

    w = torch.zeros(1000, 256, dtype=torch.bfloat16)     # (V, H) as a model stores it
    assert ops._weight_layout(w.t(), torch.bfloat16) == _lib.W_VH
    assert ops._weight_layout(w.t().contiguous(), torch.bfloat16) == _lib.W_HV
    assert ops._weight_layout(w.t(), torch.float32) == _lib.W_HV                      # fp32 activations: copied
    assert ops._weight_layout(torch.zeros(1000, 100, dtype=torch.bfloat16).t(), torch.bfloat16) == _lib.W_HV  # H % 8
    assert ops._weight_layout(torch.zeros(1000, 264, dtype=torch.bfloat16)[:, :256].t(), torch.bfloat16) == _lib.W_VH
    assert ops._weight_layout(torch.zeros(1000, 256, dtype=torch.float32).t(), torch.float16) == _lib.W_VH  # master weight


def test_a_weight_that_cannot_be_read_in_place_is_copied_with_one_warning():
    """A weight the kernels cannot read in place (here: (V, H) storage with H % 8 != 0, handed over transposed) is
    copied on every call; the host says so once, naming shape, strides and size, and stays silent afterwards.
    A weight that is read in place raises nothing."""
    import warnings

    from linear_cross_entropy_loss_amd import ops

    ops._copy_warned.clear()
    good = torch.zeros(64, 1000, dtype=torch.bfloat16)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        assert ops._weight_rows(good, ops._weight_layout(good, torch.bfloat16)) is good
    bad = torch.zeros(1000, 100, dtype=torch.bfloat16).t()  # (H, V) = (100, 1000) view of a (V, H) matrix
    with pytest.warns(UserWarning, match=r"weight of shape \(100, 1000\).*copied on every call"):
        w = ops._weight_rows(bad, ops._weight_layout(bad, torch.bfloat16))
    assert w.stride(1) == 1 and w.stride(0) % 8 == 0 and torch.equal(w, bad)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        ops._weight_rows(bad, ops._weight_layout(bad, torch.bfloat16))  # the second copy is silent


def test_one_pass_plan_stays_within_the_bound_and_covers_all_tokens(lib):
    """lce_forward_backward_plan: chunks of whole token tiles that cover N, a workspace within n_chunk * V * 4
    bytes, and no one-pass route for fp32 tensors, monitoring, or a bound that the fp32 plane of dW alone fills."""
    import random

    from linear_cross_entropy_loss_amd import _lib

    rng = random.Random(5)
    took = 0
    for _ in range(300):
        N = rng.choice([1, 255, 256, 1000, 4096, 16384, 65536, 100000])
        H = rng.choice([64, 520, 2048, 4096, 8192])
        V = rng.choice([777, 4096, 32768, 131072, 262144])
        n_chunk = rng.choice([256, 1024, 4096, 8192, 32768])
        dt = rng.choice([torch.bfloat16, torch.float16])
        prob = _lib.make_problem(N, H, V, H + (-H) % 8, V + (-V) % 8, H + (-H) % 8, V + (-V) % 8, dt, dt, dt, dt, -1, 1.0,
                                 0.0, n_chunk, False, route=_lib.ROUTE_ONE_PASS)
        auto = _lib.make_problem(N, H, V, H + (-H) % 8, V + (-V) % 8, H + (-H) % 8, V + (-V) % 8, dt, dt, dt, dt, -1, 1.0,
                                 0.0, n_chunk, False)
        never = _lib.make_problem(N, H, V, H + (-H) % 8, V + (-V) % 8, H + (-H) % 8, V + (-V) % 8, dt, dt, dt, dt, -1, 1.0,
                                  0.0, n_chunk, False, route=_lib.ROUTE_TWO_PASS)
        chunks, rows = _lib.forward_backward_plan(prob)
        assert _lib.forward_backward_plan(never) == (0, 0)
        assert _lib.forward_backward_plan(auto) in ((0, 0), (chunks, rows))  # the library's choice: the same plan, or two passes
        total = _lib.forward_backward_workspace_bytes(prob)
        if chunks == 0:
            assert total == max(_lib.workspace_bytes(prob))
            continue
        took += 1
        assert rows % 256 == 0 and rows > 0
        assert chunks * rows >= N and (chunks - 1) * rows < N + 255
        assert total <= n_chunk * V * 4, (N, H, V, n_chunk, total)
        if chunks > 1:  # the lower halves of the fp32 sums of dW are part of it (the upper halves lie in dW itself),
            assert total >= (H + (-H) % 256) * (V + (-V) % 256)  # cut to a byte each where two do not fit the bound
    assert took > 50
    # the benchmark's default shape: four chunks of 16 token tiles
    prob = _lib.make_problem(16384, 2048, 131072, 2048, 131072, 2048, 131072, torch.bfloat16, torch.bfloat16,
                             torch.bfloat16, torch.bfloat16, -1, 1.0, 0.0, 4096, False)
    assert _lib.forward_backward_plan(prob) == (4, 4096)
    # no one-pass route for fp32 activations
    for kw in (dict(x=torch.float32, w=torch.float32),):
        xd, wd, Hh = kw.get("x", torch.bfloat16), kw.get("w", torch.bfloat16), kw.get("H", 512)
        prob = _lib.make_problem(4096, Hh, 8192, Hh, 8192, Hh, 8192, xd, wd, xd, wd, -1, 1.0, 0.0, 4096,
                                 kw.get("mon", False), route=_lib.ROUTE_ONE_PASS)
        assert _lib.forward_backward_plan(prob) == (0, 0), kw
    prob = _lib.make_problem(4096, 512, 8192, 512, 8192, 512, 8192, torch.bfloat16, torch.bfloat16, torch.bfloat16,
                             torch.bfloat16, -1, 1.0, 0.0, 4096, True, route=_lib.ROUTE_ONE_PASS)
    assert _lib.forward_backward_plan(prob)[0] > 0  # the monitoring values are covered
    prob = _lib.make_problem(4096, 520, 8192, 520, 8192, 520, 8192, torch.bfloat16, torch.bfloat16, torch.bfloat16,
                             torch.bfloat16, -1, 1.0, 0.0, 4096, True, route=_lib.ROUTE_ONE_PASS)
    assert _lib.forward_backward_plan(prob)[0] > 0  # also with a hidden size that is no multiple of 128
    # H = 2 * N_chunk_size: the lower halves of a 16-bit dW's sums alone are the bound, a byte of each fits
    prob = _lib.make_problem(16384, 8192, 131072, 8192, 131072, 8192, 131072, torch.bfloat16, torch.bfloat16,
                             torch.bfloat16, torch.bfloat16, -1, 1.0, 0.0, 4096, False, route=_lib.ROUTE_ONE_PASS)
    chunks, rows = _lib.forward_backward_plan(prob)
    total = _lib.forward_backward_workspace_bytes(prob)
    assert chunks > 1 and 8192 * 131072 + rows * 131072 * 2 <= total <= 4096 * 131072 * 4 < 8192 * 131072 * 2 + rows * 131072 * 2
    # a 16-bit dW whose rows are 8 MiB apart or more: its sums over chunks cannot live in it (32-bit offsets over the
    # 256 rows of a tile), so more than one chunk is not planned; an fp32 dW is summed in place and may
    V = 1 << 22
    for dwt, want in ((torch.bfloat16, (0, 1)), (torch.float32, None)):
        prob = _lib.make_problem(8192, 256, V, 256, V, 256, V, torch.bfloat16, torch.bfloat16, torch.bfloat16, dwt, -1, 1.0,
                                 0.0, 1024, False, route=_lib.ROUTE_ONE_PASS)
        chunks = _lib.forward_backward_plan(prob)[0]
        assert (chunks in want) if want else chunks > 1, (dwt, chunks)
    # an fp32 master weight under 16-bit activations: one 16-bit copy of all of it in the workspace, and its fp32 gradient
    # is summed over the chunks in the caller's buffer (no plane)
    kw = dict(N=8192, H=1024, V=32768, ldx=1024, ldw=32768, lddx=1024, lddw=32768, x_dtype=torch.bfloat16,
              dx_dtype=torch.bfloat16, ignore_index=-1, logit_scale=1.0, z_reg=0.0, n_chunk=2048, monitoring=False,
              route=_lib.ROUTE_ONE_PASS)
    p32 = _lib.make_problem(w_dtype=torch.float32, dw_dtype=torch.float32, **kw)
    p16 = _lib.make_problem(w_dtype=torch.bfloat16, dw_dtype=torch.bfloat16, **kw)
    p16_32 = _lib.make_problem(w_dtype=torch.bfloat16, dw_dtype=torch.float32, **kw)
    c32, r32 = _lib.forward_backward_plan(p32)
    c16, r16 = _lib.forward_backward_plan(p16)
    c1632, r1632 = _lib.forward_backward_plan(p16_32)
    assert c32 > 1 and c16 > 1 and c1632 > 1
    sums, copy = 1024 * 32768, 1024 * 32768 * 2  # (a 16-bit dW: at least a byte per sum in the workspace)
    assert r1632 >= r16  # without them there is room for chunks at least as long
    assert _lib.forward_backward_workspace_bytes(p32) >= copy + r32 * 32768 * 2
    assert _lib.forward_backward_workspace_bytes(p16) >= sums + r16 * 32768 * 2
    # LCE_ROUTE_EXACT_SUMS: two bytes per sum there (the upper halves lie in dW), or no plan
    p16x = _lib.make_problem(w_dtype=torch.bfloat16, dw_dtype=torch.bfloat16, **dict(kw, route=_lib.ROUTE_ONE_PASS | _lib.ROUTE_EXACT_SUMS))
    c16x, r16x = _lib.forward_backward_plan(p16x)
    assert c16x == 0 or (r16x <= r16 and _lib.forward_backward_workspace_bytes(p16x) >= 2 * sums + r16x * 32768 * 2)
    # the flag goes with every route and with nothing else
    for r in (0, 1, 2, 4, 5, 6):
        assert lib.lce_check_problem(ctypes.byref(_lib.make_problem(**dict(kw, w_dtype=torch.bfloat16, dw_dtype=torch.bfloat16, route=r)))) == 0
    for r in (3, 7, 8, -1):
        assert lib.lce_check_problem(ctypes.byref(_lib.make_problem(**dict(kw, w_dtype=torch.bfloat16, dw_dtype=torch.bfloat16, route=r)))) == _lib.LCE_EINVAL_ARG


def test_plans_of_the_benchmark_configurations(lib):
    """What lce_forward_backward plans, by itself, for the benchmark's configurations (host-side only): the headline shape
    in four chunks of 4096 rows with exact fp32 sums of dW; config 3 and every point of config 4 on the one-pass route
    within their bounds; config 5 (fp32 master weight, fp32 dW) in ten chunks; config 1 (fp32 tensors) on two passes."""
    from linear_cross_entropy_loss_amd import _lib

    bf, fh, f32 = torch.bfloat16, torch.float16, torch.float32

    def plan(N, H, V, n_chunk, xd, wd, mon=False, route=_lib.ROUTE_AUTO):
        p = _lib.make_problem(N, H, V, H, V, H, V, xd, wd, xd, wd, -1, 1.0, 0.0, n_chunk, mon, route=route)
        return _lib.forward_backward_plan(p), _lib.forward_backward_workspace_bytes(p)

    (chunks, rows), ws = plan(16384, 2048, 131072, 4096, bf, bf)
    assert (chunks, rows) == (4, 4096) and 2048 * 131072 * 2 + 4096 * 131072 * 2 <= ws <= 4096 * 131072 * 4
    assert plan(16384, 2048, 131072, 4096, bf, bf, route=_lib.ROUTE_AUTO | _lib.ROUTE_EXACT_SUMS)[0] == (4, 4096)
    (chunks, rows), ws = plan(16384, 4096, 131072, 4096, fh, fh, mon=True)
    assert (chunks, rows) == (4, 4096) and ws <= 4096 * 131072 * 4
    (chunks, rows), _ = plan(16384, 4096, 131072, 4096, fh, fh, mon=True, route=_lib.ROUTE_AUTO | _lib.ROUTE_EXACT_SUMS)
    assert chunks > 4 and rows < 4096  # (exact sums: two bytes per sum in the workspace leave shorter chunks)
    for V in (32768, 65536, 131072, 262144):
        for n_chunk in (2048, 4096, 8192):
            (chunks, rows), ws = plan(16384, 2048, V, n_chunk, bf, bf)
            assert chunks >= 1 and chunks * rows >= 16384 and ws <= n_chunk * V * 4, (V, n_chunk, chunks, rows, ws)
    (chunks, rows), ws = plan(65536, 8192, 262144, 8192, fh, f32)
    assert chunks == 10 and ws <= 8192 * 262144 * 4
    assert plan(2048, 2048, 16384, 4096, f32, f32)[0] == (0, 0)

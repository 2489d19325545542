"""ctypes binding of liblce_gfx950.so (the C ABI declared in include/lce.h)."""
from __future__ import annotations

import ctypes
from pathlib import Path

import torch

_PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = _PKG_DIR / "liblce_gfx950.so"

LCE_BF16, LCE_F16, LCE_F32 = 0, 1, 2
LCE_OK = 0
PHASE_FWD_TILES, PHASE_FWD_REDUCE, PHASE_BWD_DZ, PHASE_BWD_DX, PHASE_BWD_DW, PHASE_PACK = 1, 2, 4, 8, 16, 32
PACK_AUTO, PACK_ALWAYS, PACK_NEVER = 0, 1, 2
ROUTE_AUTO, ROUTE_ONE_PASS, ROUTE_TWO_PASS = 0, 1, 2  # lce_problem.route (lce_forward_backward)
ROUTE_EXACT_SUMS = 4  # a flag for the same field: dW's sums over chunks never at fewer than 32 bits
W_HV, W_VH = 0, 1  # lce_problem.w_layout: weight stored (H, V) / (V, H) row-major
LCE_EINVAL_SHAPE, LCE_EINVAL_DTYPE, LCE_EINVAL_ARG, LCE_EWORKSPACE, LCE_EHIP, LCE_ESTATIC = -1, -2, -3, -4, -5, -6
STATIC_SCRATCH_BYTES = 64 << 20

EXPORTS = (
    "lce_version",
    "lce_strerror",
    "lce_last_hip_error",
    "lce_check_problem",
    "lce_workspace_bytes",
    "lce_backward_plan",
    "lce_forward",
    "lce_forward_static",
    "lce_backward",
    "lce_forward_backward_workspace_bytes",
    "lce_forward_backward_plan",
    "lce_forward_backward",
    "lce_scale",
)

_DTYPES = {torch.bfloat16: LCE_BF16, torch.float16: LCE_F16, torch.float32: LCE_F32}


class LceProblem(ctypes.Structure):
    """Mirror of ``struct lce_problem``."""

    _fields_ = [
        ("N", ctypes.c_int64),
        ("H", ctypes.c_int64),
        ("V", ctypes.c_int64),
        ("ldx", ctypes.c_int64),
        ("ldw", ctypes.c_int64),
        ("lddx", ctypes.c_int64),
        ("lddw", ctypes.c_int64),
        ("x_dtype", ctypes.c_int32),
        ("w_dtype", ctypes.c_int32),
        ("dx_dtype", ctypes.c_int32),
        ("dw_dtype", ctypes.c_int32),
        ("ignore_index", ctypes.c_int64),
        ("logit_scale", ctypes.c_float),
        ("z_reg", ctypes.c_float),
        ("n_chunk", ctypes.c_int64),
        ("monitoring", ctypes.c_int32),
        ("phases", ctypes.c_int32),
        ("pack_rows", ctypes.c_int32),
        ("max_workgroups", ctypes.c_int32),
        ("w_layout", ctypes.c_int32),
        ("route", ctypes.c_int32),
    ]


_lib = None


def load():
    """Load the shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension has not been built. "
            "Run `python -m linear_cross_entropy_loss_amd.build` (needs hipcc; no GPU required to build). "
            "There is no fallback path."
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    P = ctypes.POINTER(LceProblem)
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    lib.lce_version.restype = ctypes.c_int
    lib.lce_version.argtypes = []
    lib.lce_strerror.restype = ctypes.c_char_p
    lib.lce_strerror.argtypes = [ctypes.c_int]
    lib.lce_last_hip_error.restype = ctypes.c_char_p
    lib.lce_last_hip_error.argtypes = []
    lib.lce_check_problem.restype = ctypes.c_int
    lib.lce_check_problem.argtypes = [P]
    lib.lce_workspace_bytes.restype = ctypes.c_int
    lib.lce_workspace_bytes.argtypes = [P, ctypes.POINTER(sz), ctypes.POINTER(sz)]
    lib.lce_backward_plan.restype = ctypes.c_int
    lib.lce_backward_plan.argtypes = [P, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]
    lib.lce_forward.restype = ctypes.c_int
    lib.lce_forward.argtypes = [P, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    lib.lce_forward_static.restype = ctypes.c_int
    lib.lce_forward_static.argtypes = [P, vp, vp, vp, vp, vp, vp, vp]
    lib.lce_backward.restype = ctypes.c_int
    lib.lce_backward.argtypes = [P, vp, vp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    lib.lce_forward_backward_workspace_bytes.restype = ctypes.c_int
    lib.lce_forward_backward_workspace_bytes.argtypes = [P, ctypes.POINTER(sz)]
    lib.lce_forward_backward_plan.restype = ctypes.c_int
    lib.lce_forward_backward_plan.argtypes = [P, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]
    lib.lce_forward_backward.restype = ctypes.c_int
    lib.lce_forward_backward.argtypes = [P, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    lib.lce_scale.restype = ctypes.c_int
    lib.lce_scale.argtypes = [vp, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, vp, vp]
    _lib = lib
    return lib


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise ValueError(f"unsupported dtype {dt}; expected bfloat16, float16 or float32") from None


def raise_for_status(rc: int, what: str) -> None:
    """Map a negative lce_status to the exception the reference raises for the same condition."""
    if rc == LCE_OK:
        return
    lib = load()
    msg = lib.lce_strerror(rc).decode()
    if rc == LCE_EHIP:
        raise RuntimeError(f"{what}: {msg}: {lib.lce_last_hip_error().decode()}")
    if rc == LCE_EINVAL_SHAPE:
        # the reference raises ValueError("Provided shape outside the range of valid configs.")
        raise ValueError(f"{what}: Provided shape outside the range of valid configs: {msg}")
    if rc in (LCE_EINVAL_DTYPE, LCE_EINVAL_ARG):
        raise ValueError(f"{what}: {msg}")
    raise RuntimeError(f"{what}: {msg}")


def make_problem(N, H, V, ldx, ldw, lddx, lddw, x_dtype, w_dtype, dx_dtype, dw_dtype, ignore_index,
                 logit_scale, z_reg, n_chunk, monitoring, phases=0, pack_rows=0, max_workgroups=0,
                 w_layout=0, route=0) -> LceProblem:
    return LceProblem(
        N=N, H=H, V=V, ldx=ldx, ldw=ldw, lddx=lddx, lddw=lddw,
        x_dtype=dtype_code(x_dtype), w_dtype=dtype_code(w_dtype),
        dx_dtype=dtype_code(dx_dtype), dw_dtype=dtype_code(dw_dtype),
        ignore_index=int(ignore_index), logit_scale=float(logit_scale), z_reg=float(z_reg),
        n_chunk=int(n_chunk), monitoring=1 if monitoring else 0, phases=int(phases), pack_rows=int(pack_rows),
        max_workgroups=int(max_workgroups), w_layout=int(w_layout), route=int(route),
    )


def workspace_bytes(prob: LceProblem) -> tuple[int, int]:
    lib = load()
    f, b = ctypes.c_size_t(0), ctypes.c_size_t(0)
    raise_for_status(lib.lce_workspace_bytes(ctypes.byref(prob), ctypes.byref(f), ctypes.byref(b)),
                     "lce_workspace_bytes")
    return int(f.value), int(b.value)


def backward_plan(prob: LceProblem) -> tuple[int, int]:
    """(number of vocabulary slabs, slab width) lce_backward will use for `prob`."""
    lib = load()
    n, w = ctypes.c_int64(0), ctypes.c_int64(0)
    raise_for_status(lib.lce_backward_plan(ctypes.byref(prob), ctypes.byref(n), ctypes.byref(w)), "lce_backward_plan")
    return int(n.value), int(w.value)


def forward_backward_workspace_bytes(prob: LceProblem) -> int:
    lib = load()
    b = ctypes.c_size_t(0)
    raise_for_status(lib.lce_forward_backward_workspace_bytes(ctypes.byref(prob), ctypes.byref(b)),
                     "lce_forward_backward_workspace_bytes")
    return int(b.value)


def forward_backward_plan(prob: LceProblem) -> tuple[int, int]:
    """(chunks of token rows, rows per chunk) of lce_forward_backward's single pass over the logits for `prob`;
    (0, 0) when the call would run lce_forward and lce_backward one after the other instead."""
    lib = load()
    n, r = ctypes.c_int64(0), ctypes.c_int64(0)
    raise_for_status(lib.lce_forward_backward_plan(ctypes.byref(prob), ctypes.byref(n), ctypes.byref(r)),
                     "lce_forward_backward_plan")
    return int(n.value), int(r.value)

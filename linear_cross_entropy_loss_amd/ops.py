"""Host side of the fused linear + cross-entropy operator for MI355X.

Mirrors the public interface of the reference's ``linear_cross_entropy/ops.py``:

* ``LinearXentImplementation``  -- ``ops.py:661-810`` (autograd Function, same
  positional arguments, same 5-tuple, last four outputs non-differentiable)
* ``linear_cross_entropy``      -- ``ops.py:814-826``
* ``LinearCrossEntropyLoss``    -- ``ops.py:830-955`` (transposed ``(in, out)``
  weight, no bias, ``monitoring`` / ``latest_metrics``)

The device work is done by hand-written gfx950 kernels behind the C ABI of
``liblce_gfx950.so``; torch only supplies device memory and the stream.

When a gradient is wanted, ``forward`` computes it along with the loss from one
evaluation of the logits (``lce_forward_backward``), as the reference's forward
does (``ops.py:721-791``), and ``backward`` multiplies the upstream gradient in
(``ops.py:810``).  Problems that route does not cover (fp32 activations,
shapes whose scratch bound leaves no room for it) and forward-only calls compute
only the loss in ``forward`` and save ``lse``; their ``backward`` recomputes the
logit tiles (``lce_backward``).  So does a second ``backward`` over the same graph.
"""
from __future__ import annotations

import contextvars
import ctypes
import math
import warnings

import torch

from . import _lib

# Kept for import compatibility with the reference package, which exposes its
# Triton autotune lists under these names (linear_cross_entropy/__init__.py:1).
# The gfx950 kernels use one fixed tile configuration; the lists are inert.
fwd_configs: list = []
bwd_configs: list = []

# Whether tokens whose label is ignore_index are packed away on the device before the tile kernels run:
# _lib.PACK_AUTO (the library decides by problem size: the pre-pass costs about 0.04 ms per step, which
# a small problem does not earn back), _lib.PACK_ALWAYS or _lib.PACK_NEVER.  Results do not depend on it
# beyond the summation order of dW and of the loss.  A context variable: `pack_rows.set(mode)` affects the
# calling thread / task only (reset with the token it returns); the value seen by a forward call is carried
# to its backward, which autograd may run on another thread.
pack_rows: contextvars.ContextVar = contextvars.ContextVar("lce_pack_rows", default=_lib.PACK_AUTO)


# Whether a forward that needs gradients computes them in the same pass over the logits (see the module
# docstring): True -- where the library's model of its kernels says that this is the faster route (lce_problem.route
# = LCE_ROUTE_AUTO); "always" -- wherever the route fits the scratch bound; False -- never: every call takes the
# loss-only forward and the recomputing backward.
one_pass: contextvars.ContextVar = contextvars.ContextVar("lce_one_pass", default=True)

# On the one-pass route a 16-bit dW is summed over chunks of token rows in fp32 where that fits the scratch bound and
# leaves room for chunks long enough; elsewhere the sums are kept at 24 bits between chunks (16 of mantissa, rounded to
# nearest: include/lce.h).  True here rules the 24 bits out (LCE_ROUTE_EXACT_SUMS): such problems then run with shorter
# chunks or take two passes.  Read when the device call is made.
exact_dw_sums: contextvars.ContextVar = contextvars.ContextVar("lce_exact_dw_sums", default=False)


@torch.compiler.assume_constant_result
def _pack_mode() -> int:
    """Current value of `pack_rows`; while torch.compile traces, the value at trace time is baked into the graph."""
    return int(pack_rows.get())


@torch.compiler.assume_constant_result
def _route_mode() -> int:
    """Current value of `one_pass` as a number (0: False, 1: True, 2: "always"); baked into a traced graph like the
    packing mode."""
    v = one_pass.get()
    return 2 if v == "always" else (1 if v else 0)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _row_multiple(dtype):
    """Row strides must keep rows 16-byte aligned: 8 elements for 16-bit data, 4 for float32."""
    return 4 if dtype == torch.float32 else 8


_copy_warned = set()


def _warn_copy_once(what, t, why):
    """One warning per kind of copy: a weight that cannot be read in place is copied on every call (forward and
    backward), which costs its size in memory and a pass over it in time."""
    if what in _copy_warned or torch.compiler.is_compiling():
        return
    _copy_warned.add(what)
    warnings.warn(
        f"linear_cross_entropy: the {what} of shape {tuple(t.shape)}, strides {tuple(t.stride())}, {t.dtype} cannot be "
        f"read in place ({why}) and is copied on every call ({t.numel() * t.element_size() / 2**20:.0f} MiB)",
        stacklevel=3,
    )


def _aligned_rows(t, what=None):
    """`t` itself when the kernels can read it in place, else a copy whose row stride is padded with zeros.

    The kernels take any number of rows and columns, but rows must start on 16-byte boundaries.  Only a
    matrix whose row length is not a multiple of 8 (16-bit) / 4 (fp32) elements AND is stored densely needs
    the copy; padding the vocabulary or hidden size of the model to a multiple of 8 avoids it.
    """
    m = _row_multiple(t.dtype)
    if t.stride(-1) == 1 and t.stride(0) % m == 0 and t.stride(0) >= t.shape[1] and t.data_ptr() % 16 == 0:
        return t
    if what is not None:
        _warn_copy_once(what, t, f"rows must be contiguous and start on 16-byte boundaries: row strides that are "
                                 f"multiples of {m} elements")
    rows, cols = t.shape
    padded = torch.zeros((rows, -(-cols // m) * m), dtype=t.dtype, device=t.device)
    padded[:, :cols] = t
    return padded[:, :cols]


def _weight_layout(At, x_dtype):
    """_lib.W_VH when `At` (H, V) is the transposed view of a row-major (V, H) matrix -- a tied embedding or
    an ``nn.Linear(H, V)`` weight handed over as ``weight.T`` -- that the kernels can read in place, as the
    reference's kernels do through At's strides (ops.py:733-734); else _lib.W_HV.  Decided from shape,
    strides and dtypes alone, so that a traced (fake) tensor gives the same answer."""
    H, V = At.shape
    m = _row_multiple(At.dtype)
    if At.stride(1) == 1 and At.stride(0) % m == 0 and At.stride(0) >= V:
        return _lib.W_HV  # row-major (H, V): read in place
    if (x_dtype != torch.float32 and H % 8 == 0 and V > 1 and At.stride(0) == 1 and At.stride(1) % m == 0
            and At.stride(1) >= H):
        return _lib.W_VH
    return _lib.W_HV  # any other striding: copied into a row-major (H, V) matrix


def _weight_rows(At, layout):
    """The matrix the kernels read: (H, V) rows for W_HV, (V, H) rows for W_VH (no copy unless misaligned)."""
    if layout == _lib.W_VH:
        w = At.t()
        if w.data_ptr() % 16 == 0:
            return w
        _warn_copy_once("weight", At, "its first element is not on a 16-byte boundary")
        return w.clone(memory_format=torch.contiguous_format)
    return _aligned_rows(At, "weight")


def _empty_rows(rows, cols, dtype, device):
    """Uninitialised (rows, cols) matrix whose row stride satisfies the kernels' alignment rule."""
    m = 8  # gradients are stored in pieces of up to 8 elements
    return torch.empty((rows, -(-cols // m) * m), dtype=dtype, device=device)[:, :cols]


def _autocast_x(x, At):
    """Under autocast the activations take the 16-bit type the weight already has, or -- fp32 master weight,
    which is not copied -- the autocast dtype.  (The reference casts x and the whole weight to fp16, ops.py:665.)"""
    if not torch.is_autocast_enabled("cuda"):
        return x
    target = At.dtype if At.dtype in (torch.float16, torch.bfloat16) else torch.get_autocast_dtype("cuda")
    return x if x.dtype == target else x.to(target)


def _check_inputs(x, y, At):
    if not (x.is_cuda and y.is_cuda and At.is_cuda):
        raise RuntimeError(
            "linear_cross_entropy needs its tensors on an AMD GPU (device type 'cuda' under ROCm); "
            "there is no CPU path"
        )
    if y.dtype != torch.int64:
        raise ValueError("labels must be a torch.long tensor")
    if At.dim() != 2:
        raise ValueError("weight must be 2-D with shape (in_features, out_features)")


def _check_dtypes(x, At):
    if x.dtype != At.dtype and not (At.dtype == torch.float32 and x.dtype in (torch.float16, torch.bfloat16)):
        raise ValueError(
            f"input is {x.dtype} but the weight is {At.dtype}: they must share a dtype, or the weight may be a "
            "float32 master weight under 16-bit activations (under torch.autocast the input is cast for you)")


def _problem_views(x_in, y, At):
    """The (x, y, w) views the kernels read, w's layout, and the shapes (N, H, V)."""
    _check_inputs(x_in, y, At)
    _check_dtypes(x_in, At)
    x = _aligned_rows(x_in.reshape(-1, x_in.shape[-1]))
    y1 = y.reshape(-1).contiguous()
    N, H = x.shape
    H_A, V = At.shape
    if H_A != H:
        raise ValueError(f"weight has in_features={H_A}, input has {H}")
    if y1.shape != (N,):
        raise ValueError("labels must have one entry per input row")
    layout = _weight_layout(At, x.dtype)
    w = _weight_rows(At, layout)
    return x, y1, w, layout, N, H, V


def _alloc_grads(x, w, layout, N, H, V, need_dx, need_dw):
    vh = layout == _lib.W_VH
    dx = _empty_rows(N, H, x.dtype, x.device) if need_dx else None
    dw = (_empty_rows(V, H, w.dtype, x.device) if vh else _empty_rows(H, V, w.dtype, x.device)) if need_dw else None
    return dx, dw


def _finish_grads(dx, dw, layout):
    if dx is not None and not dx.is_contiguous():
        dx = dx.contiguous()  # H not a multiple of 8
    if dw is not None and not dw.is_contiguous():
        dw = dw.contiguous()  # V not a multiple of 8
    if dw is not None and layout == _lib.W_VH:
        dw = dw.t()
    return dx, dw


def _stand_in_gradient(x, y1, ignore_index):
    """The upstream gradient that gradients are formed for before the real one is known: 1 for bf16 / fp32 ones.  fp16
    ones would fall below fp16's normal range on the way (entries of order 1/n_valid; a loss scale arrives too late to
    save them): they are formed for the largest power of two that is not above the number of valid labels -- entries
    of the order of the per-token gradient -- and divided by it again when the real one is multiplied in."""
    if x.dtype == torch.float16:
        return torch.exp2(torch.floor(torch.log2((y1 != ignore_index).sum().clamp(min=1).to(torch.float32)))).reshape(1)
    return torch.ones(1, dtype=torch.float32, device=x.device)


def _one_pass_impl(x_in, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, monitoring, pack, need_dx,
                   need_dw, always=None):
    """Runs lce_forward_backward when its one-pass route covers the problem.  Returns None otherwise, else
    (out5, lse, n_valid, x, y1, w, layout, dx, dw, pre): the gradients for an upstream gradient of `pre` (a device
    scalar; None stands for 1).  `always`: take the route wherever it fits (default: what `one_pass` says)."""
    if always is None:
        always = one_pass.get() == "always"
    with torch.cuda.device(x_in.device):
        x, y1, w, layout, N, H, V = _problem_views(x_in, y, At)
        if x.dtype == torch.float32 or w.dtype not in (x.dtype, torch.float32):
            return None
        vh = layout == _lib.W_VH
        w_cols = H if vh else V
        prob = _lib.make_problem(
            N, H, V, x.stride(0), w.stride(0), H + (-H) % 8, w_cols + (-w_cols) % 8, x.dtype, w.dtype, x.dtype, w.dtype,
            ignore_index, logit_scale, z_regularization, N_chunk_size, monitoring, 0, pack, 0, layout,
            (_lib.ROUTE_ONE_PASS if always else _lib.ROUTE_AUTO) | (_lib.ROUTE_EXACT_SUMS if exact_dw_sums.get() else 0),
        )
        lib = _lib.load()
        _lib.raise_for_status(lib.lce_check_problem(ctypes.byref(prob)), "linear_cross_entropy")
        if _lib.forward_backward_plan(prob)[0] == 0:
            return None
        dev = x.device
        dx, dw = _alloc_grads(x, w, layout, N, H, V, need_dx, need_dw)
        nbytes = _lib.forward_backward_workspace_bytes(prob)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        lse = torch.empty(N, dtype=torch.float32, device=dev)
        out5 = torch.empty(5, dtype=torch.float32, device=dev)
        n_valid = torch.empty(1, dtype=torch.int64, device=dev)
        pre = _stand_in_gradient(x, y1, ignore_index)  # (the upstream gradient is not known yet)
        stream = torch.cuda.current_stream(dev).cuda_stream
        rc = lib.lce_forward_backward(ctypes.byref(prob), _ptr(x), _ptr(w), _ptr(y1), _ptr(pre), _ptr(lse), _ptr(out5),
                                      _ptr(n_valid), _ptr(dx), _ptr(dw), _ptr(ws), nbytes, ctypes.c_void_p(stream))
        _lib.raise_for_status(rc, "lce_forward_backward")
        del ws
    return out5, lse, n_valid, x, y1, w, layout, dx, dw, (pre if x.dtype == torch.float16 else None)


def _scale_grad(t, grad_output):
    """t *= grad_output in place, the product formed in fp32 (nothing is touched when grad_output is 1)."""
    if t is None:
        return
    lib = _lib.load()
    with torch.cuda.device(t.device):
        g = grad_output.detach().to(device=t.device, dtype=torch.float32).reshape(1).contiguous()
        stream = torch.cuda.current_stream(t.device).cuda_stream
        rc = lib.lce_scale(_ptr(t), _lib.dtype_code(t.dtype), t.shape[0], t.shape[1], t.stride(0), _ptr(g),
                           ctypes.c_void_p(stream))
        _lib.raise_for_status(rc, "lce_scale")


def _forward_impl(x_in, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, monitoring, pack):
    """Runs lce_forward.  Returns (out5, lse, n_valid), the (x, y, w) views the kernels read and w's layout."""
    _check_inputs(x_in, y, At)
    _check_dtypes(x_in, At)
    with torch.cuda.device(x_in.device):
        x = _aligned_rows(x_in.reshape(-1, x_in.shape[-1]))
        y1 = y.reshape(-1).contiguous()
        N, H = x.shape
        H_A, V = At.shape
        if H_A != H:
            raise ValueError(f"weight has in_features={H_A}, input has {H}")
        if y1.shape != (N,):
            raise ValueError("labels must have one entry per input row")
        layout = _weight_layout(At, x.dtype)
        w = _weight_rows(At, layout)
        lddw = (H if layout == _lib.W_VH else V + (-V) % 8)  # (not used by the forward)
        prob = _lib.make_problem(
            N, H, V, x.stride(0), w.stride(0), H + (-H) % 8, lddw, x.dtype, w.dtype, x.dtype, w.dtype,
            ignore_index, logit_scale, z_regularization, N_chunk_size, monitoring, 0, pack, 0, layout,
        )
        lib = _lib.load()
        _lib.raise_for_status(lib.lce_check_problem(ctypes.byref(prob)), "linear_cross_entropy")
        fwd_bytes, _ = _lib.workspace_bytes(prob)
        dev = x.device
        ws = torch.empty(fwd_bytes, dtype=torch.uint8, device=dev)
        lse = torch.empty(N, dtype=torch.float32, device=dev)
        out5 = torch.empty(5, dtype=torch.float32, device=dev)
        n_valid = torch.empty(1, dtype=torch.int64, device=dev)
        stream = torch.cuda.current_stream(dev).cuda_stream
        rc = lib.lce_forward(ctypes.byref(prob), _ptr(x), _ptr(w), _ptr(y1), _ptr(lse), _ptr(out5),
                             _ptr(n_valid), _ptr(ws), fwd_bytes, ctypes.c_void_p(stream))
        _lib.raise_for_status(rc, "lce_forward")
        del ws
    return out5, lse, n_valid, x, y1, w, layout


def _backward_impl(x, y1, w, lse, n_valid, grad_output, ignore_index, z_regularization, logit_scale,
                   N_chunk_size, need_dx, need_dw, pack, layout=0):
    """Runs lce_backward on what _forward_impl returned.  dx is (N, H); dw is (H, V) -- for a weight stored
    (V, H) (layout W_VH) the transposed view of a gradient stored the same way; None when not needed."""
    N, H = x.shape
    vh = layout == _lib.W_VH
    V = w.shape[0] if vh else w.shape[1]
    w_cols = H if vh else V
    with torch.cuda.device(x.device):
        dev = x.device
        dx = _empty_rows(N, H, x.dtype, dev) if need_dx else None
        dw = (_empty_rows(V, H, w.dtype, dev) if vh else _empty_rows(H, V, w.dtype, dev)) if need_dw else None
        if need_dx or need_dw:
            prob = _lib.make_problem(
                N, H, V, x.stride(0), w.stride(0), dx.stride(0) if need_dx else H + (-H) % 8,
                dw.stride(0) if need_dw else w_cols + (-w_cols) % 8, x.dtype, w.dtype, x.dtype, w.dtype,
                ignore_index, logit_scale, z_regularization, N_chunk_size, False, 0, pack, 0, layout,
            )
            lib = _lib.load()
            _, bwd_bytes = _lib.workspace_bytes(prob)
            ws = torch.empty(bwd_bytes, dtype=torch.uint8, device=dev)
            g = grad_output.detach().to(device=dev, dtype=torch.float32).reshape(1).contiguous()
            stream = torch.cuda.current_stream(dev).cuda_stream
            rc = lib.lce_backward(ctypes.byref(prob), _ptr(x), _ptr(w), _ptr(y1), _ptr(lse), _ptr(n_valid),
                                  _ptr(g), _ptr(dx), _ptr(dw), _ptr(ws), bwd_bytes, ctypes.c_void_p(stream))
            _lib.raise_for_status(rc, "lce_backward")
            del ws
    if dx is not None and not dx.is_contiguous():
        dx = dx.contiguous()  # H not a multiple of 8
    if dw is not None and not dw.is_contiguous():
        dw = dw.contiguous()  # V not a multiple of 8
    if dw is not None and vh:
        dw = dw.t()
    return dx, dw


class LinearXentImplementation(torch.autograd.Function):
    """The reference's autograd Function (``ops.py:661-810``): same arguments, same 5-tuple."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(
        ctx,
        x_in,
        y,
        At,
        ignore_index=-100,
        z_regularization: float = 0.0,
        logit_scale: float = 1.0,
        N_chunk_size: int = 4096,
        monitoring: bool = True,
    ):
        # Under autocast the activations take the weight's 16-bit type or the autocast dtype; a float32 weight
        # is NOT copied: the library rounds the fp32 master weight one vocabulary slab at a time, inside its
        # workspace.
        x_in = _autocast_x(x_in, At)
        pack = _pack_mode()
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[2]
        done = None
        if (need_dx or need_dw) and one_pass.get():
            done = _one_pass_impl(x_in, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, monitoring, pack,
                                  need_dx, need_dw)
        if done is not None:
            out5, lse, n_valid, x, y1, w, layout, dx, dw, pre = done
            ctx.lce_grads = [dx, dw, pre]  # for the first backward; dropped there
        else:
            out5, lse, n_valid, x, y1, w, layout = _forward_impl(
                x_in, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, monitoring, pack)
            ctx.lce_grads = None
        ctx.save_for_backward(x, y1, w, lse, n_valid)
        ctx.lce_cfg = (ignore_index, z_regularization, logit_scale, N_chunk_size, pack, layout)
        ctx.x_shape = x_in.shape
        loss, z_reg, logit_max, logit_ent, logit_norm = out5.unbind(0)
        ctx.mark_non_differentiable(z_reg, logit_max, logit_ent, logit_norm)
        return loss, z_reg, logit_max, logit_ent, logit_norm

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output, void0=None, void1=None, void2=None, void3=None):
        x, y1, w, lse, n_valid = ctx.saved_tensors
        ignore_index, z_regularization, logit_scale, N_chunk_size, pack, layout = ctx.lce_cfg
        grads, ctx.lce_grads = ctx.lce_grads, None
        if grads is not None:
            # computed in the forward for an upstream gradient of 1 (ops.py:810 does the same multiplication); a
            # later backward over the same graph finds nothing here and recomputes
            dx, dw, pre = grads
            factor = grad_output.detach().to(torch.float32) if pre is None else grad_output.detach().to(torch.float32) / pre
            _scale_grad(dx, factor)
            _scale_grad(dw, factor)
            dx, dw = _finish_grads(dx, dw, layout)
        else:
            dx, dw = _backward_impl(x, y1, w, lse, n_valid, grad_output, ignore_index, z_regularization, logit_scale,
                                    N_chunk_size, ctx.needs_input_grad[0], ctx.needs_input_grad[2], pack, layout)
        if dx is not None:
            dx = dx.view(ctx.x_shape)
        return dx, None, dw, None, None, None, None, None


# ---------------------------------------------------------------------------------------------------------
# torch.library registration: the same two device calls as opaque operators with fake (shape-only)
# implementations and an autograd formula, so that torch.compile / torch.export can trace through a
# model that ends in this loss without touching the ctypes calls.  (The reference leaves
# `torch._dynamo.disable` commented out on its Function, ops.py:664, and hard-codes fp16 autocast,
# ops.py:665-667; here autocast follows the active autocast dtype.)
# ---------------------------------------------------------------------------------------------------------
@torch.library.custom_op("lce_amd::forward", mutates_args=(), device_types="cuda")
def _op_forward(x: torch.Tensor, y: torch.Tensor, At: torch.Tensor, ignore_index: int, z_regularization: float,
                logit_scale: float, N_chunk_size: int, monitoring: bool,
                pack_rows_mode: int = 0) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    out5, lse, n_valid, _, _, _, _ = _forward_impl(x, y, At, ignore_index, z_regularization, logit_scale,
                                                   N_chunk_size, monitoring, pack_rows_mode)
    return out5, lse, n_valid


@_op_forward.register_fake
def _(x, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, monitoring, pack_rows_mode=0):
    n = x.numel() // x.shape[-1]
    return (x.new_empty((5,), dtype=torch.float32), x.new_empty((n,), dtype=torch.float32),
            x.new_empty((1,), dtype=torch.int64))


@torch.library.custom_op("lce_amd::backward", mutates_args=(), device_types="cuda")
def _op_backward(x: torch.Tensor, y: torch.Tensor, At: torch.Tensor, lse: torch.Tensor, n_valid: torch.Tensor,
                 grad_loss: torch.Tensor, ignore_index: int, z_regularization: float, logit_scale: float,
                 N_chunk_size: int, need_dx: bool, need_dw: bool,
                 pack_rows_mode: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
    x2 = _aligned_rows(x.reshape(-1, x.shape[-1]))
    layout = _weight_layout(At, x2.dtype)
    dx, dw = _backward_impl(x2, y.reshape(-1).contiguous(), _weight_rows(At, layout), lse, n_valid, grad_loss,
                            ignore_index, z_regularization, logit_scale, N_chunk_size, need_dx, need_dw,
                            pack_rows_mode, layout)
    dx = dx.view(x.shape) if dx is not None else x.new_empty((0,))
    dw = dw if dw is not None else At.new_empty((0,))
    return dx, dw


@_op_backward.register_fake
def _(x, y, At, lse, n_valid, grad_loss, ignore_index, z_regularization, logit_scale, N_chunk_size, need_dx, need_dw,
      pack_rows_mode=0):
    return _fake_grads(x, At, need_dx, need_dw)


def _op_setup_context(ctx, inputs, output):
    x, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, _, pack = inputs
    _, lse, n_valid = output
    ctx.save_for_backward(x, y, At, lse, n_valid)
    ctx.lce_cfg = (ignore_index, z_regularization, logit_scale, N_chunk_size, pack)


def _op_autograd(ctx, grad_out5, grad_lse, grad_n_valid):
    # Only the loss (entry 0 of the 5 scalars) is differentiable; the monitoring values are treated as
    # constants, as the reference marks them non-differentiable (ops.py:798-800).
    x, y, At, lse, n_valid = ctx.saved_tensors
    ignore_index, z_regularization, logit_scale, N_chunk_size, pack = ctx.lce_cfg
    need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[2]
    dx = dw = None
    if need_dx or need_dw:
        gx, gw = _op_backward(x, y, At, lse, n_valid, grad_out5[0:1].to(torch.float32), ignore_index,
                              z_regularization, logit_scale, N_chunk_size, need_dx, need_dw, pack)
        dx = gx if need_dx else None
        dw = gw if need_dw else None
    return dx, None, dw, None, None, None, None, None, None


_op_forward.register_autograd(_op_autograd, setup_context=_op_setup_context)


# Loss and gradients from one call, for traced graphs whose loss needs a gradient: what LinearXentImplementation does
# in eager mode.  The gradients come out for the stand-in upstream gradient `pre`; the autograd formula multiplies the
# real one in (lce_amd::scale, which returns a new tensor: the saved gradients stay as they are, so the graph can be
# differentiated again).
@torch.library.custom_op("lce_amd::forward_grads", mutates_args=(), device_types="cuda")
def _op_forward_grads(x: torch.Tensor, y: torch.Tensor, At: torch.Tensor, ignore_index: int, z_regularization: float,
                      logit_scale: float, N_chunk_size: int, monitoring: bool, need_dx: bool, need_dw: bool,
                      pack_rows_mode: int = 0, always: bool = False
                      ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_inputs(x, y, At)
    _check_dtypes(x, At)
    done = _one_pass_impl(x, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, monitoring,
                          pack_rows_mode, need_dx, need_dw, always)
    if done is not None:
        out5, lse, n_valid, x2, y1, _, layout, dx, dw, pre = done
        dx, dw = _finish_grads(dx, dw, layout)
        if pre is None:
            pre = torch.ones(1, dtype=torch.float32, device=x.device)
    else:  # (a problem the one-pass route does not cover: the two device calls, one after the other)
        out5, lse, n_valid, x2, y1, w, layout = _forward_impl(x, y, At, ignore_index, z_regularization, logit_scale,
                                                              N_chunk_size, monitoring, pack_rows_mode)
        pre = _stand_in_gradient(x2, y1, ignore_index)
        dx, dw = _backward_impl(x2, y1, w, lse, n_valid, pre, ignore_index, z_regularization, logit_scale, N_chunk_size,
                                need_dx, need_dw, pack_rows_mode, layout)
    dx = dx.view(x.shape) if dx is not None else x.new_empty((0,))
    dw = dw if dw is not None else At.new_empty((0,))
    return out5, lse, n_valid, dx, dw, pre


def _fake_grads(x, At, need_dx, need_dw):
    if not need_dw:
        dw = At.new_empty((0,))
    elif _weight_layout(At, x.dtype) == _lib.W_VH:
        dw = At.new_empty((At.shape[1], At.shape[0])).t()  # stored like the weight: (V, H) rows
    else:
        dw = torch.empty_like(At, memory_format=torch.contiguous_format)
    return (torch.empty_like(x, memory_format=torch.contiguous_format) if need_dx else x.new_empty((0,))), dw


@_op_forward_grads.register_fake
def _(x, y, At, ignore_index, z_regularization, logit_scale, N_chunk_size, monitoring, need_dx, need_dw,
      pack_rows_mode=0, always=False):
    n = x.numel() // x.shape[-1]
    dx, dw = _fake_grads(x, At, need_dx, need_dw)
    return (x.new_empty((5,), dtype=torch.float32), x.new_empty((n,), dtype=torch.float32),
            x.new_empty((1,), dtype=torch.int64), dx, dw, x.new_empty((1,), dtype=torch.float32))


@torch.library.custom_op("lce_amd::scale", mutates_args=(), device_types="cuda")
def _op_scale(t: torch.Tensor, factor: torch.Tensor) -> torch.Tensor:
    """A copy of t (dense, row-major or the transposed view of such a matrix) times factor[0], the product formed in fp32."""
    out = t.clone()
    flat = out.view(-1) if out.is_contiguous() else out.t().view(-1)
    n = flat.numel()
    if n:
        lib = _lib.load()
        with torch.cuda.device(t.device):
            g = factor.detach().to(device=t.device, dtype=torch.float32).reshape(1).contiguous()
            stream = torch.cuda.current_stream(t.device).cuda_stream
            # (one row of n elements: any dense tensor, whatever its row length)
            rc = lib.lce_scale(_ptr(flat), _lib.dtype_code(t.dtype), 1, n, n + (-n) % 8, _ptr(g), ctypes.c_void_p(stream))
            _lib.raise_for_status(rc, "lce_scale")
    return out


@_op_scale.register_fake
def _(t, factor):
    return torch.empty_like(t)


def _fg_setup_context(ctx, inputs, output):
    _, _, _, dx, dw, pre = output
    ctx.save_for_backward(dx, dw, pre)


def _fg_autograd(ctx, grad_out5, grad_lse, grad_n_valid, grad_dx, grad_dw, grad_pre):
    # only the loss (entry 0 of the 5 scalars) is differentiable, as above
    dx, dw, pre = ctx.saved_tensors
    factor = grad_out5[0:1].to(torch.float32) / pre
    gx = _op_scale(dx, factor) if ctx.needs_input_grad[0] else None
    gw = _op_scale(dw, factor) if ctx.needs_input_grad[2] else None
    return gx, None, gw, None, None, None, None, None, None, None, None, None


_op_forward_grads.register_autograd(_fg_autograd, setup_context=_fg_setup_context)


def linear_cross_entropy(
    x,
    y,
    At,
    ignore_index=-100,
    z_regularization: float = 0.0,
    logit_scale: float = 1.0,
    N_chunk_size: int = 4096,
    monitoring: bool = False,
):
    """Functional form (``ops.py:814-826``); returns ``(loss, z_reg, logit_max, logit_entropy, logit_norm)``.

    While ``torch.compile`` / ``torch.export`` trace, the call goes through registered operators, so it can
    sit inside a compiled region: ``torch.ops.lce_amd.forward_grads`` when an input needs a gradient (loss and
    gradients from one evaluation of the logits, the upstream gradient multiplied in by ``lce_amd.scale`` in
    the backward graph), else -- and with ``one_pass`` off at trace time -- ``torch.ops.lce_amd.forward`` (loss
    in the forward, gradients by a backward that recomputes the logit tiles).  In eager mode it goes through
    ``LinearXentImplementation``, which makes the same device calls with about 80 us less dispatch overhead
    per forward+backward and bit-identical results.  Under autocast ``x`` takes the weight's 16-bit dtype, or the autocast
    dtype when the weight is fp32; an fp32 weight is read as is (no 16-bit copy) and gets an fp32 gradient.
    fp32 ``x`` with an fp32 weight (no autocast) is computed as bf16 pairs, accurate to about 1e-5 of the
    largest gradient entry, at three times the matrix work of 16-bit tensors.
    """
    _check_inputs(x, y, At)
    if not torch.compiler.is_compiling():
        loss, z_reg, logit_max, logit_ent, logit_norm = LinearXentImplementation.apply(
            x, y, At, int(ignore_index), float(z_regularization), float(logit_scale), int(N_chunk_size),
            bool(monitoring))
        return loss, z_reg, logit_max, logit_ent, logit_norm
    x = _autocast_x(x, At)
    route = _route_mode()
    need_dx, need_dw = x.requires_grad, At.requires_grad
    if route and torch.is_grad_enabled() and (need_dx or need_dw):
        out5 = _op_forward_grads(x, y, At, int(ignore_index), float(z_regularization), float(logit_scale),
                                 int(N_chunk_size), bool(monitoring), need_dx, need_dw, _pack_mode(), route == 2)[0]
    else:
        out5 = _op_forward(x, y, At, int(ignore_index), float(z_regularization), float(logit_scale),
                           int(N_chunk_size), bool(monitoring), _pack_mode())[0]
    loss, z_reg, logit_max, logit_ent, logit_norm = out5.unbind(0)
    return loss, z_reg.detach(), logit_max.detach(), logit_ent.detach(), logit_norm.detach()


class LinearCrossEntropyLoss(torch.nn.Linear):
    """``loss = cross_entropy(logit_scale * x @ weight, y)`` fused on the GPU.

    An ``nn.Linear`` subclass so that initialisation passes that look for ``nn.Linear`` find it, but the
    weight is stored transposed, ``(in_features, out_features)``, and there is no bias.

    Args:
        in_features: hidden size (any; multiples of 8 avoid a padded copy of the input).
        out_features: vocabulary size / number of classes (any; multiples of 8 avoid a padded copy of
            the weight and of its gradient).  The reference requires multiples of 256 / 4096
            (``ops.py:905-906``); those restrictions are lifted here.
        ignore_index: label value that is skipped. Default -100.
        logit_scale: positive factor applied to the logits before the loss. Default 1.0.
        z_regularization: weight of the ``mean(logsumexp(z)^2)`` penalty. Default 0.0.
        N_chunk_size: bound on the scratch memory, ``N_chunk_size * out_features * 4`` bytes (what the reference spends
            on one chunk of logits).  Where it leaves room, a forward that needs gradients computes them from its one
            evaluation of the logits, in chunks of token rows (16-bit staging of a chunk against the whole vocabulary plus
            an fp32 sum of the weight gradient, ``in_features * out_features * 4`` bytes); otherwise the backward
            recomputes the logits and works through the vocabulary in as many slabs as the bound takes, and the forward
            through the tokens in chunks of ``max(N_chunk_size, 16384)`` rows.  A larger value buys longer chunks (faster)
            at more scratch.  The number of rows of ``x`` is free.  Default 4096.
        init_method: optional callable applied to the weight instead of the default truncated normal.

    Set ``module.monitoring = True`` to also collect ``logit_norm``, ``logit_max``, ``logit_entropy`` and
    ``z_value`` into ``module.latest_metrics`` on every forward.
    """

    def __init__(
        self,
        in_features: int,
        out_features: int,
        device=None,
        dtype=None,
        ignore_index: int = -100,
        logit_scale: float = 1.0,
        z_regularization: float = 0.0,
        N_chunk_size: int = 4096,
        init_method=None,
    ):
        factory_kwargs = {"device": device, "dtype": dtype}
        torch.nn.Module.__init__(self)

        assert in_features > 0 and out_features > 0 and N_chunk_size > 0
        assert logit_scale > 0
        assert z_regularization >= 0

        self.in_features = in_features
        self.out_features = out_features
        self.weight = torch.nn.Parameter(torch.empty((in_features, out_features), **factory_kwargs))

        self.logit_scale = logit_scale
        self.ignore_index = ignore_index
        self.z_regularization = z_regularization
        self.N_chunk_size = N_chunk_size

        self.monitoring = False
        self.latest_metrics = {}
        self.init_method = init_method

        self.reset_parameters()

    def reset_parameters(self) -> None:
        if self.init_method is not None:
            self.init_method(self.weight)
        else:
            std = math.sqrt(1 / self.in_features)
            torch.nn.init.trunc_normal_(self.weight, mean=0.0, std=std, a=-3 * std, b=3 * std)

    def forward(self, x, y):
        loss, z_reg, logit_max, logit_ent, logit_norm = linear_cross_entropy(
            x, y, self.weight, self.ignore_index, self.z_regularization, self.logit_scale,
            self.N_chunk_size, self.monitoring,
        )
        if self.monitoring:
            self.latest_metrics = {
                "logit_norm": logit_norm,
                "logit_max": logit_max,
                "logit_entropy": logit_ent,
                "z_value": z_reg,
            }
        return loss

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, bias=False"

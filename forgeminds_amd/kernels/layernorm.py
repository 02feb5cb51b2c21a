"""``layer_norm`` and ``add_layer_norm``: ``F.layer_norm`` (and its residual-add form) on the
HIP kernels.

The reference ships RMSNorm kernels only (``forgemind/kernels/norm.py``); LayerNorm follows the
same contract here: the call shape of ``rms_norm`` / ``add_rms_norm``
(``kernels/norm.py:1152-1277``), fp32 math on the stored values with one rounding
(``kernels/_fallback.py:15-35``), ``autograd.Function`` eagerly,
``torch.ops.forgemind.{layer_norm,add_layer_norm}`` (+ ``*_backward``) while tracing, and the
torch expression whenever the gate says no.
"""

from __future__ import annotations

import typing

import torch

from . import _fallback as fb
from . import _hip, _ops
from ._common import _note, fast_ok, wants_grad


def _c(t):
    return t if t is None or t.is_contiguous() else t.contiguous()


def _launch_fwd(x, w, b, eps, delta=None):
    return _hip.layernorm_fwd(_c(x), _c(w), _c(b), eps, _c(delta))


def _launch_bwd(x, w, mean, rstd, dy, gxn=None, want_dw=True, want_db=True):
    return _hip.layernorm_bwd(_c(x), _c(w), mean, rstd, _c(dy), _c(gxn), want_dw, want_db)


# ------------------------------------------------------------------ eager: autograd.Function
class _LayerNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, b, eps):
        _, y, mean, rstd = _launch_fwd(x, w, b, eps)
        ctx.save_for_backward(x, w, mean, rstd)
        ctx.has_bias = b is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w, mean, rstd = ctx.saved_tensors
        dx, dw, db = _launch_bwd(x, w, mean, rstd, dy, None, ctx.needs_input_grad[1],
                                 ctx.has_bias and ctx.needs_input_grad[2])
        return dx, dw, db, None


class _AddLayerNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, delta, w, b, eps):
        xn, y, mean, rstd = _launch_fwd(x, w, b, eps, delta)
        ctx.save_for_backward(xn, w, mean, rstd)
        ctx.has_bias = b is not None
        return xn, y

    @staticmethod
    def backward(ctx, gxn, gy):
        xn, w, mean, rstd = ctx.saved_tensors
        if gy is None:            # only the residual output was used downstream
            return gxn, gxn, None, None, None
        dx, dw, db = _launch_bwd(xn, w, mean, rstd, gy, gxn, ctx.needs_input_grad[2],
                                 ctx.has_bias and ctx.needs_input_grad[3])
        # d(x) and d(delta) are the same values; autograd accepts one tensor for both slots
        return dx, dx, dw, db, None


# ------------------------------------------------------------------ traced: custom ops
def _stats_like(x):
    rows = x.numel() // x.shape[-1]
    return (torch.empty(rows, device=x.device, dtype=torch.float32),
            torch.empty(rows, device=x.device, dtype=torch.float32))


def _ln_impl(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor,
             eps: float) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _, y, mean, rstd = _launch_fwd(x, w, b, eps)
    return y, mean.clone(), rstd.clone()      # mean / rstd are two rows of one buffer


def _ln_fake(x, w, b, eps):
    return (torch.empty_like(x),) + _stats_like(x)


def _ln_bwd_impl(x: torch.Tensor, w: torch.Tensor, mean: torch.Tensor, rstd: torch.Tensor,
                 dy: torch.Tensor) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_bwd(x, w, mean, rstd, dy)


def _ln_bwd_fake(x, w, mean, rstd, dy):
    return torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)


def _ln_setup(ctx, inputs, output):
    x, w, _b, _eps = inputs
    ctx.save_for_backward(x, w, output[1], output[2])


def _ln_autograd(ctx, dy, _dmean, _drstd):
    x, w, mean, rstd = ctx.saved_tensors
    dx, dw, db = _LN_BWD_OP(x, w, mean, rstd, dy)
    return dx, dw, db, None


def _addln_impl(x: torch.Tensor, delta: torch.Tensor, w: torch.Tensor, b: torch.Tensor,
                eps: float) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    xn, y, mean, rstd = _launch_fwd(x, w, b, eps, delta)
    return xn, y, mean.clone(), rstd.clone()


def _addln_fake(x, delta, w, b, eps):
    return (torch.empty_like(x), torch.empty_like(x)) + _stats_like(x)


def _addln_bwd_impl(xn: torch.Tensor, w: torch.Tensor, mean: torch.Tensor, rstd: torch.Tensor,
                    gxn: torch.Tensor, gy: torch.Tensor
                    ) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    dx, dw, db = _launch_bwd(xn, w, mean, rstd, gy, gxn)
    return dx, dx.clone(), dw, db      # op outputs may not alias each other


def _addln_bwd_fake(xn, w, mean, rstd, gxn, gy):
    return torch.empty_like(xn), torch.empty_like(xn), torch.empty_like(w), torch.empty_like(w)


def _addln_setup(ctx, inputs, output):
    xn, _y, mean, rstd = output
    ctx.save_for_backward(xn, inputs[2], mean, rstd)


def _addln_autograd(ctx, gxn, gy, _gmean, _grstd):
    xn, w, mean, rstd = ctx.saved_tensors
    if gxn is None:
        gxn = torch.zeros_like(xn)
    if gy is None:
        gy = torch.zeros_like(xn)
    dx, dd, dw, db = _ADDLN_BWD_OP(xn, w, mean, rstd, gxn, gy)
    return dx, dd, dw, db, None


_LN_BWD_OP = _ops.define_backward("layer_norm", _ln_bwd_impl, _ln_bwd_fake)
_ADDLN_BWD_OP = _ops.define_backward("add_layer_norm", _addln_bwd_impl, _addln_bwd_fake)
_LN_OP = _ops.define("layer_norm", _ln_impl, _ln_fake, _ln_setup, _ln_autograd)
_ADDLN_OP = _ops.define("add_layer_norm", _addln_impl, _addln_fake, _addln_setup, _addln_autograd)


# ------------------------------------------------------------------ public entry points
def _ok(x, w, b, *more) -> bool:
    if w is None or x.dim() < 1 or x.shape[-1] == 0 or x.shape[-1] != w.numel():
        _note("norm shape")
        return False
    if b is not None and (b.shape != w.shape or b.dtype != w.dtype):
        _note("norm bias")
        return False
    if x.numel() >= 2 ** 31 * 4:
        _note("norm numel")
        return False
    if not (w.dtype == x.dtype or (w.dtype == torch.float32 and x.dtype in (torch.float16,
                                                                            torch.bfloat16))):
        _note("norm weight dtype")
        return False
    tensors = (x, w) + ((b,) if b is not None else ()) + more
    return fast_ok(*tensors)


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: "torch.Tensor | None" = None,
               eps: float = 1e-5) -> torch.Tensor:
    """``F.layer_norm(x, (x.shape[-1],), w, b, eps)`` in one kernel; torch expression otherwise."""
    if not _ok(x, w, b):
        return fb.layer_norm(x, w, b, eps)
    if _LN_OP is not None and _ops.wanted():
        if b is None:       # the op takes a bias tensor; without one the torch expression is traced
            _note("layer_norm op without bias")
            return fb.layer_norm(x, w, b, eps)
        return _LN_OP(x, w, b, float(eps))[0]
    if not wants_grad(x, w, b):
        return _launch_fwd(x, w, b, float(eps))[1]
    return _LayerNormFn.apply(x, w, b, float(eps))


def add_layer_norm(x: torch.Tensor, delta: torch.Tensor, w: torch.Tensor,
                   b: "torch.Tensor | None" = None, eps: float = 1e-5):
    """``(x + delta, layer_norm(x + delta, w, b, eps))`` with the sum written once."""
    if delta.shape != x.shape or delta.dtype != x.dtype:
        _note("add_layer_norm operands differ")
        return fb.add_layer_norm(x, delta, w, b, eps)
    if not _ok(x, w, b, delta):
        return fb.add_layer_norm(x, delta, w, b, eps)
    if _ADDLN_OP is not None and _ops.wanted():
        if b is None:
            _note("layer_norm op without bias")
            return fb.add_layer_norm(x, delta, w, b, eps)
        xn, y, _mean, _rstd = _ADDLN_OP(x, delta, w, b, float(eps))
        return xn, y
    if not wants_grad(x, delta, w, b):
        return _launch_fwd(x, w, b, float(eps), delta)[:2]
    return _AddLayerNormFn.apply(x, delta, w, b, float(eps))


__all__ = ["layer_norm", "add_layer_norm"]

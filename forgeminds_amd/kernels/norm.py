"""``rms_norm`` and ``add_rms_norm``: drop-ins for ``F.rms_norm`` backed by the HIP kernels.

Call surface and dispatch follow the reference's ``forgemind/kernels/norm.py:1152-1277``:
``autograd.Function`` in eager mode, ``torch.ops.forgemind.{rms_norm,add_rms_norm}`` (+
``*_backward``) while tracing, and the torch expression whenever the gate says no.

Differences from the reference gate (``norm.py:1253-1258``), all widening:
* the weight may be fp32 next to bf16/fp16 activations (the reference fell back to torch
  there; its module wrappers cast the weight down first, ``nn.py:120-124``);
* any row width is accepted (the reference stopped at 8192 columns).
``add_rms_norm`` normalises the *rounded* sum, i.e. it has the rounding points of the
torch expression ``rms_norm(x + delta)`` (reference ``_fallback.py:33-35``), not those of
the reference's fused Triton kernel (``norm.py:1027-1030``).
"""

from __future__ import annotations

import typing

import torch

from . import _fallback as fb
from . import _hip, _ops
from ._common import _note, fast_ok, wants_grad


def _c(t: torch.Tensor) -> torch.Tensor:
    # is_contiguous() is a tenth of the cost of a contiguous() that has nothing to do
    return t if t.is_contiguous() else t.contiguous()


def _launch_rms_fwd(x, w, eps):
    return _hip.rmsnorm_fwd(_c(x), _c(w), eps)


def _launch_rms_bwd(x, w, rstd, dy, want_dw=True):
    return _hip.rmsnorm_bwd(_c(x), _c(w), rstd, _c(dy), want_dw)


def _launch_addrms_fwd(x, delta, w, eps):
    return _hip.add_rmsnorm_fwd(_c(x), _c(delta), _c(w), eps)


def _launch_addrms_bwd(xn, w, rstd, gxn, gy, want_dw=True):
    return _hip.add_rmsnorm_bwd(_c(xn), _c(w), rstd, _c(gy), None if gxn is None else _c(gxn), want_dw)


# ------------------------------------------------------------------ eager: autograd.Function
class _RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, eps):
        y, rstd = _launch_rms_fwd(x, w, eps)
        ctx.save_for_backward(x, w, rstd)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w, rstd = ctx.saved_tensors
        dx, dw = _launch_rms_bwd(x, w, rstd, dy, want_dw=ctx.needs_input_grad[1])
        return dx, dw, None


class _AddRMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, delta, w, eps):
        xn, y, rstd = _launch_addrms_fwd(x, delta, w, eps)
        ctx.save_for_backward(xn, w, rstd)
        return xn, y

    @staticmethod
    def backward(ctx, gxn, gy):
        xn, w, rstd = ctx.saved_tensors
        if gy is None:            # only the residual output was used downstream
            return gxn, gxn, None, None
        dx, dw = _launch_addrms_bwd(xn, w, rstd, gxn, gy, want_dw=ctx.needs_input_grad[2])
        # d(x) and d(delta) are the same values; autograd accepts one tensor for both slots
        return dx, dx, dw, None


# ------------------------------------------------------------------ traced: custom ops
def _rms_impl(x: torch.Tensor, w: torch.Tensor,
              eps: float) -> typing.Tuple[torch.Tensor, torch.Tensor]:
    return _launch_rms_fwd(x, w, eps)


def _rms_fake(x, w, eps):
    rows = x.numel() // x.shape[-1]
    return torch.empty_like(x), torch.empty(rows, device=x.device, dtype=torch.float32)


def _rms_bwd_impl(x: torch.Tensor, w: torch.Tensor, rstd: torch.Tensor,
                  dy: torch.Tensor) -> typing.Tuple[torch.Tensor, torch.Tensor]:
    return _launch_rms_bwd(x, w, rstd, dy, True)


def _rms_bwd_fake(x, w, rstd, dy):
    return torch.empty_like(x), torch.empty_like(w)


def _rms_setup(ctx, inputs, output):
    x, w, _eps = inputs
    ctx.save_for_backward(x, w, output[1])


def _rms_autograd(ctx, dy, _drstd):
    x, w, rstd = ctx.saved_tensors
    dx, dw = _RMS_BWD_OP(x, w, rstd, dy)
    return dx, dw, None


def _addrms_impl(x: torch.Tensor, delta: torch.Tensor, w: torch.Tensor,
                 eps: float) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _launch_addrms_fwd(x, delta, w, eps)


def _addrms_fake(x, delta, w, eps):
    rows = x.numel() // x.shape[-1]
    return (torch.empty_like(x), torch.empty_like(x),
            torch.empty(rows, device=x.device, dtype=torch.float32))


def _addrms_bwd_impl(xn: torch.Tensor, w: torch.Tensor, rstd: torch.Tensor, gxn: torch.Tensor,
                     gy: torch.Tensor) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    dx, dw = _launch_addrms_bwd(xn, w, rstd, gxn, gy, True)
    return dx, dx.clone(), dw      # op outputs may not alias each other


def _addrms_bwd_fake(xn, w, rstd, gxn, gy):
    return torch.empty_like(xn), torch.empty_like(xn), torch.empty_like(w)


def _addrms_setup(ctx, inputs, output):
    xn, _y, rstd = output
    ctx.save_for_backward(xn, inputs[2], rstd)


def _addrms_autograd(ctx, gxn, gy, _grstd):
    xn, w, rstd = ctx.saved_tensors
    if gxn is None:
        gxn = torch.zeros_like(xn)
    if gy is None:
        gy = torch.zeros_like(xn)
    dx, dd, dw = _ADDRMS_BWD_OP(xn, w, rstd, gxn, gy)
    return dx, dd, dw, None


_RMS_BWD_OP = _ops.define_backward("rms_norm", _rms_bwd_impl, _rms_bwd_fake)
_ADDRMS_BWD_OP = _ops.define_backward("add_rms_norm", _addrms_bwd_impl, _addrms_bwd_fake)
_RMS_OP = _ops.define("rms_norm", _rms_impl, _rms_fake, _rms_setup, _rms_autograd)
_ADDRMS_OP = _ops.define("add_rms_norm", _addrms_impl, _addrms_fake, _addrms_setup,
                         _addrms_autograd)


# ------------------------------------------------------------------ public entry points
def _ok(x, w, *more) -> bool:
    if w is None or x.dim() < 1 or x.shape[-1] == 0 or x.shape[-1] != w.numel():
        _note("norm shape")
        return False
    if x.numel() >= 2 ** 31 * 4:
        _note("norm numel")
        return False
    if not (w.dtype == x.dtype or (w.dtype == torch.float32 and x.dtype in (torch.float16,
                                                                            torch.bfloat16))):
        _note("norm weight dtype")
        return False
    return fast_ok(x, w, *more)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``F.rms_norm(x, (x.shape[-1],), w, eps)`` in one kernel; torch expression otherwise."""
    if not _ok(x, w):
        return fb.rms_norm(x, w, eps)
    if _RMS_OP is not None and _ops.wanted():
        return _RMS_OP(x, w, float(eps))[0]
    if not wants_grad(x, w):
        return _launch_rms_fwd(x, w, float(eps))[0]
    return _RMSNormFn.apply(x, w, float(eps))


def add_rms_norm(x: torch.Tensor, delta: torch.Tensor, w: torch.Tensor, eps: float = 1e-6):
    """``(x + delta, rms_norm(x + delta, w, eps))`` with the sum written once."""
    if delta.shape != x.shape or delta.dtype != x.dtype:
        _note("add_rms_norm operands differ")
        return fb.add_rms_norm(x, delta, w, eps)
    if not _ok(x, w, delta):
        return fb.add_rms_norm(x, delta, w, eps)
    if _ADDRMS_OP is not None and _ops.wanted():
        xn, y, _rstd = _ADDRMS_OP(x, delta, w, float(eps))
        return xn, y
    if not wants_grad(x, delta, w):
        return _launch_addrms_fwd(x, delta, w, float(eps))[:2]
    return _AddRMSNormFn.apply(x, delta, w, float(eps))

"""``swiglu`` / ``swiglu_split``: the SwiGLU epilogue on the HIP kernels.

Call surface and dispatch of the reference's ``forgemind/kernels/swiglu.py:284-309``:
``autograd.Function`` in eager mode, ``torch.ops.forgemind.{swiglu,swiglu_split}`` (+
``*_backward``) while tracing, the torch expression when the gate says no.
"""

from __future__ import annotations

import typing

import torch

from . import _fallback as fb
from . import _hip, _ops
from ._common import _note, fast_ok, wants_grad


def _launch_fwd(gate, up):
    return _hip.swiglu_fwd(gate.contiguous(), up.contiguous())


def _launch_bwd(gate, up, dy):
    return _hip.swiglu_bwd(gate.contiguous(), up.contiguous(), dy.contiguous())


def _launch_split_fwd(x):
    w = x.shape[-1]
    return _hip.swiglu_split_fwd(x.contiguous().view(-1, w)).view(x.shape[:-1] + (w // 2,))


def _launch_split_bwd(x, dy):
    w = x.shape[-1]
    return _hip.swiglu_split_bwd(x.contiguous().view(-1, w), dy.contiguous().view(-1, w // 2)).view(x.shape)


class _SwiGLUFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate, up):
        ctx.save_for_backward(gate, up)
        return _launch_fwd(gate, up)

    @staticmethod
    def backward(ctx, dy):
        gate, up = ctx.saved_tensors
        return _launch_bwd(gate, up, dy)


class _SwiGLUSplitFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return _launch_split_fwd(x)

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        return _launch_split_bwd(x, dy)


# ------------------------------------------------------------------ traced: custom ops
def _sw_impl(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return _launch_fwd(gate, up)


def _sw_bwd_impl(gate: torch.Tensor, up: torch.Tensor,
                 dy: torch.Tensor) -> typing.Tuple[torch.Tensor, torch.Tensor]:
    return _launch_bwd(gate, up, dy)


def _sws_impl(x: torch.Tensor) -> torch.Tensor:
    return _launch_split_fwd(x)


def _sws_bwd_impl(x: torch.Tensor, dy: torch.Tensor) -> torch.Tensor:
    return _launch_split_bwd(x, dy)


def _sw_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _sw_autograd(ctx, dy):
    gate, up = ctx.saved_tensors
    return _SW_BWD_OP(gate, up, dy)


def _sws_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[0])


def _sws_autograd(ctx, dy):
    (x,) = ctx.saved_tensors
    return _SWS_BWD_OP(x, dy)


_SW_BWD_OP = _ops.define_backward("swiglu", _sw_bwd_impl,
                                  lambda gate, up, dy: (torch.empty_like(gate), torch.empty_like(up)))
_SWS_BWD_OP = _ops.define_backward("swiglu_split", _sws_bwd_impl, lambda x, dy: torch.empty_like(x))
_SW_OP = _ops.define("swiglu", _sw_impl, lambda gate, up: torch.empty_like(gate), _sw_setup, _sw_autograd)
_SWS_OP = _ops.define("swiglu_split", _sws_impl,
                      lambda x: x.new_empty(x.shape[:-1] + (x.shape[-1] // 2,)), _sws_setup, _sws_autograd)


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``F.silu(gate) * up`` with fp32 math and one rounding."""
    # differing shapes go to the torch expression, which broadcasts or raises as torch does
    # (reference kernels/swiglu.py:140-142, 291-297)
    if gate.shape != up.shape or gate.dtype != up.dtype or gate.numel() == 0 or gate.device != up.device:
        _note("swiglu operands")
        return fb.swiglu(gate, up)
    if not fast_ok(gate, up):
        return fb.swiglu(gate, up)
    if _SW_OP is not None and _ops.wanted():
        return _SW_OP(gate, up)
    if not wants_grad(gate, up):
        return _launch_fwd(gate, up)
    return _SwiGLUFn.apply(gate, up)


def swiglu_split(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(x[..., :h]) * x[..., h:]`` for a fused gate|up projection of width ``2h``."""
    if gate_up.dim() < 1 or gate_up.shape[-1] % 2 != 0:
        raise ValueError(f"swiglu_split needs an even last dimension (gate|up), got {gate_up.shape[-1] if gate_up.dim() else 0}")
    if gate_up.numel() == 0:
        _note("swiglu_split empty")
        return fb.swiglu_split(gate_up)
    if not fast_ok(gate_up):
        return fb.swiglu_split(gate_up)
    if _SWS_OP is not None and _ops.wanted():
        return _SWS_OP(gate_up)
    if not wants_grad(gate_up):
        return _launch_split_fwd(gate_up)
    return _SwiGLUSplitFn.apply(gate_up)


__all__ = ["swiglu", "swiglu_split"]

"""``qk_norm_rope``: per-head RMSNorm followed by half-split RoPE on the HIP kernels.

Call surface of the reference's ``forgemind/kernels/rope.py:207-244``: ``x`` is ``[B, T, H, D]``,
``w`` is ``[D]``, ``cos`` / ``sin`` are ``[T, D/2]``; gradients flow to ``x`` and ``w``.
"""

from __future__ import annotations

import typing

import torch

from . import _fallback as fb
from . import _hip, _ops
from ._common import _note, fast_ok, wants_grad

MAX_HEAD_DIM = 512


def _f32(t):
    return t.detach().to(torch.float32).contiguous()


def _torch_path(x, w, cos, sin, eps):
    t, half = cos.shape[-2], cos.shape[-1]
    return fb.qk_norm_rope(x, w, cos.reshape(1, t, 1, half), sin.reshape(1, t, 1, half), eps)


def _launch_fwd(x, w, cos, sin, eps):
    return _hip.qk_norm_rope_fwd(x.contiguous(), w.contiguous(), _f32(cos), _f32(sin), eps)


def _launch_bwd(x, w, cos, sin, rstd, dout, want_dw=True):
    return _hip.qk_norm_rope_bwd(x.contiguous(), w.contiguous(), _f32(cos), _f32(sin), rstd,
                                 dout.contiguous(), want_dw)


class _QKNormRoPE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, cos, sin, eps):
        out, rstd = _launch_fwd(x, w, cos, sin, eps)
        ctx.save_for_backward(x, w, cos, sin, rstd)
        return out

    @staticmethod
    def backward(ctx, dout):
        x, w, cos, sin, rstd = ctx.saved_tensors
        dx, dw = _launch_bwd(x, w, cos, sin, rstd, dout, ctx.needs_input_grad[1])
        return dx, dw, None, None, None


def _impl(x: torch.Tensor, w: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
          eps: float) -> typing.Tuple[torch.Tensor, torch.Tensor]:
    return _launch_fwd(x, w, cos, sin, eps)


def _fake(x, w, cos, sin, eps):
    rows = x.numel() // x.shape[-1]
    return torch.empty_like(x), torch.empty(rows, device=x.device, dtype=torch.float32)


def _bwd_impl(x: torch.Tensor, w: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, rstd: torch.Tensor,
              dout: torch.Tensor) -> typing.Tuple[torch.Tensor, torch.Tensor]:
    return _launch_bwd(x, w, cos, sin, rstd, dout, True)


def _bwd_fake(x, w, cos, sin, rstd, dout):
    return torch.empty_like(x), torch.empty_like(w)


def _setup(ctx, inputs, output):
    x, w, cos, sin, _eps = inputs
    ctx.save_for_backward(x, w, cos, sin, output[1])


def _autograd(ctx, dout, _drstd):
    x, w, cos, sin, rstd = ctx.saved_tensors
    dx, dw = _BWD_OP(x, w, cos, sin, rstd, dout)
    return dx, dw, None, None, None


_BWD_OP = _ops.define_backward("qk_norm_rope", _bwd_impl, _bwd_fake)
_OP = _ops.define("qk_norm_rope", _impl, _fake, _setup, _autograd)


def qk_norm_rope(x: torch.Tensor, w: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                 eps: float = 1e-6) -> torch.Tensor:
    """RMSNorm over each head's ``D`` values, then rotate the two halves by ``cos`` / ``sin``."""
    if x.dim() != 4:
        raise ValueError(f"qk_norm_rope expects [B, T, H, D], got {tuple(x.shape)}")
    b, t, h, d = x.shape
    if d % 2 != 0:
        raise ValueError(f"qk_norm_rope rotates pairs of features, so the head dim must be even; got {d}")
    need = t * (d // 2)
    if w.numel() != d or cos.numel() < need or sin.numel() < need:
        raise ValueError(f"qk_norm_rope: x {tuple(x.shape)}, w {tuple(w.shape)}, cos {tuple(cos.shape)}, "
                         f"sin {tuple(sin.shape)} disagree")
    # [T, D/2] or any shape whose first T * D/2 elements are that table (reference rope.py:231-238)
    cos = cos.reshape(-1)[:need].reshape(t, d // 2)
    sin = sin.reshape(-1)[:need].reshape(t, d // 2)
    ok_w = w.dtype == x.dtype or (w.dtype == torch.float32 and x.dtype in (torch.float16, torch.bfloat16))
    if d > MAX_HEAD_DIM or x.numel() == 0 or not ok_w or cos.dim() != 2 or cos.device != x.device:
        _note("qk_norm_rope shape")
        return _torch_path(x, w, cos, sin, eps)
    if not fast_ok(x, w):
        return _torch_path(x, w, cos, sin, eps)
    if _OP is not None and _ops.wanted():
        return _OP(x, w, cos, sin, float(eps))[0]
    if not wants_grad(x, w):
        return _launch_fwd(x, w, cos, sin, float(eps))[0]
    return _QKNormRoPE.apply(x, w, cos, sin, float(eps))


__all__ = ["qk_norm_rope"]

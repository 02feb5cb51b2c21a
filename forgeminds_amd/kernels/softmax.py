"""``softmax`` over the last dimension on the HIP kernel.

Call surface of the reference's ``forgemind/kernels/softmax.py:118-139``; the backward is
the closed form ``(g - sum(g * y)) * y`` (reference ``softmax.py:107-115``), in one kernel with
fp32 math on the saved ``y`` (tensor ops when the incoming gradient has another dtype).
"""

from __future__ import annotations

import torch

from . import _common, _hip
from ._common import fast_ok, wants_grad


class _Softmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        y = _hip.softmax_fwd(x.contiguous().view(-1, x.shape[-1])).view(x.shape)
        ctx.save_for_backward(y)
        return y

    @staticmethod
    def backward(ctx, g):
        (y,) = ctx.saved_tensors
        if g is None:
            return None
        if g.dtype != y.dtype or not g.is_cuda:
            inner = (g * y).sum(dim=-1, keepdim=True)
            return (g - inner) * y
        v = y.shape[-1]
        return _hip.softmax_bwd(y.contiguous().view(-1, v), g.contiguous().view(-1, v)).view(y.shape)


def softmax(x: torch.Tensor, dim: int = -1, dtype: "torch.dtype | None" = None) -> torch.Tensor:
    """``torch.softmax(x, dim=-1)`` drop-in; other dims, traced calls and float64 use torch."""
    if x.dim() < 1:
        raise ValueError(f"softmax needs ndim >= 1, got shape {tuple(x.shape)}")
    if dim not in (-1, x.dim() - 1):
        return torch.softmax(x, dim=dim, dtype=dtype)
    if dtype is not None and dtype != x.dtype:
        x = x.to(dtype)
    if _common.tracing():
        return torch.softmax(x, dim=-1)
    if x.numel() == 0 or x.numel() >= 2 ** 31 * 4:
        _common._note("softmax numel")
        return torch.softmax(x, dim=-1)
    if not fast_ok(x):
        return torch.softmax(x, dim=-1)
    if not wants_grad(x):
        return _hip.softmax_fwd(x.contiguous().view(-1, x.shape[-1])).view(x.shape)
    return _Softmax.apply(x)


__all__ = ["softmax"]

"""``topk``: exact, deterministic top-k over the last dim on the HIP kernel.

Call surface and error behaviour of the reference's ``forgemind/kernels/topk.py:273-297``:
canonical output order (value descending, index ascending inside ties; the smallest indices
win at the k-th value; NaN is the largest value and passes through), int64 indices, values
differentiable through a scatter, ``k`` outside ``[1, n]`` raises torch's message.
"""

from __future__ import annotations

import torch

from . import _common, _fallback as fb
from . import _hip
from ._common import fast_ok, wants_grad

#: the kernel ranks at most this many outputs per row; larger k takes the torch path
MAX_K = 512


def _ok(x: torch.Tensor, k: int) -> bool:
    if k > MAX_K:
        _common._note(f"topk k>{MAX_K}")
        return False
    if x.numel() >= 2 ** 31 * 4 or x.numel() == 0:
        _common._note("topk numel")
        return False
    return fast_ok(x)


class _TopK(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, k):
        n = x.shape[-1]
        vals, idx = _hip.topk(x.contiguous().view(-1, n), k, torch.int64)
        out_shape = x.shape[:-1] + (k,)
        idx = idx.view(out_shape)
        ctx.save_for_backward(idx)
        ctx.in_shape = x.shape
        ctx.mark_non_differentiable(idx)
        return vals.view(out_shape), idx

    @staticmethod
    def backward(ctx, g_vals, _g_idx):
        (idx,) = ctx.saved_tensors
        if g_vals is None:
            return None, None
        return g_vals.new_zeros(ctx.in_shape).scatter_(-1, idx, g_vals), None


def topk(x: torch.Tensor, k: int, dim: int = -1, sorted: bool = True):
    """Top-``k`` values and int64 indices along the last dimension (``torch.topk`` drop-in).

    ``sorted=False`` still returns the canonical sorted order. Other ``dim`` values and
    traced calls use ``torch.topk``; CPU / float64 / ``k > 512`` use a stable-sort torch
    expression that produces the same canonical order.
    """
    if x.dim() < 1:
        raise ValueError(f"topk needs ndim >= 1, got shape {tuple(x.shape)}")
    if dim not in (-1, x.dim() - 1):
        return torch.topk(x, k, dim=dim, sorted=True)
    n = x.shape[-1]
    if k < 1 or k > n:
        raise RuntimeError(f"selected index k out of range (got {k} vs {n})")
    if _common.tracing():
        return torch.topk(x, k, dim=-1, sorted=True)
    if not _ok(x, k):
        if x.is_floating_point():
            return fb.topk_canonical(x, k)
        return torch.topk(x, k, dim=-1, sorted=True)
    if not wants_grad(x):
        vals, idx = _hip.topk(x.contiguous().view(-1, n), k, torch.int64)
        return vals.view(x.shape[:-1] + (k,)), idx.view(x.shape[:-1] + (k,))
    return _TopK.apply(x, k)


__all__ = ["topk", "MAX_K"]

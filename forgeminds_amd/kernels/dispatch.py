"""``moe_gather`` / ``moe_combine``: the token moves on either side of the experts.

Stand in for the indexing sequence of the reference's ``MoE.forward``
(``forgemind/moe.py:234-235, 247-248``): ``xs = x[order // k]`` before the experts and
``zeros.index_add_(0, order // k, ys * w[order])`` after them. With the ``slot`` array of
:func:`moe_route` the scatter-add is a per-token gather, so the result is deterministic and
each output row is written once (the reference's ``index_add_`` uses atomics on a GPU).
"""

from __future__ import annotations

import torch

from . import _hip
from ._common import _note, fast_ok, tracing


def _inverse(perm: torch.Tensor) -> torch.Tensor:
    inv = torch.empty_like(perm)
    inv[perm.long()] = torch.arange(perm.numel(), device=perm.device, dtype=perm.dtype)
    return inv


def _i32(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous() if t.dtype == torch.int32 else t.to(torch.int32).contiguous()


class _GatherFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, order, slot, k, have_slot):
        ctx.save_for_backward(slot)
        ctx.k = k
        if have_slot:     # from the token's side: each row read once, written k times
            return _hip.moe_scatter(x.contiguous(), slot, k)
        return _hip.moe_gather(x.contiguous(), order, k)

    @staticmethod
    def backward(ctx, g):
        (slot,) = ctx.saved_tensors
        n = slot.numel() // ctx.k
        return _hip.moe_combine(g.contiguous(), None, slot, n, ctx.k), None, None, None, None


class _CombineFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ys, weights, slot, order):
        n, k = weights.shape
        w32 = weights.detach().to(torch.float32).contiguous()
        ctx.save_for_backward(ys, w32, slot, order)
        ctx.w_dtype = weights.dtype
        return _hip.moe_combine(ys.contiguous(), w32, slot, n, k)

    @staticmethod
    def backward(ctx, g):
        ys, w32, slot, order = ctx.saved_tensors
        n, k = w32.shape
        g = g.contiguous()
        d_ys = _hip.moe_scatter(g, slot, k, w32.view(-1)) if ctx.needs_input_grad[0] else None
        d_w = None
        if ctx.needs_input_grad[1]:
            d_w = _hip.moe_combine_dw(ys.contiguous(), g, slot, n, k).to(ctx.w_dtype)
        return d_ys, d_w, None, None


def moe_gather(x: torch.Tensor, order: torch.Tensor, k: int,
               slot: "torch.Tensor | None" = None) -> torch.Tensor:
    """``x[order // k]``: tokens ``[n, d]`` copied into expert-grouped order ``[n*k, d]``.

    ``order`` / ``slot`` are the permutation arrays of :func:`moe_route`; ``slot`` (the inverse
    of ``order``) is only needed for the backward and is derived when omitted.
    """
    if x.dim() != 2 or order.dim() != 1 or order.numel() != x.shape[0] * k:
        raise ValueError(f"moe_gather: x {tuple(x.shape)}, order {tuple(order.shape)}, k={k} disagree")
    if k > 16 or x.numel() == 0 or order.device != x.device:
        _note("moe_gather shape")
        return x[(order // k).long()]
    if tracing() or not fast_ok(x):      # a traced graph gets the tensor expression
        return x[(order // k).long()]
    order = _i32(order)
    have_slot = slot is not None or x.requires_grad
    if slot is None:
        slot = _inverse(order) if x.requires_grad else order
    return _GatherFn.apply(x, order, _i32(slot), int(k), have_slot)


def moe_combine(ys: torch.Tensor, weights: torch.Tensor, slot: torch.Tensor,
                order: "torch.Tensor | None" = None) -> torch.Tensor:
    """``out[t] = sum_j weights[t, j] * ys[slot[t*k + j]]`` -- the weighted return of expert
    outputs ``[n*k, d]`` to their tokens ``[n, d]``, summed in fp32 and rounded once."""
    if ys.dim() != 2 or weights.dim() != 2 or slot.numel() != weights.numel() or ys.shape[0] != slot.numel():
        raise ValueError(f"moe_combine: ys {tuple(ys.shape)}, weights {tuple(weights.shape)}, "
                         f"slot {tuple(slot.shape)} disagree")
    n, k = weights.shape

    def torch_path():
        picked = ys[slot.long()].view(n, k, ys.shape[1]).float()
        return (picked * weights.float().unsqueeze(-1)).sum(dim=1).to(ys.dtype)

    if k > 16 or ys.numel() == 0 or slot.device != ys.device or weights.device != ys.device:
        _note("moe_combine shape")
        return torch_path()
    if tracing() or not fast_ok(ys, weights):
        return torch_path()
    slot = _i32(slot)
    if order is None:
        order = _inverse(slot)
    return _CombineFn.apply(ys, weights, slot, _i32(order))


__all__ = ["moe_gather", "moe_combine"]

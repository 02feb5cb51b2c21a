"""``moe_route``: router softmax + top-k + renormalised weights + expert counts + the stable
dispatch permutation, in two HIP launches.

Stands in for the aten sequence of the reference's ``Router.forward`` and ``MoE.forward``
(``forgemind/moe.py:86-96, 232-236``): ``softmax`` -> ``topk`` -> divide -> ``scatter_add``
histogram -> ``torch.sort(stable=True)``. Nothing like it exists in the reference's kernel
package. Ties are resolved in the canonical order of ``fm.kernels.topk`` (equal
probabilities go to the lowest expert index), which ``torch.topk`` does not promise.
"""

from __future__ import annotations

from typing import NamedTuple

import torch

from . import _fallback as fb
from . import _hip
from ._common import _note, fast_ok

MAX_EXPERTS = 512
MAX_TOP_K = 8


class Routing(NamedTuple):
    """Result of :func:`moe_route` for ``n`` tokens, ``e`` experts, top-``k``."""

    idx: torch.Tensor       # [n, k] int32 expert of each assignment, best first
    weights: torch.Tensor   # [n, k] fp32, renormalised to sum to 1 per token
    counts: torch.Tensor    # [e] int32 assignments per expert
    slot: torch.Tensor      # [n*k] int32 position of flat assignment p after the stable sort
    order: torch.Tensor     # [n*k] int32 inverse: order[slot[p]] == p (== stable argsort of idx.flat)


def _torch_route(logits: torch.Tensor, k: int) -> Routing:
    """The same result from torch ops (CPU tensors, float64, oversize shapes)."""
    probs = torch.softmax(logits.float(), dim=-1)
    top_p, idx = fb.topk_canonical(probs, k)
    weights = top_p / top_p.sum(dim=-1, keepdim=True)
    flat = idx.reshape(-1)
    e = logits.shape[-1]
    counts = torch.zeros(e, dtype=torch.int64, device=logits.device)
    counts.scatter_add_(0, flat, torch.ones_like(flat))
    order = torch.sort(flat, stable=True).indices
    slot = torch.empty_like(order)
    slot[order] = torch.arange(order.numel(), device=order.device)
    return Routing(idx.to(torch.int32), weights, counts.to(torch.int32), slot.to(torch.int32),
                   order.to(torch.int32))


class _RouteFn(torch.autograd.Function):
    """Weights are differentiable wrt the logits; every integer output is not."""

    @staticmethod
    def forward(ctx, logits, k):
        idx, w, counts, slot, order = _hip.route(logits.contiguous(), k, True)
        ctx.save_for_backward(logits, idx)
        ctx.mark_non_differentiable(idx, counts, slot, order)
        return idx, w, counts, slot, order

    @staticmethod
    def backward(ctx, _gi, gw, _gc, _gs, _go):
        logits, idx = ctx.saved_tensors
        if gw is None:
            return None, None
        # d/dlogits of (p_top / sum p_top) with p = softmax(logits): recomputed on the tiny
        # [n, e] tensor with tensor ops
        p = torch.softmax(logits.float(), dim=-1)
        pk = torch.gather(p, 1, idx.long())
        s = pk.sum(dim=-1, keepdim=True)
        w = pk / s
        g_pk = (gw - (gw * w).sum(dim=-1, keepdim=True)) / s          # through the renormalise
        g_p = torch.zeros_like(p).scatter_(1, idx.long(), g_pk)      # through the gather
        g_logits = (g_p - (g_p * p).sum(dim=-1, keepdim=True)) * p    # through the softmax
        return g_logits.to(logits.dtype), None


def moe_route(logits: torch.Tensor, k: int) -> Routing:
    """Route ``n`` tokens over ``e`` experts: ``logits`` is ``[n, e]``.

    Returns a :class:`Routing`. ``flat[p] = idx[p // k, p % k]`` is the expert of flat
    assignment ``p``; ``order`` lists the flat assignments grouped by expert, ascending ``p``
    inside each expert (what ``moe.py:233`` gets from a stable sort), ``slot`` is its inverse
    and ``counts.cumsum(0)`` gives the group boundaries.
    """
    if logits.dim() != 2:
        raise ValueError(f"moe_route expects [tokens, experts] logits, got {tuple(logits.shape)}")
    n, e = logits.shape
    if k < 1 or k > e:
        raise RuntimeError(f"selected index k out of range (got {k} vs {e})")
    if e > MAX_EXPERTS or k > MAX_TOP_K or n * k >= 2 ** 31 - 1:
        _note("route shape")
        return _torch_route(logits, k)
    if not fast_ok(logits):
        return _torch_route(logits, k)
    return Routing(*_RouteFn.apply(logits, k))


__all__ = ["moe_route", "Routing", "MAX_EXPERTS", "MAX_TOP_K"]

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
from ._common import _note, fast_ok, tracing

MAX_EXPERTS = 512
MAX_TOP_K = 16


class Routing(NamedTuple):
    """Result of :func:`moe_route` for ``n`` tokens, ``e`` experts, top-``k``."""

    idx: torch.Tensor       # [n, k] int32 expert of each assignment, best first
    weights: torch.Tensor   # [n, k] fp32, renormalised to sum to 1 per token
    counts: torch.Tensor    # [e] int32 assignments per expert
    slot: torch.Tensor      # [n*k] int32 position of flat assignment p after the stable sort
    order: torch.Tensor     # [n*k] int32 inverse: order[slot[p]] == p (== stable argsort of idx.flat)
    aux: "torch.Tensor | None" = None   # load-balance loss E * sum(frac * mean(probs)) (with_aux=True)
    z: "torch.Tensor | None" = None     # router z-loss mean(logsumexp(logits)^2)     (with_aux=True)


def _torch_route(logits: torch.Tensor, k: int, with_aux: bool = False) -> Routing:
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
    aux = z = None
    if with_aux:
        frac = counts.to(torch.float32) / max(flat.numel(), 1)
        aux = e * (frac * probs.mean(dim=0)).sum()
        z = torch.logsumexp(logits.float(), dim=-1).pow(2).mean()
    return Routing(idx.to(torch.int32), weights, counts.to(torch.int32), slot.to(torch.int32),
                   order.to(torch.int32), aux, z)


class _RouteFn(torch.autograd.Function):
    """Weights and the two auxiliary losses are differentiable wrt the logits; every integer
    output is not. The backward is one kernel that recomputes the softmax of the [n, e] logits."""

    @staticmethod
    def forward(ctx, logits, k, with_aux):
        n, e = logits.shape
        if with_aux:
            idx, w, counts, slot, order, stats = _hip.route(logits.contiguous(), k, True, True)
            aux, z = stats[e + 1], stats[e + 2]      # both losses come finished from the kernel
        else:
            idx, w, counts, slot, order = _hip.route(logits.contiguous(), k, True)
            aux = z = logits.new_zeros((), dtype=torch.float32)
        ctx.save_for_backward(logits, idx, counts)
        ctx.k, ctx.with_aux = k, with_aux
        ctx.mark_non_differentiable(idx, counts, slot, order)
        return idx, w, counts, slot, order, aux, z

    @staticmethod
    def backward(ctx, _gi, gw, _gc, _gs, _go, g_aux, g_z):
        logits, idx, counts = ctx.saved_tensors
        if not ctx.with_aux:
            g_aux = g_z = None

        def scalar(t):
            return None if t is None else t.detach().to(torch.float32).reshape(()).contiguous()
        if gw is not None:
            gw = gw.detach().to(torch.float32).contiguous()
        return _hip.route_bwd(logits.contiguous(), idx, gw, counts, scalar(g_aux), scalar(g_z)), None, None


def moe_route(logits: torch.Tensor, k: int, with_aux: bool = False) -> Routing:
    """Route ``n`` tokens over ``e`` experts: ``logits`` is ``[n, e]``.

    ``with_aux=True`` also returns the two auxiliary router losses of the reference
    (``moe.py:92-95``), computed from sums the routing kernel accumulates on the way, so the
    logits are read once; both are differentiable wrt ``logits``.

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
        return _torch_route(logits, k, with_aux)
    if tracing():      # no op is registered for the router: a traced graph gets the tensor expression
        return _torch_route(logits, k, with_aux)
    if not fast_ok(logits):
        return _torch_route(logits, k, with_aux)
    out = _RouteFn.apply(logits, k, bool(with_aux))
    return Routing(*out) if with_aux else Routing(*out[:5])


__all__ = ["moe_route", "Routing", "MAX_EXPERTS", "MAX_TOP_K"]

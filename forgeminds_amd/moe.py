"""Router and dispatch bookkeeping with the interface of the reference's ``forgemind/moe.py``
(``Router`` :79-96 and the sort / gather / counts prologue of ``MoE.forward`` :227-236),
on top of the fused ``moe_route`` kernels. Experts, expert parallelism and the all-to-all
stay with the caller.
"""

from __future__ import annotations

from typing import NamedTuple

import torch
import torch.nn as nn

from .kernels import moe_route

__all__ = ["Router", "Dispatch", "dispatch_plan"]


class Dispatch(NamedTuple):
    """What ``MoE.forward`` needs after routing (reference ``moe.py:232-241``)."""

    weights: torch.Tensor   # [n, k] in the activation dtype
    idx: torch.Tensor       # [n, k] int64
    order: torch.Tensor     # [n*k] int64: flat assignments grouped by expert (stable)
    tok: torch.Tensor       # [n*k] int64: order // k, the token of each grouped assignment
    counts: torch.Tensor    # [e] int64
    offsets: torch.Tensor   # [e] int32 inclusive cumsum of counts (torch._grouped_mm offsets)
    aux: torch.Tensor       # load-balance loss
    z: torch.Tensor         # router z-loss


def dispatch_plan(logits: torch.Tensor, top_k: int, out_dtype=None) -> Dispatch:
    """Everything the expert layer needs from ``[n, e]`` router logits."""
    e = logits.shape[-1]
    r = moe_route(logits, top_k)
    probs_mean = torch.softmax(logits.float(), dim=-1).mean(dim=0)
    frac = r.counts.to(torch.float32) / max(r.idx.numel(), 1)
    aux = e * (frac.detach() * probs_mean).sum()
    z = torch.logsumexp(logits.float(), dim=-1).pow(2).mean()
    order = r.order.long()
    counts = r.counts.long()
    w = r.weights if out_dtype is None else r.weights.to(out_dtype)
    return Dispatch(w, r.idx.long(), order, order // top_k, counts,
                    counts.cumsum(0).to(torch.int32), aux, z)


class Router(nn.Module):
    """``gate`` projection + fused routing; ``forward`` returns ``(w, idx, aux, z)`` exactly
    like the reference's ``Router.forward`` (``moe.py:86-96``)."""

    def __init__(self, dim: int, n_experts: int, top_k: int):
        super().__init__()
        self.gate = nn.Linear(dim, n_experts, bias=False)
        self.n_experts, self.top_k = int(n_experts), int(top_k)
        self.last_plan: "Dispatch | None" = None

    def forward(self, x: torch.Tensor):
        logits = self.gate(x).float()
        plan = dispatch_plan(logits, self.top_k, x.dtype)
        self.last_plan = plan       # MoE.forward reuses order / counts instead of re-sorting
        return plan.weights, plan.idx, plan.aux, plan.z

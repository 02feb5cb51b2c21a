"""Router and dispatch bookkeeping with the interface of the reference's ``forgemind/moe.py``
(``Router`` :79-96 and the sort / gather / counts prologue of ``MoE.forward`` :227-236),
on top of the fused ``moe_route`` kernels. Experts, expert parallelism and the all-to-all
stay with the caller.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .kernels import moe_combine, moe_gather, moe_route

__all__ = ["Router", "Dispatch", "dispatch_plan", "Experts", "MoE"]


class Dispatch:
    """What ``MoE.forward`` needs after routing (reference ``moe.py:232-241``).

    The kernels' own outputs are held as they come; the int64 / cumulative forms the reference
    works with (``order``, ``tok``, ``counts``, ``offsets``) are derived on first use, so a
    caller that only moves tokens through ``order32`` / ``slot`` pays for none of them."""

    __slots__ = ("weights", "idx", "slot", "order32", "counts32", "aux", "z", "top_k", "_lazy")

    def __init__(self, weights, idx, slot, order32, counts32, aux, z, top_k):
        self.weights = weights      # [n, k] in the activation dtype
        self.idx = idx              # [n, k] int64
        self.slot = slot            # [n*k] int32: inverse of `order`
        self.order32 = order32      # [n*k] int32: flat assignments grouped by expert (stable)
        self.counts32 = counts32    # [e] int32
        self.aux = aux              # load-balance loss
        self.z = z                  # router z-loss
        self.top_k = top_k
        self._lazy = {}

    def _once(self, name, make):
        if name not in self._lazy:
            self._lazy[name] = make()
        return self._lazy[name]

    @property
    def order(self) -> torch.Tensor:      # [n*k] int64, what torch.sort(flat, stable=True) returns
        return self._once("order", lambda: self.order32.long())

    @property
    def tok(self) -> torch.Tensor:        # [n*k] int64: order // k, the token of each grouped assignment
        return self._once("tok", lambda: self.order // self.top_k)

    @property
    def counts(self) -> torch.Tensor:     # [e] int64
        return self._once("counts", lambda: self.counts32.long())

    @property
    def offsets(self) -> torch.Tensor:    # [e] int32 inclusive cumsum of counts (torch._grouped_mm offsets)
        return self._once("offsets", lambda: self.counts32.cumsum(0).to(torch.int32))


def dispatch_plan(logits: torch.Tensor, top_k: int, out_dtype=None) -> Dispatch:
    """Everything the expert layer needs from ``[n, e]`` router logits."""
    r = moe_route(logits, top_k, with_aux=True)
    w = r.weights if out_dtype is None else r.weights.to(out_dtype)
    return Dispatch(w, r.idx.long(), r.slot, r.order, r.counts, r.aux, r.z, top_k)


class Router(nn.Module):
    """``gate`` projection + fused routing; ``forward`` returns ``(w, idx, aux, z)`` exactly
    like the reference's ``Router.forward`` (``moe.py:86-96``)."""

    def __init__(self, dim: int, n_experts: int, top_k: int):
        super().__init__()
        self.gate = nn.Linear(dim, n_experts, bias=False)
        self.n_experts, self.top_k = int(n_experts), int(top_k)
        self.last_plan: "Dispatch | None" = None

    def forward(self, x: torch.Tensor):
        # the reference casts the gate output to fp32 first (moe.py:87); the routing kernels read
        # half logits and do the same fp32 math, so the cast (and its backward) is not materialised
        plan = dispatch_plan(self.gate(x), self.top_k, x.dtype)
        self.last_plan = plan       # MoE.forward reuses order / counts instead of re-sorting
        return plan.weights, plan.idx, plan.aux, plan.z


class Experts(nn.Module):
    """Stacked SwiGLU experts run as a per-expert loop over contiguous token groups -- the
    eager path of the reference's ``Experts`` (``forgemind/moe.py:99-181``), with its
    constructor order ``(n_local, dim, hidden)``, its ``normal(std=0.02)`` initialisation and its
    ``forward(x, counts=None, offsets=None)``. The grouped GEMM (``grouped_mm=True`` is accepted
    and, as in the reference when ``torch._grouped_mm`` is unusable, runs the loop) and the
    host-offloaded layout are outside this build."""

    def __init__(self, n_local: int, dim: int, hidden: int, offload: bool = False, grouped_mm: bool = False):
        super().__init__()
        if offload:
            raise ValueError("Experts(offload=True): host-offloaded experts are not part of this build")
        self.n_local, self.offload, self.grouped = int(n_local), False, False
        self.w1 = nn.Parameter(torch.empty(n_local, dim, hidden))
        self.w3 = nn.Parameter(torch.empty(n_local, dim, hidden))
        self.w2 = nn.Parameter(torch.empty(n_local, hidden, dim))
        self.reset_parameters(dim, hidden)

    def reset_parameters(self, dim=None, hidden=None):
        for w in (self.w1, self.w3, self.w2):
            nn.init.normal_(w, std=0.02)

    def forward(self, x: torch.Tensor, counts=None, offsets=None) -> torch.Tensor:
        """``counts``: per-expert group sizes, a python list or a tensor; ``offsets``: cumulative
        group ends instead (reference ``moe.py:146-159``). Neither: one group."""
        if counts is None:
            if offsets is None:
                counts = [x.size(0)]
            else:
                o = offsets.to(torch.int64)
                counts = torch.diff(o, prepend=o.new_zeros(1)).tolist()
        elif torch.is_tensor(counts):
            counts = counts.tolist()
        sizes = [int(c) for c in counts]
        if sum(sizes) != x.size(0):    # the reference's x.split(sizes) raises here (moe.py:160)
            raise RuntimeError(f"Experts.forward: group sizes sum to {sum(sizes)}, but x has {x.size(0)} rows")
        if not any(sizes):
            return x.new_zeros((0,) + tuple(x.shape[1:]))
        dt = x.dtype
        out = torch.empty_like(x)
        lo = 0
        for e, c in enumerate(sizes):
            if c:
                seg = x[lo:lo + c]
                a, b, o = self.w1[e], self.w3[e], self.w2[e]
                if a.dtype is not dt:
                    a, b, o = a.to(dt), b.to(dt), o.to(dt)
                out[lo:lo + c] = (torch.nn.functional.silu(seg @ a) * (seg @ b)) @ o
            lo += c
        return out


class MoE(nn.Module):
    """Single-device mixture of experts with the forward of the reference's ``MoE.forward``
    (``forgemind/moe.py:227-251``, ``ep_size == 1``): route, gather tokens by expert, run the
    experts on contiguous groups, return the weighted outputs to their tokens (plus the shared
    SwiGLU when ``n_shared`` > 0). Routing and both token moves are fused kernels; ``last_aux``
    carries the auxiliary losses. Constructor arguments in the reference's order
    (``moe.py:184-186``); expert parallelism and offloaded experts raise."""

    def __init__(self, dim: int, hidden: int, n_experts: int, top_k: int, n_shared: int = 0, ep_size: int = 1,
                 ep_group=None, ep_rank: int = 0, offload_experts: bool = False, grouped_mm: bool = False,
                 aux_coef: float = 1e-2, z_coef: float = 1e-3):
        super().__init__()
        if ep_size != 1 or ep_group is not None or ep_rank != 0:
            raise ValueError("MoE: expert parallelism (ep_size > 1) is not part of this one-GPU build")
        self.dim, self.n_experts = int(dim), int(n_experts)
        self.ep_size, self.ep_group, self.ep_rank, self.n_local = 1, None, 0, int(n_experts)
        self.router = Router(dim, n_experts, top_k)
        self.experts = Experts(n_experts, dim, hidden, offload=offload_experts, grouped_mm=grouped_mm)
        self.shared = None
        if n_shared:
            from .nn import SwiGLU
            self.shared = SwiGLU(dim, hidden * int(n_shared))
        self.top_k, self.aux_coef, self.z_coef = int(top_k), aux_coef, z_coef
        self.last_aux = None

    @property
    def compile_friendly(self) -> bool:
        """Reference ``moe.py:199-201``: true only with working grouped GEMM experts; here the
        experts always run the per-expert loop (``Experts.grouped`` stays False)."""
        return self.ep_size == 1 and self.experts.grouped

    def probe_grouped(self, device, dtype) -> bool:
        """Reference ``moe.py:203-225`` checks ``torch._grouped_mm`` once before compilation; the
        grouped GEMM is outside this build, so the answer is always no (callers such as the
        reference's ``models/gpt.py:261`` then keep the loop)."""
        self.experts.grouped = False
        return False

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        w, _idx, aux, z = self.router(x2)
        plan = self.router.last_plan
        self.last_aux = self.aux_coef * aux + self.z_coef * z
        xs = moe_gather(x2, plan.order32, self.top_k, plan.slot)
        ys = self.experts(xs, plan.counts32.tolist())        # the one host sync of the eager path
        out = moe_combine(ys, w, plan.slot, plan.order32)
        if self.shared is not None:
            out = out + self.shared(x2)
        return out.reshape(shape)

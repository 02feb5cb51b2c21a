"""The torch expressions the kernels stand in for.

This is what runs for CPU tensors, for float64, and under ``set_backend("fallback")`` -- the
same contract as the reference's ``forgemind/kernels/_fallback.py``: accumulate in fp32 for
half-precision inputs (float64/float32 keep their own precision) and round once, at the
output cast.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def _wide(t: torch.Tensor) -> torch.Tensor:
    """fp32 for half types, unchanged for float32/float64 (reference ``_fallback.py:15-23``)."""
    return t.float() if t.dtype in (torch.float16, torch.bfloat16) else t


def rms_norm(x, w, eps: float = 1e-6):
    """Reference ``_fallback.py:26-30``."""
    xw = _wide(x)
    inv = torch.rsqrt(xw.square().mean(dim=-1, keepdim=True) + eps)
    return (xw * inv * _wide(w)).to(x.dtype)


def add_rms_norm(x, delta, w, eps: float = 1e-6):
    """Reference ``_fallback.py:33-35``: the sum is rounded to x's dtype before it is normalised."""
    summed = x + delta
    return summed, rms_norm(summed, w, eps)


def layer_norm(x, w, b=None, eps: float = 1e-5):
    """``F.layer_norm`` in the wide dtype, one rounding (the rule of ``rms_norm`` above)."""
    xw = _wide(x)
    out = torch.nn.functional.layer_norm(xw, (x.shape[-1],), _wide(w).to(xw.dtype),
                                         None if b is None else _wide(b).to(xw.dtype), eps)
    return out.to(x.dtype)


def add_layer_norm(x, delta, w, b=None, eps: float = 1e-5):
    """The sum is rounded to x's dtype before it is normalised."""
    summed = x + delta
    return summed, layer_norm(summed, w, b, eps)


def kl_div_logits(student, teacher, reduction: str = "mean", temperature: float = 1.0):
    """KL(teacher || student) over the last dim (reference ``_fallback.py:52-69``).

    Differentiable wrt ``student`` through ordinary autograd; the teacher is detached.
    ``temperature`` divides both logit tensors first (no T**2 factor).
    """
    s, t = _wide(student), _wide(teacher).detach()
    if temperature != 1.0:
        s, t = s / temperature, t / temperature
    log_s = torch.log_softmax(s, dim=-1)
    log_t = torch.log_softmax(t, dim=-1)
    rows = (log_t.exp() * (log_t - log_s)).sum(dim=-1)
    if reduction == "none":
        return rows
    if reduction == "sum":
        return rows.sum()
    return rows.sum() / max(rows.numel(), 1)


def cross_entropy(logits, labels, ignore_index: int = -100, reduction: str = "mean"):
    """fp32 loss of ``F.cross_entropy`` summed over valid rows (reference ``loss.py:63-70``).

    ``mean`` divides by ``max(1, #valid)``. The math runs in fp32 on the logits' values, so a
    bf16 input does not get a bf16-rounded loss.
    """
    total = F.cross_entropy(_wide(logits), labels, ignore_index=ignore_index, reduction="sum")
    total = total.float()
    if reduction == "sum":
        return total
    n_valid = (labels != ignore_index).sum().clamp(min=1).to(torch.float32)
    return total / n_valid


def swiglu(gate, up):
    """Reference ``_fallback.py:48-49``."""
    return (F.silu(_wide(gate)) * _wide(up)).to(gate.dtype)


def swiglu_split(gate_up):
    half = gate_up.shape[-1] // 2
    return swiglu(gate_up[..., :half], gate_up[..., half:])


def qk_norm_rope(x, w, cos, sin, eps: float = 1e-6):
    """Per-head RMSNorm then half-split RoPE, x ``[B, T, H, D]`` (reference ``_fallback.py:38-45``)."""
    xw = _wide(x)
    inv = torch.rsqrt(xw.square().mean(dim=-1, keepdim=True) + eps)
    y = xw * inv * _wide(w)
    a, b = y.chunk(2, dim=-1)
    return torch.cat((a * cos - b * sin, a * sin + b * cos), dim=-1).to(x.dtype)


def topk_canonical(x, k: int):
    """Top-k in the canonical order (value desc, index asc inside ties, NaN largest).

    ``torch.topk`` promises no tie order, so the torch path gets it from a stable sort.
    """
    key = torch.nan_to_num(_wide(x), nan=float("inf"), posinf=float("inf"))
    # NaN and +inf share the top key; NaN must still come first, so rank NaN above +inf
    bump = torch.isnan(x)
    order = torch.sort(torch.where(bump, torch.zeros_like(key), torch.ones_like(key)),
                       dim=-1, stable=True).indices           # NaN first, original order inside
    key_sorted = torch.gather(key, -1, order)
    nan_sorted = torch.gather(bump, -1, order)
    # stable descending sort by value keeps (NaN first, then ascending index) inside ties
    composite = torch.where(nan_sorted, torch.full_like(key_sorted, float("inf")), key_sorted)
    second = torch.sort(composite, dim=-1, descending=True, stable=True).indices
    idx = torch.gather(order, -1, second)[..., :k]
    return torch.gather(x, -1, idx), idx

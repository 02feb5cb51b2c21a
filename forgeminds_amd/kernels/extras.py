"""Surface names of the reference's kernel package that are outside the packed hot path.

``qk_norm_rope`` and ``newton_schulz`` (reference ``forgemind/kernels/{rope,ns}.py``) keep
their torch expression here so code written against ``fm.kernels`` imports and runs unchanged.
"""

from __future__ import annotations

import torch

from . import _fallback as fb


def qk_norm_rope(x, w, cos, sin, eps: float = 1e-6):
    """Per-head RMSNorm + half-split RoPE for ``x [B, T, H, D]``, ``cos``/``sin`` ``[T, D/2]``
    (reference ``rope.py:227-244``)."""
    t, half = cos.shape[-2], cos.shape[-1]
    return fb.qk_norm_rope(x, w, cos.reshape(1, t, 1, half), sin.reshape(1, t, 1, half), eps)


def newton_schulz(g: torch.Tensor, steps: int = 5, eps: float = 1e-7) -> torch.Tensor:
    """Quintic Newton-Schulz orthogonalisation used by Muon (reference ``ns.py:172-201``)."""
    a, b, c = 3.4445, -4.7750, 2.0315
    x = g.to(torch.bfloat16 if g.is_cuda else torch.float32)
    transposed = x.shape[-2] > x.shape[-1]
    if transposed:
        x = x.mT
    x = x / (x.norm(dim=(-2, -1), keepdim=True) + eps)
    for _ in range(steps):
        gram = x @ x.mT
        x = a * x + (b * gram + c * (gram @ gram)) @ x
    if transposed:
        x = x.mT
    return x.to(g.dtype)


__all__ = ["qk_norm_rope", "newton_schulz"]

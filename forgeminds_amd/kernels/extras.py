"""Surface names of the reference's kernel package that are outside the packed hot path.

``newton_schulz`` (reference ``forgemind/kernels/ns.py``) is GEMM-bound optimizer plumbing; it
keeps its torch expression here so code written against ``fm.kernels`` imports and runs unchanged.
"""

from __future__ import annotations

import torch



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


__all__ = ["newton_schulz"]

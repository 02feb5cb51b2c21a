"""Cross-entropy callers with the interface of the reference's ``forgemind/loss.py``.

``logits_cross_entropy`` hands the whole ``[N, V]`` tensor to the fused kernel (which needs
no fp32 temporaries, so there is nothing to chunk); ``chunked_cross_entropy`` keeps the
reference's checkpoint-per-chunk structure around ``h @ weight.T`` (``loss.py:23-51``) and
uses the fused kernel's ``sum`` reduction for each chunk.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F
from torch.utils.checkpoint import checkpoint

from .kernels import cross_entropy

__all__ = ["chunked_cross_entropy", "logits_cross_entropy"]


def logits_cross_entropy(logits, labels, ignore_index: int = -100, chunk: int = 4096):
    """Mean CE over non-ignored tokens for ready logits ``[N, V]`` or ``[B, T, V]``.

    ``chunk`` is accepted for signature compatibility; the fused kernel streams each row once.
    """
    lg = logits.reshape(-1, logits.shape[-1])
    return cross_entropy(lg, labels.reshape(-1), ignore_index, "mean")


def chunked_cross_entropy(h, weight, labels, chunk: int = 4096, ignore_index: int = -100):
    """Mean CE over ``h @ weight.T`` with one chunk of logits alive at a time."""
    h = h.reshape(-1, h.size(-1))
    y = labels.reshape(-1)
    n_valid = (y != ignore_index).sum().clamp(min=1).to(torch.float32)
    needs_grad = torch.is_grad_enabled() and (h.requires_grad or weight.requires_grad)
    w = weight if weight.dtype == h.dtype else weight.to(h.dtype)

    def piece(hc, yc):
        # the chunk's logits are a temporary nobody else reads: the gradient may overwrite them
        return cross_entropy(F.linear(hc, w), yc, ignore_index, "sum", inplace=True)

    total = None
    for lo in range(0, h.size(0), chunk):
        hc, yc = h[lo:lo + chunk], y[lo:lo + chunk]
        part = checkpoint(piece, hc, yc, use_reentrant=False) if needs_grad else piece(hc, yc)
        total = part if total is None else total + part
    if total is None:      # empty batch: a zero that can still be back-propagated
        total = h.new_zeros((), dtype=torch.float32)
        return total.requires_grad_(True) if needs_grad else total
    return total / n_valid

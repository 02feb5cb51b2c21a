"""Fused vocabulary-wide cross entropy on the HIP kernels.

Stands in for the ``F.cross_entropy(..., reduction="sum") / n`` pattern of the reference's
``forgemind/loss.py:54-70`` (there is no fused CE kernel in the reference; its path is
aten ``log_softmax`` + ``nll_loss``). One read of the logits in the forward (online
max / sum-exp, per-row ``lse`` saved), softmax recomputed from ``lse`` in the backward.

The loss is fp32 math on the logits' values; a bf16 input does not yield a bf16-rounded
loss the way the literal ``F.cross_entropy(bf16)`` call does.
"""

from __future__ import annotations

import torch

from . import _fallback as fb
from . import _hip
from ._common import _note, fast_ok


class _CrossEntropyFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, ignore_index, reduction):
        lg2 = logits.contiguous().view(-1, logits.shape[-1])
        y = labels.contiguous().view(-1)
        loss, lse, n_valid, _rows = _hip.ce_fwd(lg2, y, ignore_index, reduction)
        ctx.save_for_backward(lg2, y, lse, n_valid)
        ctx.ignore_index = ignore_index
        ctx.mean = reduction == "mean"
        ctx.shape = logits.shape
        return loss.clone()     # `loss` is a view into a 2-element scratch tensor

    @staticmethod
    def backward(ctx, g):
        lg2, y, lse, n_valid = ctx.saved_tensors
        g32 = g.detach().to(torch.float32).contiguous()
        dl = _hip.ce_bwd(lg2, y, lse, n_valid if ctx.mean else None, g32, ctx.ignore_index)
        return dl.view(ctx.shape), None, None, None


def cross_entropy(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int = -100,
                  reduction: str = "mean") -> torch.Tensor:
    """fp32 scalar CE over the last dim of ``logits``.

    ``reduction="mean"`` divides the sum over valid rows by ``max(1, #valid)`` (all-ignored
    and empty inputs give 0.0 with a usable backward, reference
    ``tests/test_edge_cases.py:21-36``); ``"sum"`` returns the plain sum, which is what one
    chunk of ``chunked_cross_entropy`` contributes. Labels are int64; rows whose label equals
    ``ignore_index`` contribute nothing and receive a zero gradient.
    """
    if reduction not in ("mean", "sum"):
        raise ValueError(f"reduction must be mean|sum, got {reduction!r}")
    if logits.dim() < 1 or labels.shape != logits.shape[:-1]:
        raise ValueError(f"labels {tuple(labels.shape)} do not match logits {tuple(logits.shape)}")
    if (labels.dtype != torch.int64 or labels.device != logits.device
            or logits.shape[-1] == 0 or logits.numel() == 0 or logits.numel() >= 2 ** 31 * 4):
        _note("ce labels dtype/device or empty")
        return fb.cross_entropy(logits, labels, ignore_index, reduction)
    if not fast_ok(logits):
        return fb.cross_entropy(logits, labels, ignore_index, reduction)
    return _CrossEntropyFn.apply(logits, labels, int(ignore_index), reduction)


__all__ = ["cross_entropy"]

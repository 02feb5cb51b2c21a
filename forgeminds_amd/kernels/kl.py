"""``kl_div_logits`` / ``kl_distill_loss``: forward KL(teacher || student) on the HIP kernels.

Call surface of the reference's ``forgemind/kernels/kl.py:194-238``. The reference kernel
writes dKL/dlogits during the forward and multiplies it by the upstream gradient in the
backward (``kl.py:143-191``); here the forward is a single pass that keeps only the two
per-row log-sum-exps, and the backward recomputes both softmaxes -- one pass fewer over the
``[N, V]`` tensors and no ``[N, V]`` buffer held between forward and backward.

``temperature`` (not in the reference) divides both logit tensors before the softmax; the
gradient is wrt the undivided student logits, with no T**2 factor.
"""

from __future__ import annotations

import torch

from . import _fallback as fb
from . import _hip
from ._common import _note, fast_ok

_REDUCTIONS = ("mean", "sum", "none")


class _KLDivFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, student, teacher, reduction, grad_dtype, temperature):
        v = student.shape[-1]
        s2 = student.contiguous().view(-1, v)
        t2 = teacher.contiguous().view(-1, v)
        inv_t = 1.0 / float(temperature)
        loss, rows, lse_s, lse_t = _hip.kl_fwd(s2, t2, inv_t, reduction)
        ctx.save_for_backward(s2, t2, lse_s, lse_t)
        ctx.meta = (student.shape, reduction, grad_dtype or student.dtype, inv_t)
        if reduction == "none":
            return rows.clone().view(student.shape[:-1])
        return loss

    @staticmethod
    def backward(ctx, g):
        s2, t2, lse_s, lse_t = ctx.saved_tensors
        shape, reduction, gdt, inv_t = ctx.meta
        n = s2.shape[0]
        g32 = g.detach().to(torch.float32).contiguous().view(-1)
        scale = 1.0 / n if reduction == "mean" else 1.0
        grad = _hip.kl_bwd(s2, t2, lse_s, lse_t, g32, reduction == "none", gdt, inv_t, scale)
        return grad.view(shape), None, None, None, None


def _kernel_ok(*tensors) -> bool:
    if any(t.numel() >= 2 ** 31 * 4 for t in tensors):
        _note("kl numel")
        return False
    return fast_ok(*tensors)


def kl_div_logits(student: torch.Tensor, teacher: torch.Tensor, reduction: str = "mean",
                  grad_dtype: "torch.dtype | None" = None,
                  temperature: float = 1.0) -> torch.Tensor:
    """``KL(softmax(teacher / T) || softmax(student / T))`` over the last dim.

    ``mean`` divides by the number of rows (there is no ignore mask, reference
    ``_fallback.py:64-67``); ``none`` returns the per-row values. The teacher is a constant.
    ``grad_dtype`` (the student's dtype by default, or ``torch.float32``) is the dtype the
    kernel writes the student gradient in.
    """
    if reduction not in _REDUCTIONS:
        raise ValueError(f"reduction must be mean|sum|none, got {reduction!r}")
    if temperature <= 0:
        raise ValueError(f"temperature must be positive, got {temperature}")
    if (student.shape != teacher.shape or student.dim() < 1 or student.shape[-1] == 0
            or student.numel() == 0 or student.dtype != teacher.dtype
            or grad_dtype not in (None, student.dtype, torch.float32)):
        _note("kl operands")
        return fb.kl_div_logits(student, teacher, reduction, temperature)
    if not _kernel_ok(student, teacher):
        return fb.kl_div_logits(student, teacher, reduction, temperature)
    return _KLDivFn.apply(student, teacher, reduction, grad_dtype, float(temperature))


def kl_distill_loss(hs: torch.Tensor, ht: torch.Tensor, w: torch.Tensor, teacher_head,
                    chunk: int = 4096) -> torch.Tensor:
    """Mean forward KL of ``softmax(teacher_head(ht)) || softmax(hs @ w.T)`` in row chunks.

    Same structure as the reference's ``kl.py:209-233``: the teacher head runs under
    ``no_grad``; one chunk of student logits exists at a time in the forward. The chunk's
    logits (not its gradient) are what is kept for the backward.
    """
    hs2 = hs.reshape(-1, hs.shape[-1])
    ht2 = ht.reshape(-1, ht.shape[-1])
    n = hs2.shape[0]
    total = None
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        with torch.no_grad():
            t_log = teacher_head(ht2[lo:hi]).detach()
        s_log = hs2[lo:hi] @ w.t()
        piece = kl_div_logits(s_log, t_log.to(s_log.dtype), "sum")
        total = piece if total is None else total + piece
    if total is None:
        return hs2.new_zeros((), dtype=torch.float32)
    return total / n


kl_div = kl_div_logits
distill_kl = kl_distill_loss

__all__ = ["kl_div_logits", "kl_div", "kl_distill_loss", "distill_kl"]

"""``kl_div_logits`` / ``kl_distill_loss``: forward KL(teacher || student) on the HIP kernels.

Call surface of the reference's ``forgemind/kernels/kl.py:194-238``. The reference kernel
writes dKL/dlogits during the forward and multiplies it by the upstream gradient in the
backward (``kl.py:143-191``). Here rows of up to 64 KiB do the same from ONE read of both
tensors (they stay in registers between the log-sum-exps and the gradient store) and the
backward's multiply is skipped on the device when the upstream gradient is 1. Wider rows, and
``reduction="none"``, keep a single-pass forward that saves only the two per-row
log-sum-exps and a backward that recomputes both softmaxes: no ``[N, V]`` buffer is held
between forward and backward.

``temperature`` (not in the reference) divides both logit tensors before the softmax; the
gradient is wrt the undivided student logits, with no T**2 factor.
"""

from __future__ import annotations

import torch

from . import _fallback as fb
import typing

from . import _hip, _ops
from ._common import _note, fast_ok, tracing

_REDUCTIONS = ("mean", "sum", "none")


class _KLDivFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, student, teacher, reduction, grad_dtype, temperature, reuse, retain):
        v = student.shape[-1]
        s2 = student.contiguous().view(-1, v)
        t2 = teacher.contiguous().view(-1, v)
        inv_t = 1.0 / float(temperature)
        gdt = grad_dtype or student.dtype
        ctx.meta = (student.shape, reduction, gdt, inv_t)
        ctx.in_forward = False
        ctx.spent = False
        # fp16 gradients are not written in the forward: (p_s - p_t) / N rounded to fp16 before the
        # upstream gradient (a loss scale) is applied would flush to zero; the two-pass backward
        # below scales in fp32 and rounds once
        if reduction != "none" and ctx.needs_input_grad[0] and gdt != torch.float16:
            # gradient written in the forward (reference kl.py:143-176); `reuse` lets it land in
            # the student's own storage when that is the tensor the caller handed in
            own = reuse and s2.data_ptr() == student.data_ptr() and gdt == s2.dtype
            loss, grad, _rows = _hip.kl_loss_grad(s2.detach(), t2, inv_t, reduction, gdt, own)
            ctx.in_forward = True
            ctx.once = own or not retain
            if ctx.once:     # only the gradient buffer lives on (reference kl.py:171)
                ctx.save_for_backward(grad)
            else:            # asked for: the intact inputs stay too, so that a later backward can redo the pass
                ctx.save_for_backward(grad, s2.detach(), t2)
            return loss
        loss, rows, lse_s, lse_t = _hip.kl_fwd(s2, t2, inv_t, reduction)
        ctx.save_for_backward(s2, t2, lse_s, lse_t)
        if reduction == "none":
            return rows.clone().view(student.shape[:-1])
        return loss

    @staticmethod
    def backward(ctx, g):
        shape, reduction, gdt, inv_t = ctx.meta
        if ctx.in_forward:
            if ctx.once:
                (grad,) = ctx.saved_tensors
                if ctx.spent:
                    raise RuntimeError("kl_div_logits: the gradient buffer written in the forward was "
                                       "already consumed by a backward pass; run the forward again, or pass "
                                       "retain=True to keep the inputs for repeated backward passes")
            else:
                grad, s2, t2 = ctx.saved_tensors
                if ctx.spent:   # retain_graph: the first backward scaled `grad` in place (the reference
                    # multiplies out of place, kl.py:183-191, so repeated backward works there too)
                    _loss, grad, _rows = _hip.kl_loss_grad(s2, t2, inv_t, reduction, gdt, False)
            ctx.spent = True
            _hip.scale_inplace(grad, g.detach().to(torch.float32).contiguous())
            return grad.view(shape), None, None, None, None, None, None
        s2, t2, lse_s, lse_t = ctx.saved_tensors
        n = s2.shape[0]
        g32 = g.detach().to(torch.float32).contiguous().view(-1)
        scale = 1.0 / n if reduction == "mean" else 1.0
        grad = _hip.kl_bwd(s2, t2, lse_s, lse_t, g32, reduction == "none", gdt, inv_t, scale)
        return grad.view(shape), None, None, None, None, None, None


class _KLDivTopkFn(torch.autograd.Function):
    """KL forward that also hands back the teacher's top-k (indices and probabilities)."""

    @staticmethod
    def forward(ctx, student, teacher, k, reduction, grad_dtype, temperature, index_dtype, retain):
        v = student.shape[-1]
        s2 = student.contiguous().view(-1, v)
        t2 = teacher.contiguous().view(-1, v)
        inv_t = 1.0 / float(temperature)
        gdt = grad_dtype or student.dtype
        ctx.in_forward = False
        ctx.spent = False
        # KL, the teacher's top-k and (when the student needs it, in its own dtype) the gradient
        # for an upstream gradient of 1, all from one launch
        with_grad = (reduction != "none" and ctx.needs_input_grad[0] and gdt == student.dtype
                     and gdt != torch.float16)
        out = _hip.kl_fwd_topk(s2.detach(), t2, k, inv_t, reduction, index_dtype, want_grad=with_grad)
        if out is None:   # row too wide for the fused kernel: two launches, same results
            with_grad = False
            loss, rows, lse_s, lse_t = _hip.kl_fwd(s2, t2, inv_t, reduction)
            vals, idx = _hip.topk(t2, k, index_dtype)
            probs = torch.exp(vals.float() * inv_t - lse_t[:, None])
        else:
            loss, rows, lse_s, lse_t, _, idx, probs = out[:7]
        if with_grad:
            ctx.in_forward = True
            ctx.once = not retain
            if ctx.once:
                ctx.save_for_backward(out[7])
            else:
                ctx.save_for_backward(out[7], s2.detach(), t2)
        else:
            ctx.save_for_backward(s2, t2, lse_s, lse_t)
        ctx.meta = (student.shape, reduction, gdt, inv_t)
        lead = student.shape[:-1]
        probs = probs.view(*lead, k)
        idx = idx.view(*lead, k)
        ctx.mark_non_differentiable(probs, idx)
        if reduction == "none":
            return rows.clone().view(lead), probs, idx
        return loss, probs, idx

    @staticmethod
    def backward(ctx, g, _gp, _gi):
        shape, reduction, gdt, inv_t = ctx.meta
        if ctx.in_forward:
            if ctx.once:
                (grad,) = ctx.saved_tensors
                if ctx.spent:
                    raise RuntimeError("kl_div_logits_topk: the gradient buffer written in the forward was "
                                       "already consumed by a backward pass; run the forward again, or pass "
                                       "retain=True to keep the inputs for repeated backward passes")
            else:
                grad, s2, t2 = ctx.saved_tensors
                if ctx.spent:       # a repeated backward redoes the gradient from the intact inputs
                    _loss, grad, _rows = _hip.kl_loss_grad(s2, t2, inv_t, reduction, gdt, False)
            ctx.spent = True
            _hip.scale_inplace(grad, g.detach().to(torch.float32).contiguous())
            return grad.view(shape), None, None, None, None, None, None, None
        s2, t2, lse_s, lse_t = ctx.saved_tensors
        n = s2.shape[0]
        g32 = g.detach().to(torch.float32).contiguous().view(-1)
        scale = 1.0 / n if reduction == "mean" else 1.0
        grad = _hip.kl_bwd(s2, t2, lse_s, lse_t, g32, reduction == "none", gdt, inv_t, scale)
        return grad.view(shape), None, None, None, None, None, None, None


# ------------------------------------------------------------------ traced: custom ops
# Two op pairs, as for the cross entropy. Sum / mean over bf16 or fp32 logits: the forward op
# returns the loss and, as an extra output, the student's gradient for an upstream gradient of 1
# (the reference's dataflow, kl.py:143-191; aux outputs as in its _ops.py:44-48); the backward is
# the op that multiplies that buffer in place. reduction="none" and fp16 keep the functional
# two-pass dataflow: the forward keeps the two per-row log-sum-exps, the backward recomputes both
# softmaxes.
_RED = ("none", "sum", "mean")


def _kl_impl(student: torch.Tensor, teacher: torch.Tensor, reduction: int,
             inv_t: float) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    v = student.shape[-1]
    s2, t2 = student.contiguous().view(-1, v), teacher.contiguous().view(-1, v)
    loss, rows, lse_s, lse_t = _hip.kl_fwd(s2, t2, inv_t, _RED[reduction])
    out = rows.clone().view(student.shape[:-1]) if reduction == 0 else loss
    return out, lse_s.clone(), lse_t.clone()       # the three are rows of one buffer


def _kl_fake(student, teacher, reduction, inv_t):
    rows = student.numel() // student.shape[-1]
    f32 = dict(device=student.device, dtype=torch.float32)
    out = torch.empty(student.shape[:-1], **f32) if reduction == 0 else torch.empty((), **f32)
    return out, torch.empty(rows, **f32), torch.empty(rows, **f32)


def _kl_bwd_impl(student: torch.Tensor, teacher: torch.Tensor, lse_s: torch.Tensor, lse_t: torch.Tensor,
                 g: torch.Tensor, reduction: int, inv_t: float, fp32_grad: bool) -> torch.Tensor:
    v = student.shape[-1]
    s2, t2 = student.contiguous().view(-1, v), teacher.contiguous().view(-1, v)
    g32 = g.detach().to(torch.float32).contiguous().view(-1)
    scale = 1.0 / s2.shape[0] if reduction == 2 else 1.0
    gdt = torch.float32 if fp32_grad else student.dtype
    return _hip.kl_bwd(s2, t2, lse_s, lse_t, g32, reduction == 0, gdt, inv_t, scale).view(student.shape)


def _kl_bwd_fake(student, teacher, lse_s, lse_t, g, reduction, inv_t, fp32_grad):
    return torch.empty_like(student, dtype=torch.float32 if fp32_grad else student.dtype)


def _kl_setup(ctx, inputs, output):
    student, teacher, reduction, inv_t = inputs
    ctx.save_for_backward(student, teacher, output[1], output[2])
    ctx.reduction, ctx.inv_t = reduction, inv_t


def _kl_autograd(ctx, g, _g1, _g2):
    student, teacher, lse_s, lse_t = ctx.saved_tensors
    return _KL_BWD_OP(student, teacher, lse_s, lse_t, g, ctx.reduction, ctx.inv_t, False), None, None, None


def _kl1_impl(student: torch.Tensor, teacher: torch.Tensor, reduction: int,
              inv_t: float) -> typing.Tuple[torch.Tensor, torch.Tensor]:
    v = student.shape[-1]
    s2, t2 = student.contiguous().view(-1, v), teacher.contiguous().view(-1, v)
    loss, grad, _rows = _hip.kl_loss_grad(s2, t2, inv_t, _RED[reduction], student.dtype, False)
    return loss, grad.view(student.shape)


def _kl1_fake(student, teacher, reduction, inv_t):
    return (torch.empty((), device=student.device, dtype=torch.float32),
            torch.empty_like(student, memory_format=torch.contiguous_format))


def _kl1_setup(ctx, inputs, output):
    ctx.save_for_backward(output[1])


def _kl1_autograd(ctx, g, _ggrad):
    from .ce import SCALE_OP
    (grad,) = ctx.saved_tensors
    SCALE_OP(grad, g)
    return grad, None, None, None


_KL1_OP = _ops.define("kl_div_grad", _kl1_impl, _kl1_fake, _kl1_setup, _kl1_autograd)
_KL_BWD_OP = _ops.define_backward("kl_div", _kl_bwd_impl, _kl_bwd_fake)
_KL_OP = _ops.define("kl_div", _kl_impl, _kl_fake, _kl_setup, _kl_autograd)


def _kernel_ok(*tensors) -> bool:
    if any(t.numel() >= 2 ** 31 * 4 for t in tensors):
        _note("kl numel")
        return False
    return fast_ok(*tensors)


def kl_div_logits(student: torch.Tensor, teacher: torch.Tensor, reduction: str = "mean",
                  grad_dtype: "torch.dtype | None" = None,
                  temperature: float = 1.0, reuse: bool = False, retain: bool = False) -> torch.Tensor:
    """``KL(softmax(teacher / T) || softmax(student / T))`` over the last dim.

    ``mean`` divides by the number of rows (there is no ignore mask, reference
    ``_fallback.py:64-67``); ``none`` returns the per-row values. The teacher is a constant.
    ``grad_dtype`` (the student's dtype by default, or ``torch.float32``) is the dtype the
    kernel writes the student gradient in. ``reuse=True`` (reference ``kl.py:146-150``) lets
    the gradient overwrite ``student``: only for a tensor the caller owns and no longer reads.
    The gradient written in the forward serves one backward pass; ``retain=True`` also keeps the
    two logit tensors so that the backward may run again (``retain_graph=True``).
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
    if _KL_OP is not None and _ops.wanted() and grad_dtype in (None, student.dtype):
        if (reduction != "none" and student.dtype != torch.float16 and student.requires_grad
                and torch.is_grad_enabled()):
            return _KL1_OP(student, teacher, _RED.index(reduction), 1.0 / float(temperature))[0]
        return _KL_OP(student, teacher, _RED.index(reduction), 1.0 / float(temperature))[0]
    return _KLDivFn.apply(student, teacher, reduction, grad_dtype, float(temperature), bool(reuse), bool(retain))


def kl_div_logits_topk(student: torch.Tensor, teacher: torch.Tensor, k: int,
                       reduction: str = "mean", grad_dtype: "torch.dtype | None" = None,
                       temperature: float = 1.0, index_dtype: torch.dtype = torch.int64,
                       retain: bool = False):
    """``kl_div_logits`` plus the teacher's exact top-``k`` from the same pass over the logits.

    Returns ``(loss, probs, idx)``: ``idx [..., k]`` are the columns ``topk(teacher, k)`` would
    return (value descending, lowest index first among equals; reference
    ``forgemind/kernels/topk.py:13-19``) and ``probs [..., k]`` (fp32) are
    ``softmax(teacher / T)`` at those columns. The reference reads the teacher twice for this
    (``kernels/kl.py:194-207`` then ``kernels/topk.py:273-297``); the kernel reads it once.
    """
    if reduction not in _REDUCTIONS:
        raise ValueError(f"reduction must be mean|sum|none, got {reduction!r}")
    if temperature <= 0:
        raise ValueError(f"temperature must be positive, got {temperature}")
    if index_dtype not in (torch.int64, torch.int32):
        raise ValueError("index_dtype must be torch.int64 or torch.int32")
    if student.dim() < 1 or not 1 <= k <= max(student.shape[-1], 1):
        raise RuntimeError("selected index k out of range")
    ok = (student.shape == teacher.shape and student.shape[-1] > 0 and student.numel() > 0
          and student.dtype == teacher.dtype and k <= 512
          and grad_dtype in (None, student.dtype, torch.float32))
    if not ok or tracing() or not _kernel_ok(student, teacher):
        if ok is False:
            _note("kl operands")
        loss = fb.kl_div_logits(student, teacher, reduction, temperature)
        with torch.no_grad():
            _, idx = fb.topk_canonical(teacher, k)
            logp = torch.log_softmax(teacher.float() / temperature, dim=-1)
            probs = torch.gather(logp, -1, idx).exp()
        return loss, probs, idx.to(index_dtype)
    return _KLDivTopkFn.apply(student, teacher, int(k), reduction, grad_dtype, float(temperature),
                              index_dtype, bool(retain))


def _distill_piece(rows_s: torch.Tensor, rows_t: torch.Tensor, w_t: torch.Tensor, teacher_head) -> torch.Tensor:
    """Summed KL of one block of rows. The student logits of the block are a temporary of this
    call, so the kernel may write their gradient over them (``reuse=True``)."""
    with torch.no_grad():
        teacher_logits = teacher_head(rows_t)
    student_logits = rows_s @ w_t
    return kl_div_logits(student_logits, teacher_logits.detach().to(student_logits.dtype), "sum", reuse=True)


def kl_distill_loss(hs: torch.Tensor, ht: torch.Tensor, w: torch.Tensor, teacher_head,
                    chunk: int = 4096) -> torch.Tensor:
    """Mean forward KL of ``softmax(teacher_head(ht)) || softmax(hs @ w.T)`` over all rows, computed
    ``chunk`` rows at a time (call surface and meaning of the reference's ``kernels/kl.py:209-233``).

    The teacher head runs under ``no_grad``. Only one block of student logits exists at a time in
    the forward; what each block leaves behind for the backward is its gradient buffer (the
    logits' own storage), so with a student that needs gradients the blocks add up to N x V again,
    as the reference's docstring says of its own.
    """
    if chunk < 1:
        raise ValueError(f"chunk must be positive, got {chunk}")
    student_rows = hs.flatten(0, -2) if hs.dim() > 1 else hs.unsqueeze(0)
    teacher_rows = ht.flatten(0, -2) if ht.dim() > 1 else ht.unsqueeze(0)
    n = student_rows.size(0)
    if teacher_rows.size(0) != n:
        raise ValueError(f"student has {n} rows, teacher {teacher_rows.size(0)}")
    if n == 0:
        return student_rows.new_zeros((), dtype=torch.float32)
    w_t = w.t()
    pieces = [_distill_piece(s_blk, t_blk, w_t, teacher_head)
              for s_blk, t_blk in zip(student_rows.split(chunk), teacher_rows.split(chunk))]
    return torch.stack(pieces).sum() / n


kl_div = kl_div_logits
distill_kl = kl_distill_loss

__all__ = ["kl_div_logits", "kl_div_logits_topk", "kl_div", "kl_distill_loss", "distill_kl"]

"""Fused vocabulary-wide cross entropy on the HIP kernels.

Stands in for the ``F.cross_entropy(..., reduction="sum") / n`` pattern of the reference's
``forgemind/loss.py:54-70`` (there is no fused CE kernel in the reference; its path is
aten ``log_softmax`` + ``nll_loss``). When the logits need a gradient the forward produces it
in the same pass (each row stays in registers between the log-sum-exp and the gradient store),
the way the reference's KL writes its gradient in the forward (``kernels/kl.py:143-191``); the
backward multiplies by the upstream gradient in place, which the kernel skips when that is 1.
Without a gradient the forward is one read of the logits (online max / sum-exp).

The loss is fp32 math on the logits' values; a bf16 input does not yield a bf16-rounded
loss the way the literal ``F.cross_entropy(bf16)`` call does.
"""

from __future__ import annotations

import torch

from . import _fallback as fb
import typing

from . import _hip, _ops
from ._common import _note, fast_ok


class _CrossEntropyFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, ignore_index, reduction, inplace, retain):
        lg2 = logits.contiguous().view(-1, logits.shape[-1])
        y = labels.contiguous().view(-1)
        ctx.shape = logits.shape
        ctx.mode = "none"
        ctx.args = (ignore_index, reduction)
        if not ctx.needs_input_grad[0]:
            loss, _lse, _n_valid, _rows = _hip.ce_fwd(lg2, y, ignore_index, reduction, for_backward=False)
            return loss.clone()     # `loss` is a view into a 2-element scratch tensor
        if logits.dtype == torch.float16:
            # (softmax - onehot) / n_valid stored in fp16 before the upstream gradient is applied
            # would flush most entries to zero or to subnormals (p / 8192 < 6e-5) and a loss
            # scaler could no longer bring them back: fp16 keeps the two-pass dataflow, whose
            # backward applies the upstream gradient in fp32 and rounds once, as autograd does
            # for F.cross_entropy (reference loss.py:65-70)
            loss, lse, n_valid, _rows = _hip.ce_fwd(lg2, y, ignore_index, reduction)
            ctx.mode = "two_pass"
            ctx.save_for_backward(lg2, y, lse, n_valid.clone())
            return loss.clone()
        # writing into the caller's storage is only done when asked for and when lg2 is that
        # storage (contiguous() did not copy)
        own = inplace and lg2.data_ptr() == logits.data_ptr()
        loss, dl, _n_valid, _rows = _hip.ce_loss_grad(lg2.detach(), y, ignore_index, reduction, own)
        ctx.mode = "retain" if (retain and not own) else "once"
        ctx.spent = False
        if ctx.mode == "retain":    # asked for: keep the (intact) logits so that a later backward can redo the pass
            ctx.save_for_backward(dl, lg2.detach(), y)
        else:                       # only the gradient buffer lives on, as in the reference (kernels/kl.py:171)
            ctx.save_for_backward(dl)
        return loss.clone()

    @staticmethod
    def backward(ctx, g):
        g32 = g.detach().to(torch.float32).contiguous()
        ignore_index, reduction = ctx.args
        if ctx.mode == "two_pass":
            lg2, y, lse, n_valid = ctx.saved_tensors
            dl = _hip.ce_bwd(lg2, y, lse, n_valid if reduction == "mean" else None, g32, ignore_index)
            return dl.view(ctx.shape), None, None, None, None, None
        if ctx.mode == "once":
            (dl,) = ctx.saved_tensors
            if ctx.spent:
                raise RuntimeError("cross_entropy: the gradient buffer written in the forward was already "
                                   "consumed by a backward pass; run the forward again, or pass retain=True "
                                   "to keep the logits for repeated backward passes")
        else:
            dl, lg2, y = ctx.saved_tensors
            if ctx.spent:   # retain_graph / a second autograd.grad: the first pass scaled `dl` in place
                _loss, dl, _n, _r = _hip.ce_loss_grad(lg2, y, ignore_index, reduction, False)
        ctx.spent = True
        _hip.scale_inplace(dl, g32)
        return dl.view(ctx.shape), None, None, None, None, None


# ------------------------------------------------------------------ traced: custom ops
# Two op pairs. bf16 / fp32 logits take the dataflow of the eager path: the forward op returns the
# loss and, as extra outputs (the way the reference's ops carry rstd and xn,
# forgemind/kernels/_ops.py:44-48), the gradient for an upstream gradient of 1; the backward is an
# op that multiplies that buffer in place (mutates_args) and hands it on. fp16 logits keep the
# two-pass dataflow (forward keeps the per-row log-sum-exp, backward recomputes the softmax and
# applies the upstream gradient in fp32), which is purely functional.
def _ce_impl(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int,
             mean: bool) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    lg2 = logits.contiguous().view(-1, logits.shape[-1])
    loss, lse, n_valid, _rows = _hip.ce_fwd(lg2, labels.contiguous().view(-1), ignore_index,
                                            "mean" if mean else "sum")
    return loss.clone(), lse, n_valid.clone()


def _ce_fake(logits, labels, ignore_index, mean):
    rows = logits.numel() // logits.shape[-1]
    f32 = dict(device=logits.device, dtype=torch.float32)
    return torch.empty((), **f32), torch.empty(rows, **f32), torch.empty((), **f32)


def _ce_bwd_impl(logits: torch.Tensor, labels: torch.Tensor, lse: torch.Tensor, n_valid: torch.Tensor,
                 g: torch.Tensor, ignore_index: int, mean: bool) -> torch.Tensor:
    lg2 = logits.contiguous().view(-1, logits.shape[-1])
    g32 = g.detach().to(torch.float32).contiguous()
    dl = _hip.ce_bwd(lg2, labels.contiguous().view(-1), lse, n_valid if mean else None, g32, ignore_index)
    return dl.view(logits.shape)


def _ce_setup(ctx, inputs, output):
    logits, labels, ignore_index, mean = inputs
    ctx.save_for_backward(logits, labels, output[1], output[2])
    ctx.ignore_index, ctx.mean = ignore_index, mean


def _ce_autograd(ctx, g, _glse, _gn):
    logits, labels, lse, n_valid = ctx.saved_tensors
    return _CE_BWD_OP(logits, labels, lse, n_valid, g, ctx.ignore_index, ctx.mean), None, None, None


def _ce1_impl(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int,
              mean: bool) -> typing.Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    lg2 = logits.contiguous().view(-1, logits.shape[-1])
    loss, dl, n_valid, _rows = _hip.ce_loss_grad(lg2, labels.contiguous().view(-1), ignore_index,
                                                 "mean" if mean else "sum", False)
    return loss.clone(), dl.view(logits.shape), n_valid.clone()


def _ce1_fake(logits, labels, ignore_index, mean):
    f32 = dict(device=logits.device, dtype=torch.float32)
    return torch.empty((), **f32), torch.empty_like(logits, memory_format=torch.contiguous_format), torch.empty((), **f32)


def _scale_impl(grad: torch.Tensor, g: torch.Tensor) -> None:
    _hip.scale_inplace(grad, g.detach().to(torch.float32).contiguous())


def _ce1_setup(ctx, inputs, output):
    ctx.save_for_backward(output[1])


def _ce1_autograd(ctx, g, _gdl, _gn):
    (dl,) = ctx.saved_tensors
    SCALE_OP(dl, g)
    return dl, None, None, None


SCALE_OP = _ops.define_inplace("scale_grad_", _scale_impl, ("grad",))
_CE1_OP = _ops.define("cross_entropy_grad", _ce1_impl, _ce1_fake, _ce1_setup, _ce1_autograd)
_CE_BWD_OP = _ops.define_backward("cross_entropy", _ce_bwd_impl,
                                  lambda logits, labels, lse, n_valid, g, ignore_index, mean: torch.empty_like(logits))
_CE_OP = _ops.define("cross_entropy", _ce_impl, _ce_fake, _ce_setup, _ce_autograd)


def cross_entropy(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int = -100,
                  reduction: str = "mean", inplace: bool = False, retain: bool = False) -> torch.Tensor:
    """fp32 scalar CE over the last dim of ``logits``.

    ``reduction="mean"`` divides the sum over valid rows by ``max(1, #valid)`` (all-ignored
    and empty inputs give 0.0 with a usable backward, reference
    ``tests/test_edge_cases.py:21-36``); ``"sum"`` returns the plain sum, which is what one
    chunk of ``chunked_cross_entropy`` contributes. Labels are int64; rows whose label equals
    ``ignore_index`` contribute nothing and receive a zero gradient.

    ``inplace=True`` lets the kernel write the gradient over ``logits`` (only for a tensor the
    caller owns and no longer reads, e.g. the output of the head projection): no second
    ``[N, V]`` buffer exists, and that buffer serves ONE backward pass (a second one raises).
    Without ``inplace`` the gradient goes to a buffer of its own, which is all that is kept for
    the backward (the logits are not pinned), and it too serves one backward pass;
    ``retain=True`` also keeps the logits so that the backward may run any number of times
    (``retain_graph=True``): the first scales the gradient the forward wrote, later ones redo
    the pass.
    fp16 logits always take the two-pass form (forward keeps the log-sum-exps, the backward
    applies the upstream gradient in fp32 before its one rounding), so a loss scaler works.
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
    if _CE_OP is not None and _ops.wanted():
        if logits.dtype != torch.float16 and logits.requires_grad and torch.is_grad_enabled():
            return _CE1_OP(logits, labels, int(ignore_index), reduction == "mean")[0]
        return _CE_OP(logits, labels, int(ignore_index), reduction == "mean")[0]
    return _CrossEntropyFn.apply(logits, labels, int(ignore_index), reduction, bool(inplace), bool(retain))


__all__ = ["cross_entropy"]

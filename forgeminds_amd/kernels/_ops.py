"""``torch.library.custom_op`` registration and the eager-vs-op dispatch rule.

Same contract as the reference's ``forgemind/kernels/_ops.py``: in eager mode a kernel is
reached through ``torch.autograd.Function`` (cheapest Python dispatch); while
``torch.compile`` / ``torch.export`` trace, the same launch is reached through
``torch.ops.forgemind.<name>`` so it becomes one graph node with a fake implementation and
a registered backward. The backward is itself an op (``<name>_backward``) because AOTAutograd
traces the registered backward with fake tensors and must never see a raw launch
(reference ``_ops.py:50-56``).

``use_custom_ops(True|False|None)`` and ``FORGEMIND_KERNEL_OPS=ops|eager`` force one path.
"""

from __future__ import annotations

import os

import torch

try:
    from torch.library import CustomOpDef

    AVAILABLE = hasattr(torch.library, "custom_op") and hasattr(CustomOpDef, "register_autograd")
except Exception:  # pragma: no cover - torch older than 2.4
    AVAILABLE = False

NAMESPACE = "forgemind"
_ENV_MODE = os.environ.get("FORGEMIND_KERNEL_OPS", "auto").strip().lower()
_forced: "bool | None" = None


def available() -> bool:
    """Does this torch have ``custom_op`` with ``register_autograd``?"""
    return AVAILABLE


def use_custom_ops(flag: "bool | None" = None) -> bool:
    """Force the op path on / off, or ``None`` for automatic (on only while tracing)."""
    global _forced
    if flag and not AVAILABLE:  # pragma: no cover
        raise RuntimeError("torch.library.custom_op with a registered backward is not "
                           f"available on torch {torch.__version__}")
    _forced = None if flag is None else bool(flag)
    return wanted()


def wanted() -> bool:
    """Should the next kernel call be routed through ``torch.ops.forgemind``?"""
    if not AVAILABLE:
        return False
    if _forced is not None:
        return _forced
    if _ENV_MODE == "ops":
        return True
    if _ENV_MODE == "eager":
        return False
    try:
        return torch.compiler.is_compiling()
    except Exception:  # pragma: no cover
        return False


def _new_op(name: str, impl, fake, mutates=()):
    qual = f"{NAMESPACE}::{name}"
    try:
        op = torch.library.custom_op(qual, mutates_args=mutates)(impl)
    except (RuntimeError, ValueError) as exc:  # module imported twice in one process
        text = str(exc)
        packet = getattr(getattr(torch.ops, NAMESPACE, None), name, None)
        if packet is None or not ("already" in text or "overriding" in text):
            raise
        return packet.default
    if fake is not None:
        op.register_fake(fake)
    return op


def define(name: str, impl, fake, setup_context, backward):
    """Differentiable op ``forgemind::<name>``; returns ``None`` when the API is missing."""
    if not AVAILABLE:  # pragma: no cover
        return None
    op = _new_op(name, impl, fake)
    if hasattr(op, "register_autograd"):
        op.register_autograd(backward, setup_context=setup_context)
    return op


def define_backward(name: str, impl, fake):
    """Non-differentiable op ``forgemind::<name>_backward`` (called from a registered backward)."""
    if not AVAILABLE:  # pragma: no cover
        return None
    return _new_op(f"{name}_backward", impl, fake)


def define_inplace(name: str, impl, mutates):
    """Op ``forgemind::<name>`` that returns nothing and writes into the arguments named in
    ``mutates`` (the in-place multiply behind the losses whose forward already wrote the gradient)."""
    if not AVAILABLE:  # pragma: no cover
        return None
    return _new_op(name, impl, lambda *a, **k: None, mutates=tuple(mutates))


__all__ = ["AVAILABLE", "available", "use_custom_ops", "wanted", "define", "define_backward", "define_inplace"]

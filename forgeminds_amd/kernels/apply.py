"""Opt-in patching of an existing model's norm (and SwiGLU MLP) modules.

Same contract as the reference's ``forgemind/kernels/apply.py``: nothing changes unless
``patch(module)`` / ``enable(model)`` is called; both are idempotent; ``revert`` restores the
original ``forward``; unrecognised modules are left alone and ``patch`` returns ``False``.
"""

from __future__ import annotations

import types

import torch
import torch.nn as nn

from .layernorm import layer_norm
from .swiglu import swiglu, swiglu_split
from .norm import rms_norm


def _has_vector_weight(m: nn.Module) -> bool:
    w = getattr(m, "weight", None)
    return isinstance(w, nn.Parameter) and w.dim() == 1


def _looks_like_rmsnorm(m: nn.Module) -> bool:
    cls = type(m).__name__.lower()
    return ("rmsnorm" in cls or "rms_norm" in cls) and _has_vector_weight(m)


def _looks_like_swiglu_mlp(m: nn.Module) -> bool:
    parts = [getattr(m, n, None) for n in ("w1", "w2", "w3")]
    if not all(isinstance(p, nn.Linear) for p in parts):
        return False
    w1, w2, w3 = parts
    return (w1.out_features == w3.out_features and w1.in_features == w3.in_features
            and w2.in_features == w1.out_features)


def _swap_forward(m: nn.Module, fn) -> None:
    m._fm_orig_forward = m.__dict__.get("forward")   # None: forward lives on the class
    m.forward = types.MethodType(fn, m)


def _patch_norm(m: nn.Module) -> None:
    # eps: a number is used as is; torch's nn.RMSNorm(eps=None) means finfo(x.dtype).eps per
    # call; a module with no eps attribute gets this library's default of 1e-6
    # (reference apply.py:53-64)
    if hasattr(m, "eps"):
        eps = None if m.eps is None else float(m.eps)
    else:
        eps = 1e-6

    def forward(self, x):
        e = torch.finfo(x.dtype).eps if eps is None else eps
        return rms_norm(x, self.weight.to(x.dtype), e)

    _swap_forward(m, forward)


def _is_last_dim_layernorm(m: nn.Module) -> bool:
    return isinstance(m, nn.LayerNorm) and len(m.normalized_shape) == 1


def _patch_layernorm(m: nn.Module) -> None:
    def forward(self, x):
        if self.weight is None:      # elementwise_affine=False
            return layer_norm(x, torch.ones(self.normalized_shape, device=x.device, dtype=x.dtype), None, self.eps)
        return layer_norm(x, self.weight, self.bias, self.eps)

    _swap_forward(m, forward)


def _patch_mlp(m: nn.Module) -> None:
    def forward(self, x):
        return self.w2(swiglu(self.w1(x), self.w3(x)))

    _swap_forward(m, forward)


def _patch_mlp_split(m: nn.Module) -> None:
    w1, w3 = m.w1, m.w3
    if (w1.bias is None) != (w3.bias is None):
        _patch_mlp(m)       # one-sided bias cannot be concatenated
        return
    fused = nn.Linear(w1.in_features, 2 * w1.out_features, bias=w1.bias is not None,
                      device=w1.weight.device, dtype=w1.weight.dtype)
    with torch.no_grad():
        fused.weight.copy_(torch.cat([w1.weight, w3.weight], dim=0))
        if fused.bias is not None:
            fused.bias.copy_(torch.cat([w1.bias, w3.bias], dim=0))
    del m.w1, m.w3
    m.gate_up = fused
    m._fm_structural = True     # parameters were rewired: revert() leaves this in place

    def forward(self, x):
        return self.w2(swiglu_split(self.gate_up(x)))

    m.forward = types.MethodType(forward, m)


def patch(module: nn.Module, split: bool = False, kind: "str | None" = None) -> bool:
    """Fuse one module in place; ``True`` if it was recognised (or already patched).

    ``kind="norm"`` / ``kind="mlp"`` skips detection by class name and validates the structure
    instead, raising ``TypeError`` when it does not fit. ``kind="layernorm"`` is the only way a
    ``torch.nn.LayerNorm`` is touched (it is not an RMSNorm, and the reference leaves it alone:
    ``tests/test_nn_blocks.py:170-172``). ``split=True`` additionally merges
    ``w1|w3`` of an MLP into one ``gate_up`` projection (renames parameters).
    """
    if getattr(module, "_fm_norm", False) or getattr(module, "_fm_mlp", False):
        return True
    if kind not in (None, "norm", "mlp", "layernorm"):
        raise ValueError(f"kind must be 'norm', 'mlp', 'layernorm' or None, got {kind!r}")
    if kind == "layernorm":
        if not _is_last_dim_layernorm(module):
            raise TypeError(f"patch(kind='layernorm') needs a torch.nn.LayerNorm over the last "
                            f"dimension, got {type(module).__name__}")
        _patch_layernorm(module)
        module._fm_norm = True
        return True
    if kind == "norm" and not _has_vector_weight(module):
        raise TypeError(f"patch(kind='norm') needs a 1-D weight Parameter, "
                        f"{type(module).__name__} has {getattr(module, 'weight', None)!r}")
    if kind == "mlp" and not _looks_like_swiglu_mlp(module):
        raise TypeError(f"patch(kind='mlp') needs Linear children w1/w2/w3, "
                        f"{type(module).__name__} does not have that layout")
    if kind == "norm" or (kind is None and _looks_like_rmsnorm(module)):
        _patch_norm(module)
        module._fm_norm = True
        return True
    if kind == "mlp" or (kind is None and _looks_like_swiglu_mlp(module)):
        (_patch_mlp_split if split else _patch_mlp)(module)
        module._fm_mlp = True
        return True
    return False


def enable(model: nn.Module, norm: bool = True, swiglu_mlp: bool = True,
           split: bool = False, layer_norm: bool = False) -> nn.Module:
    """Patch every recognised module of ``model``; counts land on ``model._fm_fused``.

    ``layer_norm=True`` (off by default) also routes ``torch.nn.LayerNorm`` modules over the last
    dimension through the LayerNorm kernels; they are counted with the norms."""
    n_norm = n_mlp = 0
    for m in model.modules():
        if getattr(m, "_fm_norm", False) or getattr(m, "_fm_mlp", False):
            continue
        if layer_norm and _is_last_dim_layernorm(m):
            patch(m, kind="layernorm")
            n_norm += 1
        elif norm and _looks_like_rmsnorm(m):
            patch(m)
            n_norm += 1
        elif swiglu_mlp and _looks_like_swiglu_mlp(m):
            patch(m, split=split)
            n_mlp += 1
    model._fm_fused = {"norm": n_norm, "mlp": n_mlp}
    return model


def revert(module: nn.Module) -> nn.Module:
    """Undo forward swaps in ``module``'s tree; structural (``split=True``) patches stay."""
    restored = structural = 0
    for m in module.modules():
        if getattr(m, "_fm_structural", False):
            structural += 1
        if hasattr(m, "_fm_orig_forward"):
            original = m._fm_orig_forward
            if original is None:
                m.__dict__.pop("forward", None)
            else:
                m.forward = original
            del m._fm_orig_forward
            m.__dict__.pop("_fm_norm", None)
            m.__dict__.pop("_fm_mlp", None)
            restored += 1
    module._fm_fused_reverted = {"restored": restored, "structural": structural}
    return module


__all__ = ["patch", "enable", "revert"]

"""Module-level callers of the packed norm kernels.

``RMSNorm`` has the interface of the reference's ``fm.nn.RMSNorm`` (``forgemind/nn.py:82-147``):
state-dict compatible with ``torch.nn.RMSNorm``, plus ``forward_with_residual`` for the
pre-norm residual fusion. ``LayerNorm`` is the same shape of module around the LayerNorm
kernels, state-dict compatible with ``torch.nn.LayerNorm`` over the last dimension.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .kernels import add_layer_norm, add_rms_norm, layer_norm, rms_norm

__all__ = ["RMSNorm", "LayerNorm"]


class RMSNorm(nn.Module):
    """``x * rsqrt(mean(x**2) + eps) * weight`` over the last dimension.

    ``forward_with_residual(x, residual)`` returns ``(normed, x + residual)``: the residual
    stream is written once and normalised in the same pass. ``residual=None`` starts from zero.
    """

    def __init__(self, dim: int, eps: float = 1e-6, elementwise_affine: bool = True,
                 device=None, dtype=None):
        super().__init__()
        self.dim = int(dim)
        if self.dim <= 0:
            raise ValueError(f"RMSNorm needs dim > 0, got {dim}")
        self.eps = float(eps)
        self.elementwise_affine = bool(elementwise_affine)
        if self.elementwise_affine:
            self.weight = nn.Parameter(torch.ones(self.dim, device=device, dtype=dtype))
        else:
            self.register_parameter("weight", None)

    def extra_repr(self) -> str:
        return f"{self.dim}, eps={self.eps}, elementwise_affine={self.elementwise_affine}"

    def _weight_for(self, x: torch.Tensor) -> torch.Tensor:
        if self.weight is None:
            return torch.ones(self.dim, device=x.device, dtype=x.dtype)
        # an fp32 parameter next to half activations is consumed as is by the kernels; any
        # other mismatch is cast to the activation dtype like the reference does (nn.py:120-124)
        if self.weight.dtype == x.dtype or (self.weight.dtype == torch.float32 and x.is_cuda
                                            and x.dtype in (torch.float16, torch.bfloat16)):
            return self.weight
        return self.weight.to(x.dtype)

    def _check(self, x: torch.Tensor) -> None:
        if x.shape[-1] != self.dim:
            raise ValueError(f"RMSNorm({self.dim}) got a tensor with last dim {x.shape[-1]}; "
                             f"norms run over the last dimension of [..., {self.dim}]")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        self._check(x)
        return rms_norm(x, self._weight_for(x), self.eps)

    def forward_with_residual(self, x: torch.Tensor, residual: "torch.Tensor | None" = None):
        self._check(x)
        if residual is None:
            residual = torch.zeros_like(x)
        elif residual.shape != x.shape:
            raise ValueError(f"residual shape {tuple(residual.shape)} does not match x "
                             f"{tuple(x.shape)}; a residual stream must be the same shape")
        new_residual, normed = add_rms_norm(x, residual, self._weight_for(x), self.eps)
        return normed, new_residual


class LayerNorm(nn.Module):
    """``torch.nn.LayerNorm(dim)`` over the last dimension on the packed kernels.

    ``forward_with_residual(x, residual)`` returns ``(normed, x + residual)`` like
    ``RMSNorm.forward_with_residual``.
    """

    def __init__(self, dim: int, eps: float = 1e-5, elementwise_affine: bool = True, bias: bool = True,
                 device=None, dtype=None):
        super().__init__()
        self.dim = int(dim)
        if self.dim <= 0:
            raise ValueError(f"LayerNorm needs dim > 0, got {dim}")
        self.eps = float(eps)
        self.elementwise_affine = bool(elementwise_affine)
        if self.elementwise_affine:
            self.weight = nn.Parameter(torch.ones(self.dim, device=device, dtype=dtype))
        else:
            self.register_parameter("weight", None)
        if self.elementwise_affine and bias:
            self.bias = nn.Parameter(torch.zeros(self.dim, device=device, dtype=dtype))
        else:
            self.register_parameter("bias", None)

    def extra_repr(self) -> str:
        return f"{self.dim}, eps={self.eps}, elementwise_affine={self.elementwise_affine}"

    def _params_for(self, x: torch.Tensor):
        if self.weight is None:
            return torch.ones(self.dim, device=x.device, dtype=x.dtype), None
        keep = self.weight.dtype == x.dtype or (self.weight.dtype == torch.float32 and x.is_cuda
                                                and x.dtype in (torch.float16, torch.bfloat16))
        w = self.weight if keep else self.weight.to(x.dtype)
        b = self.bias
        if b is not None and b.dtype != w.dtype:
            b = b.to(w.dtype)
        return w, b

    def _check(self, x: torch.Tensor) -> None:
        if x.shape[-1] != self.dim:
            raise ValueError(f"LayerNorm({self.dim}) got a tensor with last dim {x.shape[-1]}; "
                             f"norms run over the last dimension of [..., {self.dim}]")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        self._check(x)
        w, b = self._params_for(x)
        return layer_norm(x, w, b, self.eps)

    def forward_with_residual(self, x: torch.Tensor, residual: "torch.Tensor | None" = None):
        self._check(x)
        if residual is None:
            residual = torch.zeros_like(x)
        elif residual.shape != x.shape:
            raise ValueError(f"residual shape {tuple(residual.shape)} does not match x "
                             f"{tuple(x.shape)}; a residual stream must be the same shape")
        w, b = self._params_for(x)
        new_residual, normed = add_layer_norm(x, residual, w, b, self.eps)
        return normed, new_residual

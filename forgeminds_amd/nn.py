"""Module-level callers of the packed norm kernels.

``RMSNorm`` has the interface of the reference's ``fm.nn.RMSNorm`` (``forgemind/nn.py:82-147``):
state-dict compatible with ``torch.nn.RMSNorm``, plus ``forward_with_residual`` for the
pre-norm residual fusion. ``LayerNorm`` is the same shape of module around the LayerNorm
kernels, state-dict compatible with ``torch.nn.LayerNorm`` over the last dimension.
``SwiGLU`` has the interface of ``fm.nn.SwiGLU`` (``forgemind/nn.py:150-217``): the gated MLP
whose ``silu(gate) * up`` runs on the packed kernel, with the two input projections either
separate (``w1``, ``w3``) or as one ``gate_up`` GEMM.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .kernels import add_layer_norm, add_rms_norm, layer_norm, rms_norm, swiglu, swiglu_split

__all__ = ["RMSNorm", "LayerNorm", "SwiGLU"]


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


class SwiGLU(nn.Module):
    """Gated MLP ``w2(silu(w1(x)) * w3(x))``; the elementwise part is one kernel.

    With ``split=True`` the gate and up projections are a single ``gate_up`` Linear of
    ``2 * hidden`` outputs (gate rows first) feeding ``swiglu_split``: one GEMM and one pass
    over its output. The parameter names differ between the two layouts (``w1``/``w3`` against
    ``gate_up``); the results do not. ``hidden`` defaults to ``4 * dim``.
    """

    def __init__(self, dim: int, hidden: "int | None" = None, bias: bool = False, split: bool = False,
                 device=None, dtype=None):
        super().__init__()
        self.dim = int(dim)
        self.hidden = 4 * self.dim if hidden is None else int(hidden)
        if self.dim <= 0 or self.hidden <= 0:
            raise ValueError(f"SwiGLU needs dim > 0 and hidden > 0, got dim={dim}, hidden={hidden}")
        self.split = bool(split)
        opts = {"bias": bool(bias), "device": device, "dtype": dtype}
        if self.split:
            self.gate_up = nn.Linear(self.dim, 2 * self.hidden, **opts)
        else:
            self.w1 = nn.Linear(self.dim, self.hidden, **opts)   # gate
            self.w3 = nn.Linear(self.dim, self.hidden, **opts)   # up
        self.w2 = nn.Linear(self.hidden, self.dim, **opts)       # down

    def extra_repr(self) -> str:
        return f"{self.dim} -> {self.hidden} -> {self.dim}, split={self.split}"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.split:
            return self.w2(swiglu_split(self.gate_up(x)))
        return self.w2(swiglu(self.w1(x), self.w3(x)))

    @torch.no_grad()
    def to_split(self, inplace: bool = True) -> "SwiGLU":
        """The same function with ``w1`` and ``w3`` stacked into ``gate_up``.

        ``inplace=True`` rewires this module (its ``w1``/``w3`` parameters disappear, so an
        optimizer or checkpoint that names them has to be rebuilt) and returns it;
        ``inplace=False`` returns a new module and leaves this one alone. A module that is
        already split is returned as is.
        """
        if self.split:
            return self
        gate, up, down = self.w1, self.w3, self.w2
        if (gate.bias is None) != (up.bias is None):
            raise ValueError("to_split() needs the gate and up projections to both have a bias or "
                             "both lack one; stacking them would drop it")
        where = {"device": gate.weight.device, "dtype": gate.weight.dtype}
        stacked = nn.Linear(self.dim, 2 * self.hidden, bias=gate.bias is not None, **where)
        stacked.weight.copy_(torch.cat((gate.weight, up.weight), dim=0))
        if stacked.bias is not None:
            stacked.bias.copy_(torch.cat((gate.bias, up.bias), dim=0))
        if inplace:
            target = self
            del target.w1, target.w3
        else:
            target = SwiGLU(self.dim, self.hidden, bias=down.bias is not None, split=True,
                            device=down.weight.device, dtype=down.weight.dtype)
            target.w2.load_state_dict(down.state_dict())
        target.gate_up = stacked
        target.split = True
        return target

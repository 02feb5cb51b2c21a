"""Packed kernels for MI355X: the ``fm.kernels`` call surface on hand-written HIP.

    import forgeminds_amd as fm
    y = fm.kernels.rms_norm(x, w, 1e-6)                  # == F.rms_norm(x, (d,), w, eps)
    xn, y = fm.kernels.add_rms_norm(x, delta, w, 1e-6)   # residual add + norm, one pass
    loss = fm.kernels.cross_entropy(logits, labels)      # fp32, mean over valid rows
    loss = fm.kernels.kl_div_logits(student, teacher)    # KL(teacher || student)
    v, i = fm.kernels.topk(x, 64)                        # canonical, deterministic order
    r = fm.kernels.moe_route(router_logits, k=2)         # idx, weights, counts, slot, order
    xs = fm.kernels.moe_gather(x, r.order, 2, r.slot)    # tokens grouped by expert
    out = fm.kernels.moe_combine(ys, r.weights, r.slot, r.order)   # weighted return to tokens

    fm.kernels.enable(model)              # patch RMSNorm / SwiGLU modules in place
    fm.kernels.set_backend("fallback")    # force the torch expressions (A/B, debugging)
    fm.kernels.stats()                    # which path ran, how often, and why

Every function is a drop-in for a torch expression and keeps its autograd contract. CPU
tensors, float64 and ``set_backend("fallback")`` run that torch expression; GPU tensors run
the HIP kernels in ``libfmhip.so`` (``autograd.Function`` eagerly, ``torch.ops.forgemind.*``
while ``torch.compile`` traces).
"""

from . import _common
from ._common import HAS_TRITON, get_backend, reset_stats, set_backend, stats
from ._ops import use_custom_ops
from .apply import enable, patch, revert
from .ce import cross_entropy
from .dispatch import moe_combine, moe_gather
from .extras import newton_schulz
from .kl import distill_kl, kl_distill_loss, kl_div, kl_div_logits, kl_div_logits_topk
from .layernorm import add_layer_norm, layer_norm
from .norm import add_rms_norm, rms_norm
from .rope import qk_norm_rope
from .route import Routing, moe_route
from .softmax import softmax
from .swiglu import swiglu, swiglu_split
from .topk import topk

__all__ = [
    "HAS_TRITON", "set_backend", "get_backend", "stats", "reset_stats",
    "rms_norm", "add_rms_norm", "qk_norm_rope", "swiglu", "swiglu_split",
    "layer_norm", "add_layer_norm", "kl_div_logits", "kl_div_logits_topk", "kl_div", "kl_distill_loss", "distill_kl",
    "newton_schulz", "topk", "softmax", "cross_entropy", "moe_route", "Routing",
    "moe_gather", "moe_combine",
    "enable", "patch", "revert", "available", "use_custom_ops",
]


def available() -> bool:
    """True when the HIP kernels can actually run here: library built and a GPU visible."""
    import torch

    return _common.extension_available() and torch.cuda.is_available()

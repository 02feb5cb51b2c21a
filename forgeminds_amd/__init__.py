"""forgeminds_amd: ForgeMind's packed-kernel hot path, rebuilt for MI355X (gfx950).

``forgeminds_amd.kernels`` mirrors the reference's ``forgemind.kernels`` surface; ``nn``,
``loss`` and ``moe`` hold the thin callers that sit directly on top of it.
"""

from . import kernels, loss, moe, nn
from .kernels import available

__version__ = "0.1.0"

__all__ = ["kernels", "nn", "loss", "moe", "available", "__version__"]

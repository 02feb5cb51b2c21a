"""Backend switch, call statistics and the gate that decides kernel vs torch expression.

Mirrors the contract of the reference's ``forgemind/kernels/_common.py:47-119``:

* ``set_backend("auto" | "fallback" | "triton")`` -- ``"triton"`` is kept as the name of
  "force the native kernels" so code written against the reference keeps working; ``"hip"``
  is an alias for it;
* every wrapper takes the torch expression when the gate says no, and ``stats()`` records how
  often and why (``"backend=fallback"``, ``"not cuda"``, ``"dtype torch.float64"``, ...);
* nothing is counted while ``torch.compile`` traces (a dict update inside a checkpointed
  region would force a graph break, reference ``_common.py:84-96``).

The library missing or unloadable is the reference's ``"no triton"`` case
(``_common.py:104-106``): under ``"auto"`` the wrappers run the torch expression and
``stats()["reasons"]`` counts ``"no extension"``; ``available()`` is False. A forced backend
(``"triton"`` / ``"hip"``) raises instead, and so do ``bench.py`` and ``smoke()``, which ask for
the library itself.
"""

from __future__ import annotations

import torch

from . import _hip

#: widest row the reference's norm kernels accepted (``_common.py:47``); kept for callers that
#: read it. The HIP kernels take any width.
MAX_DIM = 8192
#: the reference exported this flag; there is no Triton here by design.
HAS_TRITON = False

_hip.loaded()      # resolve the library once at import, outside any traced region

_BACKENDS = ("auto", "fallback", "triton", "hip")
_BACKEND = "auto"
_STATS = {"fast": 0, "fallback": 0, "reason": {}}
_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def set_backend(name: str) -> None:
    """``"auto"`` (default), ``"fallback"`` (force torch), ``"triton"``/``"hip"`` (force kernels)."""
    global _BACKEND
    if name not in _BACKENDS:
        raise ValueError(f"unknown kernel backend {name!r}; use auto|fallback|triton")
    _BACKEND = name


def get_backend() -> str:
    return _BACKEND


def forced() -> bool:
    return _BACKEND in ("triton", "hip")


def stats() -> dict:
    """Calls that took the kernel path vs the torch path, and the reasons for the latter."""
    return {"fast": _STATS["fast"], "fallback": _STATS["fallback"],
            "reasons": dict(_STATS["reason"])}


def reset_stats() -> None:
    _STATS.update(fast=0, fallback=0, reason={})


def extension_available() -> bool:
    return _hip.loaded()


def tracing() -> bool:
    """True while ``torch.compile`` / ``torch.export`` trace this code."""
    try:
        return torch.compiler.is_compiling()
    except Exception:  # pragma: no cover - torch without the API
        return False


def _note(why: str) -> None:
    if tracing():
        return
    _STATS["fallback"] += 1
    _STATS["reason"][why] = _STATS["reason"].get(why, 0) + 1


def fast_ok(*tensors) -> bool:
    """Can the HIP kernels run on these tensors right now? (Order of the checks as in the
    reference, ``_common.py:99-119``: backend, extension, then the tensors.)"""
    if _BACKEND == "fallback":
        _note("backend=fallback")
        return False
    if not _hip.loaded():
        if forced():
            raise RuntimeError(f"kernel backend {_BACKEND!r} is forced but the HIP extension is "
                               f"unavailable ({_hip.load_error()})")
        _note("no extension")
        return False
    for t in tensors:
        if not isinstance(t, torch.Tensor):
            continue
        if not t.is_cuda:
            if forced():
                raise RuntimeError(f"kernel backend {_BACKEND!r} is forced but a tensor lives on "
                                   f"{t.device}; the HIP kernels need GPU tensors")
            _note("not cuda")
            return False
        if t.dtype not in _FLOATS:
            _note(f"dtype {t.dtype}")
            return False
    if not tracing():
        _STATS["fast"] += 1
    return True


def wants_grad(*tensors) -> bool:
    """Will autograd record this call? An inference call goes straight to the launcher and skips
    the ``autograd.Function`` object (a few microseconds of host time per call)."""
    if not torch.is_grad_enabled():
        return False
    for t in tensors:
        if t is not None and t.requires_grad:
            return True
    return False


def next_pow2(n: int) -> int:
    n = max(int(n), 1)
    return 1 << (n - 1).bit_length()

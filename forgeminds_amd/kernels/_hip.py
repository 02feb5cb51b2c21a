"""ctypes binding of ``libfmhip.so`` (the C ABI declared in ``include/fm_hip.h``).

Nothing here computes: each wrapper checks shapes the kernels assume, resolves the current
device and stream of the tensor, passes raw device pointers and raises ``RuntimeError`` with
the library's message on a non-zero status. Outputs are allocated by the callers in
``norm.py`` / ``ce.py`` / ... with ``torch.empty``; the library itself never allocates.
"""

from __future__ import annotations

import contextlib
import ctypes as C
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# FORGEMINDS_AMD_LIB points at another build of the library (a release next to a debug build)
LIB_PATH = os.environ.get("FORGEMINDS_AMD_LIB") or os.path.join(os.path.dirname(_HERE), "_lib", "libfmhip.so")

F32, F16, BF16 = 0, 1, 2
REDUCE = {"none": 0, "sum": 1, "mean": 2}
_DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

_lib = None
_lib_err: "str | None" = None
_lock = threading.Lock()

_vp, _i64, _int, _f32, _sz = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_size_t

# name -> (restype, argtypes); mirrors include/fm_hip.h one to one
SIGNATURES = {
    "fm_version": (_int, []),
    "fm_last_error": (C.c_char_p, []),
    "fm_last_kernel": (C.c_char_p, []),
    "fm_set_param": (_int, [C.c_char_p, _int]),
    "fm_stream_probe": (_int, [_vp, _vp, _vp, _sz, _int, _vp]),
    "fm_stream_probe_mix": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _int, _int, _int, _int, _int, _i64, _vp]),
    "fm_rmsnorm_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _f32, _vp]),
    "fm_rmsnorm_bwd_workspace": (_sz, [_i64, _i64, _int]),
    "fm_rmsnorm_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64, _int, _int, _vp]),
    "fm_rmsnorm_bwd_static": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "fm_add_rmsnorm_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _f32, _vp]),
    "fm_add_rmsnorm_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64,
                                  _int, _int, _vp]),
    "fm_layernorm_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _f32, _vp]),
    "fm_add_layernorm_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _f32, _vp]),
    "fm_layernorm_bwd_workspace": (_sz, [_i64, _i64, _int]),
    "fm_layernorm_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64, _int, _int,
                                _vp]),
    "fm_ce_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _i64, _int, _vp]),
    "fm_ce_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _i64, _vp]),
    "fm_ce_loss_grad": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _i64, _int, _vp]),
    "fm_scale_inplace": (_int, [_vp, _vp, _i64, _int, _vp]),
    "fm_kl_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _f32, _int, _vp]),
    "fm_kl_loss_grad": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _f32, _int, _vp]),
    "fm_kl_fwd_topk": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _int,
                              _f32, _int, _vp]),
    "fm_kl_loss_grad_topk": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _int,
                                    _int, _f32, _int, _vp]),
    "fm_kl_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _i64, _i64, _int, _int, _f32, _f32, _vp]),
    "fm_topk": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _int, _vp]),
    "fm_softmax_fwd": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "fm_softmax_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _vp]),
    "fm_route_workspace": (_sz, [_i64, _int, _int]),
    "fm_moe_gather": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "fm_moe_scatter": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "fm_moe_combine": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "fm_moe_combine_dw": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "fm_swiglu_fwd": (_int, [_vp, _vp, _vp, _i64, _int, _vp]),
    "fm_swiglu_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _vp]),
    "fm_swiglu_split_fwd": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "fm_swiglu_split_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _vp]),
    "fm_qk_norm_rope_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _f32, _vp]),
    "fm_qk_norm_rope_bwd_workspace": (_sz, [_i64, _i64, _i64, _i64]),
    "fm_qk_norm_rope_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64, _i64, _i64,
                                   _int, _int, _vp]),
    "fm_route": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _int, _int, _int, _vp]),
    "fm_route_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _int, _vp]),
}


def _load():
    global _lib, _lib_err
    with _lock:
        if _lib is not None or _lib_err is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            _lib_err = (f"{LIB_PATH} is missing; build it with "
                        "`python -m forgeminds_amd.build` (needs hipcc)")
            return None
        try:
            lib = C.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype, fn.argtypes = res, args
        except (OSError, AttributeError) as exc:
            _lib_err = f"could not load {LIB_PATH}: {exc}"
            return None
        _lib = lib
        return _lib


def loaded() -> bool:
    """True when ``libfmhip.so`` is built and loads in this process."""
    # lock-free once resolved: this sits on the dispatch path, which dynamo also traces
    if _lib is not None:
        return True
    if _lib_err is not None:
        return False
    return _load() is not None


def load_error() -> "str | None":
    _load()
    return _lib_err


def lib():
    """The loaded library; raises if it is missing -- the GPU path never degrades silently."""
    l = _lib if _lib is not None else _load()
    if l is None:
        raise RuntimeError(f"forgeminds_amd: HIP extension unavailable: {_lib_err}")
    return l


def reset_for_tests() -> None:
    """Forget a failed load (used after the test-suite builds the library)."""
    global _lib, _lib_err
    with _lock:
        _lib, _lib_err = None, None


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise RuntimeError(f"forgeminds_amd: dtype {dt} is not supported by the HIP kernels") from None


def _ptr(t: "torch.Tensor | None"):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor):
    """The raw ``hipStream_t`` torch is currently enqueueing on for ``t``'s device."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


_SAME_DEVICE = contextlib.nullcontext()


_current_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _guard(dev: torch.device):
    """Make ``dev`` current for the launch; free when it already is (the usual case)."""
    if dev.index is None or dev.index == _current_device():
        return _SAME_DEVICE
    return torch.cuda.device(dev)


def _rows(x: torch.Tensor):
    """(rows, width) of a dense tensor whose last dimension is the row."""
    d = x.shape[-1]
    return x.numel() // d, d


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().fm_last_error()
        raise RuntimeError(f"{what} failed (status {rc}): {msg.decode() if msg else ''}")


def _dense(*ts):
    for t in ts:
        if t is not None and not t.is_contiguous():
            raise RuntimeError("forgeminds_amd: the HIP kernels take contiguous tensors")


def last_kernel() -> str:
    """Name of the last main kernel this thread enqueued (template arguments resolved)."""
    return lib().fm_last_kernel().decode()


def set_param(name: str, value: int) -> None:
    _check(lib().fm_set_param(name.encode(), int(value)), "fm_set_param")
    # workspace sizes follow the launch shapes, which the tuning parameters move
    for cache in _SIZE_CACHES:
        cache.clear()


_SIZE_CACHES: list = []


# ------------------------------------------------------------------ norm
def rmsnorm_fwd(x2: torch.Tensor, w: torch.Tensor, eps: float):
    """x2 [..., d] contiguous, w [d] -> (y like x2, rstd [rows] fp32)."""
    _dense(x2, w)
    n, d = _rows(x2)
    y = torch.empty_like(x2)
    rstd = torch.empty(n, device=x2.device, dtype=torch.float32)
    with _guard(x2.device):
        _check(lib().fm_rmsnorm_fwd(_ptr(x2), _ptr(w), _ptr(y), _ptr(rstd), n, d,
                                    dtype_code(x2.dtype), dtype_code(w.dtype), float(eps),
                                    _stream(x2)), "fm_rmsnorm_fwd")
    return y, rstd


_WS_BYTES: dict = {}     # (device, rows, width, dtype) -> bytes, until a tuning parameter changes
_SIZE_CACHES.append(_WS_BYTES)


def _norm_ws(n: int, d: int, x: torch.Tensor, want_dw: bool):
    if not want_dw:
        return None, 0
    key = (x.device.index, n, d, x.dtype)
    nbytes = _WS_BYTES.get(key)
    if nbytes is None:
        nbytes = _WS_BYTES[key] = int(lib().fm_rmsnorm_bwd_workspace(n, d, dtype_code(x.dtype)))
    return torch.empty(max(nbytes, 16), device=x.device, dtype=torch.uint8), nbytes


def rmsnorm_bwd(x2, w, rstd, dy2, want_dw: bool = True):
    """-> (dx [n, d], dw [d] in w.dtype or None)."""
    _dense(x2, w, rstd, dy2)
    n, d = _rows(x2)
    dx = torch.empty_like(x2)
    dw = torch.empty_like(w) if want_dw else None
    with _guard(x2.device):
        ws, nbytes = _norm_ws(n, d, x2, want_dw)
        _check(lib().fm_rmsnorm_bwd(_ptr(x2), _ptr(w), _ptr(rstd), _ptr(dy2), _ptr(dx), _ptr(dw),
                                    _ptr(ws), nbytes, n, d, dtype_code(x2.dtype),
                                    dtype_code(w.dtype), _stream(x2)), "fm_rmsnorm_bwd")
    return dx, dw


def add_rmsnorm_fwd(x2, delta2, w, eps: float):
    """-> (xn [n, d], y [n, d], rstd [n] fp32)."""
    _dense(x2, delta2, w)
    n, d = _rows(x2)
    xn = torch.empty_like(x2)
    y = torch.empty_like(x2)
    rstd = torch.empty(n, device=x2.device, dtype=torch.float32)
    with _guard(x2.device):
        _check(lib().fm_add_rmsnorm_fwd(_ptr(x2), _ptr(delta2), _ptr(w), _ptr(xn), _ptr(y),
                                        _ptr(rstd), n, d, dtype_code(x2.dtype),
                                        dtype_code(w.dtype), float(eps), _stream(x2)),
               "fm_add_rmsnorm_fwd")
    return xn, y, rstd


def add_rmsnorm_bwd(xn2, w, rstd, gy2, gxn2, want_dw: bool = True):
    """-> (dx [n, d] (== ddelta), dw or None). gxn2 may be None (no gradient on the sum)."""
    _dense(xn2, w, rstd, gy2, gxn2)
    n, d = _rows(xn2)
    dx = torch.empty_like(xn2)
    dw = torch.empty_like(w) if want_dw else None
    with _guard(xn2.device):
        ws, nbytes = _norm_ws(n, d, xn2, want_dw)
        _check(lib().fm_add_rmsnorm_bwd(_ptr(xn2), _ptr(w), _ptr(rstd), _ptr(gy2), _ptr(gxn2),
                                        _ptr(dx), None, _ptr(dw), _ptr(ws), nbytes, n, d,
                                        dtype_code(xn2.dtype), dtype_code(w.dtype),
                                        _stream(xn2)), "fm_add_rmsnorm_bwd")
    return dx, dw


def layernorm_fwd(x2, w, b, eps: float, delta2=None):
    """-> (xn or None, y [n, d], mean [n], rstd [n]); with ``delta2`` the residual-add form."""
    _dense(x2, w, b, delta2)
    n, d = _rows(x2)
    y = torch.empty_like(x2)
    stats = torch.empty(2, n, device=x2.device, dtype=torch.float32)
    xn = torch.empty_like(x2) if delta2 is not None else None
    with _guard(x2.device):
        if delta2 is None:
            _check(lib().fm_layernorm_fwd(_ptr(x2), _ptr(w), _ptr(b), _ptr(y), stats[0].data_ptr(),
                                          stats[1].data_ptr(), n, d, dtype_code(x2.dtype),
                                          dtype_code(w.dtype), float(eps), _stream(x2)), "fm_layernorm_fwd")
        else:
            _check(lib().fm_add_layernorm_fwd(_ptr(x2), _ptr(delta2), _ptr(w), _ptr(b), _ptr(xn), _ptr(y),
                                              stats[0].data_ptr(), stats[1].data_ptr(), n, d,
                                              dtype_code(x2.dtype), dtype_code(w.dtype), float(eps),
                                              _stream(x2)), "fm_add_layernorm_fwd")
    return xn, y, stats[0], stats[1]


def layernorm_bwd(x2, w, mean, rstd, dy2, gxn2=None, want_dw: bool = True, want_db: bool = True):
    """-> (dx [n, d], dw or None, db or None); ``x2`` is the normalised input (xn of the add form)."""
    _dense(x2, w, mean, rstd, dy2, gxn2)
    n, d = _rows(x2)
    dx = torch.empty_like(x2)
    dw = torch.empty_like(w) if want_dw else None
    db = torch.empty_like(w) if want_db else None
    with _guard(x2.device):
        ws, nbytes = None, 0
        if want_dw or want_db:
            nbytes = int(lib().fm_layernorm_bwd_workspace(n, d, dtype_code(x2.dtype)))
            ws = torch.empty(max(nbytes, 16), device=x2.device, dtype=torch.uint8)
        _check(lib().fm_layernorm_bwd(_ptr(x2), _ptr(w), _ptr(mean), _ptr(rstd), _ptr(dy2), _ptr(gxn2),
                                      _ptr(dx), _ptr(dw), _ptr(db), _ptr(ws), nbytes, n, d,
                                      dtype_code(x2.dtype), dtype_code(w.dtype), _stream(x2)),
               "fm_layernorm_bwd")
    return dx, dw, db


# ------------------------------------------------------------------ cross entropy
def ce_fwd(logits2, labels, ignore_index: int, reduction: str, for_backward: bool = True):
    """logits2 [n, v], labels [n] int64 -> (loss fp32 scalar, lse [n], n_valid fp32 scalar, row_loss).

    ``for_backward=False`` (no gradient will be asked for) passes no ``lse`` buffer: the library then
    streams the logits past the caches throughout instead of leaving their last 256 MB where a
    backward would find them, and ``lse`` comes back as None."""
    _dense(logits2, labels)
    n, v = logits2.shape
    dev = logits2.device
    lse = torch.empty(n, device=dev, dtype=torch.float32) if for_backward else None
    row_loss = torch.empty(n, device=dev, dtype=torch.float32)
    scal = torch.empty(2, device=dev, dtype=torch.float32)
    with _guard(dev):
        _check(lib().fm_ce_fwd(_ptr(logits2), _ptr(labels), _ptr(lse), _ptr(row_loss),
                               scal.data_ptr(), scal.data_ptr() + 4, n, v,
                               dtype_code(logits2.dtype), int(ignore_index), REDUCE[reduction],
                               _stream(logits2)), "fm_ce_fwd")
    return scal[0], lse, scal[1], row_loss


def ce_loss_grad(logits2, labels, ignore_index: int, reduction: str, inplace: bool = False):
    """-> (loss fp32 scalar, dlogits [n, v], n_valid, row_loss); the gradient is for an upstream
    gradient of 1 and lands in ``logits2`` itself when ``inplace``."""
    _dense(logits2, labels)
    n, v = logits2.shape
    dev = logits2.device
    buf = torch.empty(2, max(n, 1), device=dev, dtype=torch.float32)
    scalars = torch.empty(2, device=dev, dtype=torch.float32)
    dl = logits2 if inplace else torch.empty_like(logits2)
    with _guard(dev):
        _check(lib().fm_ce_loss_grad(_ptr(logits2), _ptr(labels), buf[0].data_ptr(), buf[1].data_ptr(),
                                     scalars[0:].data_ptr(), scalars[1:].data_ptr(), _ptr(dl), n, v,
                                     dtype_code(logits2.dtype), int(ignore_index), REDUCE[reduction],
                                     _stream(logits2)), "fm_ce_loss_grad")
    return scalars[0], dl, scalars[1], buf[1][:n]


def scale_inplace(x, factor):
    """x *= factor (fp32 device scalar), skipped on the device when the factor is exactly 1."""
    _dense(x, factor)
    with _guard(x.device):
        _check(lib().fm_scale_inplace(_ptr(x), _ptr(factor), x.numel(), dtype_code(x.dtype), _stream(x)),
               "fm_scale_inplace")
    return x


def ce_bwd(logits2, labels, lse, n_valid, grad_out, ignore_index: int):
    """-> dlogits [n, v]; n_valid / grad_out are fp32 device scalars or None."""
    _dense(logits2, labels, lse)
    n, v = logits2.shape
    dl = torch.empty_like(logits2)
    with _guard(logits2.device):
        _check(lib().fm_ce_bwd(_ptr(logits2), _ptr(labels), _ptr(lse), _ptr(n_valid),
                               _ptr(grad_out), _ptr(dl), n, v, dtype_code(logits2.dtype),
                               int(ignore_index), _stream(logits2)), "fm_ce_bwd")
    return dl


# ------------------------------------------------------------------ KL
def kl_fwd(s2, t2, inv_temperature: float, reduction: str):
    """-> (loss fp32 scalar or None, row_kl [n], lse_s [n], lse_t [n])."""
    _dense(s2, t2)
    n, v = s2.shape
    dev = s2.device
    buf = torch.empty(3, n, device=dev, dtype=torch.float32)
    loss = torch.empty((), device=dev, dtype=torch.float32) if reduction != "none" else None
    with _guard(dev):
        _check(lib().fm_kl_fwd(_ptr(s2), _ptr(t2), buf[0].data_ptr(), buf[1].data_ptr(),
                               buf[2].data_ptr(), _ptr(loss), n, v, dtype_code(s2.dtype),
                               float(inv_temperature), REDUCE[reduction], _stream(s2)), "fm_kl_fwd")
    return loss, buf[2], buf[0], buf[1]


def kl_loss_grad(s2, t2, inv_temperature: float, reduction: str, grad_dtype, inplace: bool = False):
    """-> (loss fp32 scalar, dstudent [n, v], row_kl); the gradient is for an upstream gradient of 1
    and lands in ``s2`` itself when ``inplace`` and the gradient has the student's dtype."""
    _dense(s2, t2)
    n, v = s2.shape
    dev = s2.device
    buf = torch.empty(3, n, device=dev, dtype=torch.float32)
    loss = torch.empty((), device=dev, dtype=torch.float32)
    inplace = inplace and grad_dtype == s2.dtype
    g = s2 if inplace else torch.empty((n, v), device=dev, dtype=grad_dtype)
    with _guard(dev):
        _check(lib().fm_kl_loss_grad(_ptr(s2), _ptr(t2), buf[0].data_ptr(), buf[1].data_ptr(),
                                     buf[2].data_ptr(), _ptr(loss), _ptr(g), n, v, dtype_code(s2.dtype),
                                     dtype_code(grad_dtype), float(inv_temperature), REDUCE[reduction],
                                     _stream(s2)), "fm_kl_loss_grad")
    return loss, g, buf[2]


def kl_fwd_topk(s2, t2, k: int, inv_temperature: float, reduction: str, index_dtype=torch.int64,
                want_values: bool = False, want_probs: bool = True, want_grad: bool = False):
    """-> (loss or None, row_kl, lse_s, lse_t, values or None, idx, probs or None); None when the
    shape is outside what the fused kernel takes (the caller then runs the two kernels).
    ``want_grad`` (reduction sum or mean) appends the student's gradient for an upstream
    gradient of 1, written by the same launch."""
    _dense(s2, t2)
    n, v = s2.shape
    dev = s2.device
    grad = torch.empty_like(s2) if want_grad else None
    buf = torch.empty(3, n, device=dev, dtype=torch.float32)
    loss = torch.empty((), device=dev, dtype=torch.float32) if reduction != "none" else None
    vals = torch.empty((n, k), device=dev, dtype=t2.dtype) if want_values else None
    probs = torch.empty((n, k), device=dev, dtype=torch.float32) if want_probs else None
    idx = torch.empty((n, k), device=dev, dtype=index_dtype)
    bits = 64 if index_dtype == torch.int64 else 32
    with _guard(dev):
        if want_grad:
            rc = lib().fm_kl_loss_grad_topk(_ptr(s2), _ptr(t2), buf[0].data_ptr(), buf[1].data_ptr(),
                                            buf[2].data_ptr(), _ptr(loss), _ptr(grad), _ptr(vals), _ptr(idx),
                                            _ptr(probs), n, v, int(k), dtype_code(s2.dtype), bits,
                                            float(inv_temperature), REDUCE[reduction], _stream(s2))
        else:
            rc = lib().fm_kl_fwd_topk(_ptr(s2), _ptr(t2), buf[0].data_ptr(), buf[1].data_ptr(),
                                      buf[2].data_ptr(), _ptr(loss), _ptr(vals), _ptr(idx), _ptr(probs),
                                      n, v, int(k), dtype_code(s2.dtype), bits, float(inv_temperature),
                                      REDUCE[reduction], _stream(s2))
    if rc == 2:   # FM_ERR_UNSUPPORTED
        return None
    _check(rc, "fm_kl_loss_grad_topk" if want_grad else "fm_kl_fwd_topk")
    if want_grad:
        return loss, buf[2], buf[0], buf[1], vals, idx, probs, grad
    return loss, buf[2], buf[0], buf[1], vals, idx, probs


def kl_bwd(s2, t2, lse_s, lse_t, grad_out, per_row: bool, grad_dtype, inv_temperature: float,
           scale: float):
    _dense(s2, t2, lse_s, lse_t, grad_out)
    n, v = s2.shape
    g = torch.empty((n, v), device=s2.device, dtype=grad_dtype)
    with _guard(s2.device):
        _check(lib().fm_kl_bwd(_ptr(s2), _ptr(t2), _ptr(lse_s), _ptr(lse_t), _ptr(grad_out),
                               1 if per_row else 0, _ptr(g), n, v, dtype_code(s2.dtype),
                               dtype_code(grad_dtype), float(inv_temperature), float(scale),
                               _stream(s2)), "fm_kl_bwd")
    return g


# ------------------------------------------------------------------ top-k / softmax / router
def topk(x2, k: int, index_dtype=torch.int64, want_values: bool = True):
    _dense(x2)
    n, v = x2.shape
    vals = torch.empty((n, k), device=x2.device, dtype=x2.dtype) if want_values else None
    idx = torch.empty((n, k), device=x2.device, dtype=index_dtype)
    bits = 64 if index_dtype == torch.int64 else 32
    with _guard(x2.device):
        _check(lib().fm_topk(_ptr(x2), _ptr(vals), _ptr(idx), n, v, int(k), dtype_code(x2.dtype),
                             bits, _stream(x2)), "fm_topk")
    return vals, idx


def softmax_fwd(x2):
    _dense(x2)
    n, v = x2.shape
    y = torch.empty_like(x2)
    with _guard(x2.device):
        _check(lib().fm_softmax_fwd(_ptr(x2), _ptr(y), n, v, dtype_code(x2.dtype), _stream(x2)),
               "fm_softmax_fwd")
    return y


def softmax_bwd(y2, dy2):
    """dx = (dy - sum(dy * y, -1)) * y for y2 = softmax(x2)."""
    _dense(y2, dy2)
    n, v = y2.shape
    dx = torch.empty_like(y2)
    with _guard(y2.device):
        _check(lib().fm_softmax_bwd(_ptr(y2), _ptr(dy2), _ptr(dx), n, v, dtype_code(y2.dtype),
                                    _stream(y2)), "fm_softmax_bwd")
    return dx


_ROUTE_WS: dict = {}     # (rows, experts, k) -> workspace bytes, until a tuning parameter changes
_SIZE_CACHES.append(_ROUTE_WS)


def route(logits2, k: int, want_permutation: bool = True, want_stats: bool = False):
    """-> (idx int32 [n, k], weights fp32 [n, k], counts int32 [e], slot, order int32 [n*k])
    and, with want_stats, a sixth item: fp32 [e+3] = column sums of probs, sum(lse^2), then the
    load-balance loss and the z-loss themselves."""
    _dense(logits2)
    n, e = logits2.shape
    dev = logits2.device
    idx = torch.empty((n, k), device=dev, dtype=torch.int32)
    wts = torch.empty((n, k), device=dev, dtype=torch.float32)
    counts = torch.empty(e, device=dev, dtype=torch.int32)
    slot = torch.empty(n * k, device=dev, dtype=torch.int32) if want_permutation else None
    order = torch.empty(n * k, device=dev, dtype=torch.int32) if want_permutation else None
    stats = torch.empty(e + 3, device=dev, dtype=torch.float32) if want_stats else None
    with _guard(dev):
        key = (n, e, k)
        nbytes = _ROUTE_WS.get(key)
        if nbytes is None:
            nbytes = _ROUTE_WS[key] = int(lib().fm_route_workspace(n, e, k))
        ws = torch.empty(max(nbytes, 16), device=dev, dtype=torch.uint8)
        _check(lib().fm_route(_ptr(logits2), _ptr(idx), _ptr(wts), _ptr(counts), _ptr(slot),
                              _ptr(order), _ptr(stats), _ptr(ws), nbytes, n, e, int(k),
                              dtype_code(logits2.dtype), _stream(logits2)), "fm_route")
    if want_stats:
        return idx, wts, counts, slot, order, stats
    return idx, wts, counts, slot, order


def route_bwd(logits2, idx, gweights, counts, g_aux, g_z):
    """-> dlogits like logits2. gweights fp32 [n, k] or None; g_aux / g_z fp32 device scalars or
    None (g_aux needs counts)."""
    _dense(logits2, idx, gweights, counts)
    n, e = logits2.shape
    k = idx.shape[1]
    out = torch.empty_like(logits2)
    with _guard(logits2.device):
        _check(lib().fm_route_bwd(_ptr(logits2), _ptr(idx), _ptr(gweights), _ptr(counts), _ptr(g_aux),
                                  _ptr(g_z), _ptr(out), n, e, int(k), dtype_code(logits2.dtype),
                                  _stream(logits2)), "fm_route_bwd")
    return out


# ------------------------------------------------------------------ token moves around the permutation
def moe_gather(x2, order, k: int, scale_flat=None):
    """x2 [n, d], order int32 [n*k] -> xs [n*k, d] = scale * x2[order // k]."""
    _dense(x2, order, scale_flat)
    n, d = x2.shape
    xs = torch.empty((n * k, d), device=x2.device, dtype=x2.dtype)
    with _guard(x2.device):
        _check(lib().fm_moe_gather(_ptr(x2), _ptr(order), _ptr(scale_flat), _ptr(xs), n, d, int(k),
                                   dtype_code(x2.dtype), _stream(x2)), "fm_moe_gather")
    return xs


def moe_scatter(x2, slot, k: int, scale_flat=None):
    """x2 [n, d], slot int32 [n*k] -> xs [n*k, d] with xs[slot[t*k+j]] = scale * x2[t]: the result of
    ``moe_gather`` from the token's side (each token row is read once)."""
    _dense(x2, slot, scale_flat)
    n, d = x2.shape
    xs = torch.empty((n * k, d), device=x2.device, dtype=x2.dtype)
    with _guard(x2.device):
        _check(lib().fm_moe_scatter(_ptr(x2), _ptr(slot), _ptr(scale_flat), _ptr(xs), n, d, int(k),
                                    dtype_code(x2.dtype), _stream(x2)), "fm_moe_scatter")
    return xs


def moe_combine(ys, weights, slot, n: int, k: int):
    """ys [n*k, d], weights fp32 [n, k] or None, slot int32 [n*k] -> out [n, d]."""
    _dense(ys, weights, slot)
    d = ys.shape[1]
    out = torch.empty((n, d), device=ys.device, dtype=ys.dtype)
    with _guard(ys.device):
        _check(lib().fm_moe_combine(_ptr(ys), _ptr(weights), _ptr(slot), _ptr(out), n, d, int(k),
                                    dtype_code(ys.dtype), _stream(ys)), "fm_moe_combine")
    return out


def moe_combine_dw(ys, dout, slot, n: int, k: int):
    """-> dweights fp32 [n, k] = <ys[slot[t*k+j]], dout[t]>."""
    _dense(ys, dout, slot)
    d = ys.shape[1]
    dw = torch.empty((n, k), device=ys.device, dtype=torch.float32)
    with _guard(ys.device):
        _check(lib().fm_moe_combine_dw(_ptr(ys), _ptr(dout), _ptr(slot), _ptr(dw), n, d, int(k),
                                       dtype_code(ys.dtype), _stream(ys)), "fm_moe_combine_dw")
    return dw


# ------------------------------------------------------------------ SwiGLU epilogues
def swiglu_fwd(gate, up):
    _dense(gate, up)
    y = torch.empty_like(gate)
    with _guard(gate.device):
        _check(lib().fm_swiglu_fwd(_ptr(gate), _ptr(up), _ptr(y), gate.numel(), dtype_code(gate.dtype),
                                   _stream(gate)), "fm_swiglu_fwd")
    return y


def swiglu_bwd(gate, up, dy):
    _dense(gate, up, dy)
    dg, du = torch.empty_like(gate), torch.empty_like(up)
    with _guard(gate.device):
        _check(lib().fm_swiglu_bwd(_ptr(gate), _ptr(up), _ptr(dy), _ptr(dg), _ptr(du), gate.numel(),
                                   dtype_code(gate.dtype), _stream(gate)), "fm_swiglu_bwd")
    return dg, du


def swiglu_split_fwd(x2):
    """x2 [rows, 2h] -> y [rows, h]."""
    _dense(x2)
    rows, w = x2.shape
    y = torch.empty((rows, w // 2), device=x2.device, dtype=x2.dtype)
    with _guard(x2.device):
        _check(lib().fm_swiglu_split_fwd(_ptr(x2), _ptr(y), rows, w // 2, dtype_code(x2.dtype),
                                         _stream(x2)), "fm_swiglu_split_fwd")
    return y


def swiglu_split_bwd(x2, dy2):
    _dense(x2, dy2)
    rows, w = x2.shape
    dx = torch.empty_like(x2)
    with _guard(x2.device):
        _check(lib().fm_swiglu_split_bwd(_ptr(x2), _ptr(dy2), _ptr(dx), rows, w // 2,
                                         dtype_code(x2.dtype), _stream(x2)), "fm_swiglu_split_bwd")
    return dx


# ------------------------------------------------------------------ per-head RMSNorm + RoPE
def qk_norm_rope_fwd(x4, w, cos, sin, eps: float):
    """x4 [b, t, h, d], cos/sin fp32 [t, d/2] -> (out like x4, rstd fp32 [b*t*h])."""
    _dense(x4, w, cos, sin)
    b, t, h, d = x4.shape
    out = torch.empty_like(x4)
    rstd = torch.empty(b * t * h, device=x4.device, dtype=torch.float32)
    with _guard(x4.device):
        _check(lib().fm_qk_norm_rope_fwd(_ptr(x4), _ptr(w), _ptr(cos), _ptr(sin), _ptr(out), _ptr(rstd),
                                         b, t, h, d, dtype_code(x4.dtype), dtype_code(w.dtype), float(eps),
                                         _stream(x4)), "fm_qk_norm_rope_fwd")
    return out, rstd


def qk_norm_rope_bwd(x4, w, cos, sin, rstd, dout, want_dw: bool = True):
    _dense(x4, w, cos, sin, rstd, dout)
    b, t, h, d = x4.shape
    dx = torch.empty_like(x4)
    dw = torch.empty_like(w) if want_dw else None
    with _guard(x4.device):
        nbytes = int(lib().fm_qk_norm_rope_bwd_workspace(b, t, h, d)) if want_dw else 0
        ws = torch.empty(max(nbytes, 16), device=x4.device, dtype=torch.uint8) if want_dw else None
        _check(lib().fm_qk_norm_rope_bwd(_ptr(x4), _ptr(w), _ptr(cos), _ptr(sin), _ptr(rstd), _ptr(dout),
                                         _ptr(dx), _ptr(dw), _ptr(ws), nbytes, b, t, h, d,
                                         dtype_code(x4.dtype), dtype_code(w.dtype), _stream(x4)),
               "fm_qk_norm_rope_bwd")
    return dx, dw

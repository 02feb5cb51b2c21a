"""CPU oracle for the packed-kernel hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A plain torch/numpy restatement of what the reference (xygamer179-boop/ForgeMinds) computes
on this path, written from its source text. Only ``tests/``, ``__graft_entry__.smoke()`` and
``bench.py``'s ``cpu_baseline`` leg may import this module; nothing under ``forgeminds_amd/``
does. It runs on CPU tensors only and knows nothing about the HIP library.

Every function names the reference lines it follows. Gradients are written as closed forms
(not autograd) so that ``tests/test_oracle.py`` can pin them against torch's own autograd of
the library routines (``F.rms_norm``, ``F.cross_entropy``, ``F.kl_div``), against the
reference's known-answer tests, and against brute-force loops -- a dropped term or a wrong
sign here fails there.

Pinning status (see tests/test_oracle.py): every function below is pinned; none is
"parity unpinned". The reference's own tests hold no value-level vectors for the router
(idx / weights / permutation); those are pinned by the integer closed forms instead
(bincount, stable argsort, inverse permutation) and by brute force on small inputs; the
router's gradient is pinned against torch's autograd of the reference expression.

``acc`` is the accumulation dtype: ``torch.float32`` reproduces the reference's fallback
(fp32 for half inputs, reference forgemind/kernels/_fallback.py:15-23), ``torch.float64`` is
the tighter yardstick used for the fp32-loss tolerances.
"""

from __future__ import annotations

import numpy as np
import torch


def _up(t: torch.Tensor, acc) -> torch.Tensor:
    assert not t.is_cuda, "the oracle is a CPU restatement"
    return t.to(acc)


# ------------------------------------------------------------------ RMSNorm
def rms_norm(x, w, eps=1e-6, acc=torch.float32):
    """y, rstd. Reference forgemind/kernels/_fallback.py:26-30; multiply order (x*r)*w of
    forgemind/kernels/norm.py:170-174; rstd as saved by norm.py:787."""
    xf, wf = _up(x, acc), _up(w, acc)
    rstd = torch.rsqrt((xf * xf).mean(dim=-1, keepdim=True) + eps)
    y = ((xf * rstd) * wf).to(x.dtype)
    return y, rstd.squeeze(-1)


def rms_norm_bwd(x, w, dy, eps=1e-6, acc=torch.float32):
    """dx (x.dtype), dw (w.dtype). Row math of forgemind/kernels/norm.py:179-231:
    xh = x*rstd; g = dy*w; dx = rstd/n * (n*g - xh*sum(g*xh)); dw = sum_rows dy*xh
    (norm.py:265-293, cast to w.dtype at norm.py:983)."""
    xf, wf, gf = _up(x, acc), _up(w, acc), _up(dy, acc)
    n = x.shape[-1]
    rstd = torch.rsqrt((xf * xf).mean(dim=-1, keepdim=True) + eps)
    xh = xf * rstd
    g = gf * wf
    dx = rstd / n * (n * g - xh * (g * xh).sum(dim=-1, keepdim=True))
    dw = (gf * xh).reshape(-1, n).sum(dim=0)
    return dx.to(x.dtype), dw.to(w.dtype)


def add_rms_norm(x, delta, w, eps=1e-6, acc=torch.float32):
    """xn, y, rstd. Reference _fallback.py:33-35: the sum is a tensor add in x's dtype (so it
    is rounded for bf16/fp16) and the norm is taken of the rounded sum."""
    xn = x + delta
    y, rstd = rms_norm(xn, w, eps, acc)
    return xn, y, rstd


def add_rms_norm_bwd(xn, w, gy, gxn, eps=1e-6, acc=torch.float32):
    """dx (== ddelta), dw. Reference forgemind/kernels/norm.py:1050-1086:
    dx = (w*gy - xh*c)*r + gxn with c = sum(xh*w*gy)/d, one rounding to x's dtype; ddelta
    is the same values (norm.py:1076-1083); dw = sum_rows gy*xh in fp32 (norm.py:1148).
    `gxn` (gradient of the residual output) may be None."""
    xf, wf, gf = _up(xn, acc), _up(w, acc), _up(gy, acc)
    d = xn.shape[-1]
    r = torch.rsqrt((xf * xf).mean(dim=-1, keepdim=True) + eps)
    xh = xf * r
    wdy = gf * wf
    c = (xh * wdy).sum(dim=-1, keepdim=True) / d
    dx = (wdy - xh * c) * r
    if gxn is not None:
        dx = dx + _up(gxn, acc)
    dw = (gf * xh).reshape(-1, d).sum(dim=0)
    return dx.to(xn.dtype), dw.to(w.dtype)


# ------------------------------------------------------------------ LayerNorm
def layer_norm(x, w, b=None, eps=1e-5, acc=torch.float32):
    """y, mean, rstd. torch.nn.functional.layer_norm's arithmetic in `acc` on the stored
    values, one rounding to x's dtype -- the rounding rule the reference applies to its norm
    fallback (forgemind/kernels/_fallback.py:15-35); the reference has no LayerNorm of its own.
    Biased variance of the centred values, as F.layer_norm."""
    xf, wf = _up(x, acc), _up(w, acc)
    mean = xf.mean(dim=-1, keepdim=True)
    xc = xf - mean
    rstd = torch.rsqrt((xc * xc).mean(dim=-1, keepdim=True) + eps)
    y = (xc * rstd) * wf
    if b is not None:
        y = y + _up(b, acc)
    return y.to(x.dtype), mean.squeeze(-1), rstd.squeeze(-1)


def layer_norm_bwd(x, w, dy, eps=1e-5, gxn=None, acc=torch.float32):
    """dx (x.dtype), dw, db (w.dtype): g = dy*w, xh = (x-mean)*rstd,
    dx = rstd*((g - mean(g)) - xh*mean(g*xh)) [+ gxn]; dw = sum_rows dy*xh; db = sum_rows dy."""
    xf, wf, gf = _up(x, acc), _up(w, acc), _up(dy, acc)
    d = x.shape[-1]
    mean = xf.mean(dim=-1, keepdim=True)
    xc = xf - mean
    rstd = torch.rsqrt((xc * xc).mean(dim=-1, keepdim=True) + eps)
    xh = xc * rstd
    g = gf * wf
    dx = ((g - g.mean(dim=-1, keepdim=True)) - xh * (g * xh).mean(dim=-1, keepdim=True)) * rstd
    if gxn is not None:
        dx = dx + _up(gxn, acc)
    dw = (gf * xh).reshape(-1, d).sum(dim=0)
    db = gf.reshape(-1, d).sum(dim=0)
    return dx.to(x.dtype), dw.to(w.dtype), db.to(w.dtype)


def add_layer_norm(x, delta, w, b=None, eps=1e-5, acc=torch.float32):
    """xn, y, mean, rstd: the sum is a tensor add in x's dtype (rounded for bf16/fp16, as
    forgemind/kernels/_fallback.py:33-35 does for RMSNorm), the norm is taken of the rounded sum."""
    xn = x + delta
    y, mean, rstd = layer_norm(xn, w, b, eps, acc)
    return xn, y, mean, rstd


# ------------------------------------------------------------------ cross entropy
def cross_entropy(logits, labels, ignore_index=-100, acc=torch.float32):
    """loss (0-d, `acc`), dlogits (logits.dtype) for upstream gradient 1.

    Reference forgemind/loss.py:54-70: n = max(1, #(labels != ignore_index));
    loss = sum over valid rows of (logsumexp(row) - row[label]) / n. The arithmetic is
    torch's F.cross_entropy (not in the reference tree; torch>=2.6 per its pyproject.toml:10),
    restated as logsumexp. Gradient (what autograd derives): (softmax(row) - onehot) / n on
    valid rows, 0 on ignored rows. Math in `acc` on the logits' values: the literal bf16 call
    of loss.py:65 rounds each chunk sum to bf16, which is not the contract tested here."""
    lg = _up(logits.reshape(-1, logits.shape[-1]), acc)
    y = labels.reshape(-1)
    valid = y != ignore_index
    n = max(1, int(valid.sum()))
    if lg.shape[0] == 0:
        return torch.zeros((), dtype=acc), torch.zeros_like(logits)
    lse = torch.logsumexp(lg, dim=-1)
    safe = torch.where(valid, y, torch.zeros_like(y))
    picked = lg.gather(1, safe[:, None]).squeeze(1)
    rows = torch.where(valid, lse - picked, torch.zeros_like(lse))
    loss = rows.sum() / n
    p = torch.exp(lg - lse[:, None])
    p[torch.arange(lg.shape[0]), safe] -= 1.0
    grad = torch.where(valid[:, None], p / n, torch.zeros_like(p))
    return loss, grad.to(logits.dtype).reshape(logits.shape)


# ------------------------------------------------------------------ KL(teacher || student)
def kl_div(student, teacher, reduction="mean", temperature=1.0, acc=torch.float32):
    """loss, dstudent (student.dtype) for upstream gradient 1 (per-row 1 for "none").

    Reference forgemind/kernels/_fallback.py:52-69: ls = log_softmax(s), lt = log_softmax(t),
    pt = exp(lt); per_row = sum(pt*(lt-ls)); mean divides by the number of rows (no mask);
    grad = (exp(ls) - pt) * scale. The temperature is this build's extension: both logit
    tensors are divided by T before the softmax and the chain rule adds one factor 1/T."""
    v = student.shape[-1]
    s = _up(student.reshape(-1, v), acc) / temperature
    t = _up(teacher.reshape(-1, v), acc) / temperature
    ls = s - torch.logsumexp(s, dim=-1, keepdim=True)
    lt = t - torch.logsumexp(t, dim=-1, keepdim=True)
    pt = lt.exp()
    rows = (pt * (lt - ls)).sum(dim=-1)
    n = rows.numel()
    if reduction == "none":
        loss, scale = rows.reshape(student.shape[:-1]), 1.0
    elif reduction == "sum":
        loss, scale = rows.sum(), 1.0
    elif reduction == "mean":
        loss, scale = rows.sum() / n, 1.0 / n
    else:
        raise ValueError(f"reduction must be mean|sum|none, got {reduction!r}")
    grad = (ls.exp() - pt) * (scale / temperature)
    return loss, grad.to(student.dtype).reshape(student.shape)


# ------------------------------------------------------------------ softmax
def softmax(x, acc=torch.float32):
    """Reference forgemind/kernels/softmax.py:27-80: exp(x - max) / sum, stored in x.dtype."""
    xf = _up(x, acc)
    e = torch.exp(xf - xf.max(dim=-1, keepdim=True).values)
    return (e / e.sum(dim=-1, keepdim=True)).to(x.dtype)


def softmax_bwd(y, dy, acc=torch.float32):
    """Reference forgemind/kernels/softmax.py:108-115: (dy - sum(dy * y)) * y from the saved
    output, here in ``acc`` on the stored values with one rounding to y.dtype."""
    yf, gf = _up(y, acc), _up(dy, acc)
    return ((gf - (gf * yf).sum(dim=-1, keepdim=True)) * yf).to(y.dtype)


# ------------------------------------------------------------------ top-k (canonical order)
def topk(x, k):
    """values (x.dtype), indices (int64). Canonical order of forgemind/kernels/topk.py:13-19,
    276-281: value descending, index ascending inside ties, smallest indices win at the k-th
    value, NaN is the largest value and passes through; -0.0 == +0.0.

    Implemented as a lexicographic sort on (-value, index) per row in float64 (exact for
    fp32/fp16/bf16 inputs), which is the definition itself rather than an algorithm."""
    n = x.shape[-1]
    if x.dim() < 1:
        raise ValueError(f"topk needs ndim >= 1, got shape {tuple(x.shape)}")
    if k < 1 or k > n:
        raise RuntimeError(f"selected index k out of range (got {k} vs {n})")
    rows = x.reshape(-1, n)
    val = rows.to(torch.float64).numpy()
    key = np.where(np.isnan(val), np.inf, val)          # NaN ties with nothing below it ...
    is_nan = np.isnan(val)
    cols = np.broadcast_to(np.arange(n), val.shape)
    # primary: NaN first; then value descending; then index ascending
    out = np.ascontiguousarray(np.lexsort((cols, -key, ~is_nan), axis=-1)[:, :k]).astype(np.int64)
    idx = torch.from_numpy(out)
    vals = torch.gather(rows, 1, idx)
    shape = x.shape[:-1] + (k,)
    return vals.reshape(shape), idx.reshape(shape)


# ------------------------------------------------------------------ MoE router + permutation
def router(logits, k):
    """idx int64 [n,k], weights fp32 [n,k], counts int64 [e], slot int64 [n*k], order int64 [n*k].

    Reference forgemind/moe.py:86-91: probs = softmax(logits.float()); (w, idx) = topk(probs, k);
    w = w / w.sum(-1). torch.topk's tie order is unspecified, so ties follow the canonical
    order of kernels/topk.py:13-16 (lowest index first).
    counts: moe.py:52-60 (zeros + scatter_add == bincount).
    order: moe.py:233 `torch.sort(flat, stable=True).indices` with flat[p] = idx[p // k, p % k];
    slot is its inverse permutation (slot[order[s]] == s)."""
    probs = torch.softmax(_up(logits, torch.float32), dim=-1)
    top_p, idx = topk(probs, k)
    weights = top_p / top_p.sum(dim=-1, keepdim=True)
    flat = idx.reshape(-1).numpy()
    e = logits.shape[-1]
    counts = np.bincount(flat, minlength=e).astype(np.int64)
    order = np.argsort(flat, kind="stable").astype(np.int64)
    slot = np.empty_like(order)
    slot[order] = np.arange(order.size, dtype=np.int64)
    return (idx, weights, torch.from_numpy(counts), torch.from_numpy(slot),
            torch.from_numpy(order))


def router_aux(logits, idx):
    """aux, z of forgemind/moe.py:92-95: aux = E * sum(frac * mean_rows(probs)),
    frac = counts / idx.numel(); z = mean(logsumexp(logits)^2)."""
    lf = _up(logits, torch.float32)
    probs = torch.softmax(lf, dim=-1)
    e = logits.shape[-1]
    counts = torch.from_numpy(np.bincount(idx.reshape(-1).numpy(), minlength=e)).to(torch.float32)
    frac = counts / max(idx.numel(), 1)
    aux = e * (frac * probs.mean(dim=0)).sum()
    z = torch.logsumexp(lf, dim=-1).pow(2).mean()
    return aux, z


def router_bwd(logits, k, gweights=None, g_aux=None, g_z=None, acc=torch.float64):
    """d(sum(weights * gweights) + g_aux * aux + g_z * z) / d logits, [n, e] in `acc`.

    The closed form of what autograd derives from the reference's Router.forward
    (forgemind/moe.py:86-95), with the top-k indices and the per-expert fractions held constant
    (moe.py:92-93 computes `frac` under no_grad; indices carry no gradient):
      w_j = p[idx_j] / S, S = sum_j p[idx_j]   ->  g_p[idx_j] = (gw_j - sum_i gw_i w_i) / S
      aux = E * sum_e frac_e * mean_rows(p)_e  ->  g_p[e] += g_aux * E / n * frac_e
      softmax                                  ->  g_x = (g_p - sum_e g_p p) p
      z = mean_rows(lse^2)                     ->  g_x += g_z * 2 / n * lse * p."""
    idx, _w, counts, _slot, _order = router(logits, k)
    n, e = logits.shape
    lf = _up(logits, torch.float32).to(acc)
    lse = torch.logsumexp(lf, dim=-1, keepdim=True)
    p = torch.exp(lf - lse)
    g_p = torch.zeros_like(p)
    if gweights is not None:
        pk = torch.gather(p, 1, idx)
        s = pk.sum(dim=-1, keepdim=True)
        gw = gweights.to(acc)
        g_p.scatter_(1, idx, (gw - (gw * pk / s).sum(dim=-1, keepdim=True)) / s)
    if g_aux is not None:
        g_p = g_p + float(g_aux) * (e / max(n, 1)) * (counts.to(acc) / max(idx.numel(), 1))
    g = (g_p - (g_p * p).sum(dim=-1, keepdim=True)) * p
    if g_z is not None:
        g = g + float(g_z) * (2.0 / max(n, 1)) * lse * p
    return g


# ------------------------------------------------------------------ token moves around the permutation
def moe_gather(x, order, k):
    """xs = x[order // k]. Reference forgemind/moe.py:234-235 (tok = order // top_k; xs = x[tok])."""
    return x[(order // k).long()]


def moe_combine(ys, weights, order, k, n):
    """out [n, d]. Reference forgemind/moe.py:247-248, rounding points included:
    ys = ys * w.reshape(-1)[order].unsqueeze(-1)   (product in ys' dtype, w in the activation dtype)
    out = zeros_like(x).index_add_(0, order // k, ys)   (accumulated in the activation dtype)."""
    w = weights.to(ys.dtype).reshape(-1)[order.long()].unsqueeze(-1)
    scaled = ys * w
    out = torch.zeros(n, ys.shape[1], dtype=ys.dtype)
    return out.index_add_(0, (order // k).long(), scaled)

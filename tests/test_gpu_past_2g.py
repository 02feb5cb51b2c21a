"""Tensors of more than 2**31 elements (the reference's gate stops below that,
``forgemind/kernels/_common.py:114``; this library takes them): every offset is 64-bit.

Row-local outputs of the big call are compared bit for bit with the same kernel on a handful of
rows cut out of the big tensor (first rows, the rows around element 2**31, last rows), whose own
parity against the oracle the other test files establish, and against the oracle directly on
those rows. Whole-tensor outputs (losses, weight gradients) are checked against reductions of
the per-row outputs done with plain tensor ops on the GPU."""

import pytest
import torch

from forgeminds_amd.kernels import _hip
from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF16 = torch.bfloat16


def picks(n, width):
    b = 2 ** 31 // width
    rows = sorted(set([0, 1] + list(range(b - 2, b + 3)) + [n - 2, n - 1]))
    return torch.tensor([r for r in rows if 0 <= r < n], device=DEV)


def randn(shape, seed, scale=1.0, dtype=BF16):
    g = torch.Generator(device=DEV).manual_seed(seed)
    out = torch.empty(shape, device=DEV, dtype=dtype)
    rows = shape[0]
    step = max(1, 2 ** 28 // max(1, out[0].numel()))       # fp32 temporaries of at most 1 GiB
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        out[r0:r1] = (scale * torch.randn((r1 - r0,) + tuple(shape[1:]), device=DEV, generator=g)).to(dtype)
    return out


def lowp_close(got, ref, ulps=3.0, cancel=0.0):
    got, ref = got.float().cpu(), ref.float().cpu()
    scale = ref.abs().max()
    bound = ulps * 2.0 ** -8 * ref.abs() + 1e-6 * scale + 8 * 2.0 ** -23 * cancel
    return bool(((got - ref).abs() <= bound).all())


def test_add_rmsnorm_past_2g():
    n, d = 262176, 8192
    assert n * d > 2 ** 31
    x, delta = randn((n, d), 1), randn((n, d), 2)
    w = (1 + 0.02 * torch.randn(d, generator=torch.Generator().manual_seed(3))).to(DEV)
    xn, y, rstd = _hip.add_rmsnorm_fwd(x, delta, w, 1e-5)
    p = picks(n, d)
    sxn, sy, srstd = _hip.add_rmsnorm_fwd(x[p], delta[p], w, 1e-5)
    assert torch.equal(xn[p], sxn) and torch.equal(y[p], sy) and torch.equal(rstd[p], srstd)
    oxn, oy, _ = O.add_rms_norm(x[p].cpu(), delta[p].cpu(), w.cpu(), 1e-5)
    assert torch.equal(xn[p].cpu(), oxn) and lowp_close(y[p], oy, 2.0)
    del x, delta, y
    gy, gxn = randn((n, d), 4), randn((n, d), 5)
    dx, dw = _hip.add_rmsnorm_bwd(xn, w, rstd, gy, gxn)
    sdx, _ = _hip.add_rmsnorm_bwd(xn[p], w, rstd[p], gy[p], gxn[p])
    assert torch.equal(dx[p], sdx)
    odx, _ = O.add_rms_norm_bwd(xn[p].cpu(), w.cpu(), gy[p].cpu(), gxn[p].cpu(), 1e-5)
    assert lowp_close(dx[p], odx, 3.0, cancel=8.0)
    ref = torch.zeros(d, device=DEV, dtype=torch.float64)
    for r0 in range(0, n, 16384):
        sl = slice(r0, min(n, r0 + 16384))
        ref += (gy[sl].float() * (xn[sl].float() * rstd[sl, None])).double().sum(0)
    assert ((dw.double() - ref).abs().max() / ref.abs().max()).item() < 1e-4


def test_rmsnorm_narrow_rows_past_2g():
    n, d = 2 ** 24 + 64, 128                # the several-rows-per-wave form of the norm kernels
    x = randn((n, d), 6)
    w = (1 + 0.02 * torch.randn(d, generator=torch.Generator().manual_seed(7))).to(DEV)
    y, rstd = _hip.rmsnorm_fwd(x, w, 1e-6)
    p = picks(n, d)
    sy, srstd = _hip.rmsnorm_fwd(x[p], w, 1e-6)
    assert torch.equal(y[p], sy) and torch.equal(rstd[p], srstd)
    dy = randn((n, d), 8)
    dx, dw = _hip.rmsnorm_bwd(x, w, rstd, dy)
    sdx, _ = _hip.rmsnorm_bwd(x[p], w, rstd[p], dy[p])
    assert torch.equal(dx[p], sdx)
    ref = torch.zeros(d, device=DEV, dtype=torch.float64)
    for r0 in range(0, n, 2 ** 21):
        sl = slice(r0, min(n, r0 + 2 ** 21))
        ref += (dy[sl].float() * (x[sl].float() * rstd[sl, None])).double().sum(0)
    assert ((dw.double() - ref).abs().max() / ref.abs().max()).item() < 1e-4


@pytest.mark.parametrize("n,v", [(67200, 32000), (42800, 50257)])
def test_cross_entropy_past_2g(n, v):
    assert n * v > 2 ** 31
    lg = randn((n, v), 11, 2.0)
    g = torch.Generator().manual_seed(12)
    y = torch.randint(0, v, (n,), generator=g)
    y[torch.rand(n, generator=g) < 0.05] = -100
    yd = y.to(DEV)
    n_all = int((y != -100).sum())
    loss, lse, nv, rows = _hip.ce_fwd(lg, yd, -100, "mean")
    dl = _hip.ce_bwd(lg, yd, lse, nv, None, -100)
    assert nv.item() == n_all
    assert loss.item() == pytest.approx((rows.double().sum() / n_all).item(), rel=1e-6)
    p = picks(n, v)
    pc = p.cpu()
    o_loss, og = O.cross_entropy(lg[p].cpu(), y[pc])
    n_s = max(1, int((y[pc] != -100).sum()))
    assert (rows[p].sum().item() / n_s) == pytest.approx(float(o_loss), rel=1e-4)
    assert lowp_close(dl[p], og.float() * (n_s / n_all), 3.0, cancel=1.0 / n_all)
    if v % 8 == 0:          # same vector split in the cut-out rows: same bits
        _, slse, _, srows = _hip.ce_fwd(lg[p], yd[p], -100, "mean")
        assert torch.equal(lse[p], slse) and torch.equal(rows[p], srows)
    # loss and gradient from one read, over the logits
    loss1, dl1, nv1, rows1 = _hip.ce_loss_grad(lg, yd, -100, "mean", inplace=True)
    assert dl1.data_ptr() == lg.data_ptr()
    assert loss1.item() == pytest.approx(loss.item(), rel=1e-6) and nv1.item() == n_all
    assert lowp_close(dl1[p], dl[p], 1.0, cancel=1.0 / n_all)
    ign = yd == -100
    assert not dl1[ign].any()


def test_kl_topk_softmax_past_2g():
    n, v, k, T = 16800, 128256, 64, 2.0
    assert n * v > 2 ** 31
    s = randn((n, v), 21, 3.0)
    t = randn((n, v), 22, 3.0)
    p = picks(n, v)
    loss, rows, lse_s, lse_t = _hip.kl_fwd(s, t, 1.0 / T, "mean")
    assert loss.item() == pytest.approx((rows.double().sum() / n).item(), rel=1e-6)
    orow, og = O.kl_div(s[p].cpu(), t[p].cpu(), "none", T)
    assert torch.allclose(rows[p].cpu(), orow.float(), rtol=1e-4, atol=1e-6)
    ds = _hip.kl_bwd(s, t, lse_s, lse_t, None, False, BF16, 1.0 / T, 1.0 / n)
    assert lowp_close(ds[p], og.float() / n, 3.0, cancel=1.0 / n)
    del ds
    fused = _hip.kl_fwd_topk(s, t, k, 1.0 / T, "mean", torch.int32)
    assert fused is not None
    oi = O.topk(t[p].cpu(), k)[1]
    assert torch.equal(fused[5][p].cpu().long(), oi)
    assert torch.allclose(fused[1], rows, rtol=1e-4, atol=1e-6)
    _, idx = _hip.topk(t, k, torch.int32, want_values=False)
    assert torch.equal(idx[p].cpu().long(), oi)
    del s
    y = _hip.softmax_fwd(t)
    assert torch.equal(y[p], _hip.softmax_fwd(t[p]))
    assert lowp_close(y[p], O.softmax(t[p].cpu()), 2.0)


def test_swiglu_past_2g():
    rows, h = 75008, 28672
    assert rows * h > 2 ** 31 and rows * 2 * h > 2 ** 32
    x = randn((rows, 2 * h), 31)
    dy = randn((rows, h), 32)
    y = _hip.swiglu_split_fwd(x)
    dx = _hip.swiglu_split_bwd(x, dy)
    p = torch.cat((picks(rows, 2 * h), picks(rows, h), torch.tensor([2 ** 32 // (2 * h)], device=DEV))).unique()
    assert torch.equal(y[p], _hip.swiglu_split_fwd(x[p]))
    assert torch.equal(dx[p], _hip.swiglu_split_bwd(x[p], dy[p]))
    ref = torch.nn.functional.silu(x[p][:, :h].float()) * x[p][:, h:].float()
    assert lowp_close(y[p], ref, 2.0)
    gate, up = x[:, :h].contiguous(), x[:, h:].contiguous()
    del x, dx
    assert torch.equal(_hip.swiglu_fwd(gate, up), y)
    dg, du = _hip.swiglu_bwd(gate, up, dy)
    sdg, sdu = _hip.swiglu_bwd(gate[p], up[p], dy[p])
    assert torch.equal(dg[p], sdg) and torch.equal(du[p], sdu)


def test_token_moves_past_2g():
    n, d, k, e = 300000, 4096, 2, 64
    assert n * k * d > 2 ** 31
    x = randn((n, d), 41)
    logits = randn((n, e), 42, 1.0, torch.float32)
    r = _hip.route(logits, k)
    idx, w, counts, slot, order = r[0], r[1], r[2], r[3], r[4]
    xs = _hip.moe_gather(x, order, k)
    flat = torch.arange(n * k, device=DEV)
    assert torch.equal(order.long()[slot.long()], flat)
    tok = torch.div(order.long(), k, rounding_mode="floor")
    for s0 in (0, 2 ** 31 // d - 2, n * k - 4):
        assert torch.equal(xs[s0:s0 + 4], x[tok[s0:s0 + 4]])
    out = _hip.moe_combine(xs, w, slot, n, k)
    p = picks(n, d)
    ref = sum(w[p, j, None] * xs[slot.long().view(n, k)[p, j]].float() for j in range(k))
    assert lowp_close(out[p], ref, 2.0)


def test_qk_norm_rope_past_2g():
    b, t, h, hd = 17, 8192, 128, 64
    d = 2 * hd
    rows = b * t * h
    assert rows * d > 2 ** 31
    x = randn((rows, d), 51).view(b, t, h, d)
    do = randn((rows, d), 52).view(b, t, h, d)
    g = torch.Generator().manual_seed(53)
    w = (1 + 0.1 * torch.randn(d, generator=g)).to(DEV)
    ang = torch.rand(t, hd, generator=g) * 6.28
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    out, rstd = _hip.qk_norm_rope_fwd(x, w, cos, sin, 1e-6)
    dx, dw = _hip.qk_norm_rope_bwd(x, w, cos, sin, rstd, do)

    def expression(xf, dof, tt):          # reference kernels/_fallback.py:38-45 on flat rows
        r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)
        y = xf * r * w
        y1, y2 = y.chunk(2, -1)
        c, s = cos[tt], sin[tt]
        return torch.cat((y1 * c - y2 * s, y1 * s + y2 * c), -1), r

    p = picks(rows, d)
    tt = torch.div(p, h, rounding_mode="floor") % t
    xr = x.view(-1, d)[p].float().requires_grad_(True)
    ref, _ = expression(xr, None, tt)   # w, cos, sin: the device tensors above
    ref.backward(do.view(-1, d)[p].float())
    assert lowp_close(out.view(-1, d)[p], ref.detach(), 3.0, cancel=float(ref.detach().abs().max()))
    assert lowp_close(dx.view(-1, d)[p], xr.grad, 4.0, cancel=4 * float(xr.grad.abs().max()))
    acc = torch.zeros(d, device=DEV, dtype=torch.float64)
    c, s = cos.view(1, t, 1, hd), sin.view(1, t, 1, hd)
    for i in range(b):
        d1, d2 = do[i:i + 1].float().chunk(2, -1)
        gy = torch.cat((d1 * c + d2 * s, d2 * c - d1 * s), -1)      # gradient before the rotation
        acc += (gy * x[i:i + 1].float() * rstd.view(b, t, h, 1)[i:i + 1]).double().sum((0, 1, 2))
    assert ((dw.double() - acc).abs().max() / acc.abs().max()).item() < 1e-4

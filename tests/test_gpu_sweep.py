"""A bounded, seeded slice of the randomised shape sweep: forty shapes per operator drawn from a
fixed seed (widths 1 to 70 000, the three dtypes, fp32 or matching weights, temperatures, ties),
every launch through the library against the CPU oracle, stopping at the first mismatch.

Tolerances: indices, counts and permutations bit-exact; low-precision tensors within a few
units in the last place of the output type per element, plus a few 2^-23 of the magnitude of the
terms that cancel in the expression (the fp32 rounding of those terms, which no output rounding
can undo); fp32 scalars within 1e-4 relative of fp64 math on the same stored values.
"""

import random

import pytest
import torch

from forgeminds_amd.kernels import _hip
from oracle import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32
SHAPES = 40
SEED = 20250


def _width(rng):
    r = rng.random()
    if r < 0.3:
        return rng.randint(1, 70)
    if r < 0.6:
        return rng.randint(71, 3000)
    if r < 0.85:
        return rng.choice([256, 512, 1024, 1025, 2048, 4096, 4104, 8192, 8200, 16384, 32000, 32001, 50257])
    if r < 0.95:
        return rng.randint(3000, 70000)
    return rng.choice([40960, 65536, 66000])


def _within(got, ref, dt, cancel=0.0, ulps=3.0):
    """|got - ref| <= ulps * eps(dt) * |ref| + 1e-6 * max|ref| + 8 * 2^-23 * cancel, per element."""
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    eps = {BF16: 2.0 ** -8, F16: 2.0 ** -11, F32: 2.0 ** -20}[dt]
    scale = ref.abs().max().clamp_min(max(1e-3 * cancel, 1e-30))
    bound = ulps * eps * ref.abs() + 1e-6 * scale + 8 * 2.0 ** -23 * cancel + (2.0 ** -24 if dt == F16 else 0)
    return bool(((got - ref).abs() <= bound).all())


def _cases(salt):
    rng = random.Random(SEED + salt)
    g = torch.Generator().manual_seed(rng.randint(0, 1 << 30))
    for i in range(SHAPES):
        yield i, rng, g


def test_sweep_norms():
    for i, rng, g in _cases(1):
        n, d = rng.randint(1, 40), _width(rng)
        dt = rng.choice([BF16, F16, F32])
        wdt, eps = rng.choice([dt, F32]), rng.choice([1e-5, 1e-6])
        case = (i, n, d, dt, wdt, eps)
        x = (rng.choice([0.0, 0.5, 3.0]) + torch.randn(n, d, generator=g)).to(dt)
        w = (1 + 0.1 * torch.randn(d, generator=g)).to(wdt)
        b = (0.1 * torch.randn(d, generator=g)).to(wdt)
        dy = torch.randn(n, d, generator=g).to(dt)
        xd, wd, bd, dyd = x.to(DEV), w.to(DEV), b.to(DEV), dy.to(DEV)
        y, rstd = _hip.rmsnorm_fwd(xd, wd, eps)
        oy, orstd = O.rms_norm(x, w, eps)
        assert _within(y, oy, dt, ulps=2.0), ("rms_norm", case)
        dx, dw = _hip.rmsnorm_bwd(xd, wd, rstd, dyd)
        odx, odw = O.rms_norm_bwd(x, w, dy, eps)
        nat = (dy.float().abs().max() * w.float().abs().max() * orstd.max()).item() * 4
        assert _within(dx, odx, dt, cancel=nat), ("rms_norm dx", case)
        ref_dw = (dy.double() * x.double() * orstd.double()[:, None]).sum(0)
        assert (dw.double().cpu() - ref_dw).abs().max() <= 2e-2 * ref_dw.abs().max().clamp_min(1e-6), ("rms_norm dw", case)
        if d > 1:
            _, yl, mean, rs = _hip.layernorm_fwd(xd, wd, bd, eps)
            oyl, _, ors = O.layer_norm(x, w, b, eps)
            cancel = 4 * w.float().abs().max().item() + b.float().abs().max().item()
            assert _within(yl, oyl, dt, cancel=cancel, ulps=2.0), ("layer_norm", case)
            dxl, dwl, dbl = _hip.layernorm_bwd(xd, wd, mean, rs, dyd)
            odxl, odwl, odbl = O.layer_norm_bwd(x, w, dy, eps)
            natl = (dy.float().abs().max() * w.float().abs().max() * ors.max()).item() * 4
            assert _within(dxl, odxl, dt, cancel=natl), ("layer_norm dx", case)
            assert ((dbl.float().cpu() - odbl.float()).abs().max()
                    <= 2e-2 * odbl.float().abs().max().clamp_min(1e-6)), ("layer_norm db", case)


def test_sweep_cross_entropy_and_kl():
    for i, rng, g in _cases(2):
        v = _width(rng)
        n = rng.randint(1, 24) if v > 1024 else rng.randint(1, 600)
        dt, T = rng.choice([BF16, F16, F32]), rng.choice([1.0, 2.0, 0.7])
        case = (i, n, v, dt, T)
        lg = (2 * torch.randn(n, v, generator=g)).to(dt)
        lab = torch.randint(0, v, (n,), generator=g)
        lab[torch.rand(n, generator=g) < 0.2] = -100
        o64, _ = O.cross_entropy(lg, lab, acc=torch.float64)
        _, og = O.cross_entropy(lg, lab)
        nv = max(1, int((lab != -100).sum()))
        lgd, labd = lg.to(DEV), lab.to(DEV)
        loss, dl, _, _ = _hip.ce_loss_grad(lgd, labd, -100, "mean")
        assert abs(loss.item() - o64.item()) <= 1e-4 * abs(o64.item()) + 1e-6, ("ce one-pass loss", case)
        assert _within(dl, og, dt, cancel=1.0 / nv), ("ce one-pass grad", case)
        l2, lse, nvt, _ = _hip.ce_fwd(lgd, labd, -100, "mean")
        assert abs(l2.item() - o64.item()) <= 1e-4 * abs(o64.item()) + 1e-6, ("ce fwd loss", case)
        assert _within(_hip.ce_bwd(lgd, labd, lse, nvt, None, -100), og, dt, cancel=1.0 / nv), ("ce bwd", case)
        s = (3 * torch.randn(n, v, generator=g)).to(dt)
        t = (s.float() + 0.5 * torch.randn(n, v, generator=g)).to(dt)
        orow, _ = O.kl_div(s, t, "none", T, acc=torch.float64)
        _, ogk = O.kl_div(s, t, "mean", T)
        sd, td = s.to(DEV), t.to(DEV)
        _, rows, ls, lt = _hip.kl_fwd(sd, td, 1.0 / T, "none")
        assert torch.allclose(rows.cpu().double(), orow, rtol=3e-4, atol=3e-6), ("kl rows", case)
        lm = 1.0 + float(torch.logsumexp(s.double() / T, -1).abs().max())   # |z/T - lse| cancels to log p
        gk = _hip.kl_bwd(sd, td, ls, lt, None, False, dt, 1.0 / T, 1.0 / n)
        assert _within(gk, ogk, dt, cancel=2 * lm / (T * n)), ("kl bwd", case)
        _, g1, r1 = _hip.kl_loss_grad(sd, td, 1.0 / T, "mean", dt)
        assert _within(g1, ogk, dt, cancel=2 * lm / (T * n)), ("kl one-launch grad", case)
        assert torch.allclose(r1.cpu().double(), orow, rtol=3e-4, atol=3e-6), ("kl one-launch rows", case)


def test_sweep_topk_softmax():
    for i, rng, g in _cases(3):
        v = _width(rng)
        n = rng.randint(1, 24) if v > 1024 else rng.randint(1, 600)
        dt = rng.choice([BF16, F16, F32])
        k = rng.randint(1, min(v, 512))
        case = (i, n, v, k, dt)
        s = (3 * torch.randn(n, v, generator=g)).to(dt)
        t = (s.float() + 0.5 * torch.randn(n, v, generator=g)).to(dt)
        if rng.random() < 0.3:      # heavy ties: a handful of distinct values
            t = torch.randint(0, rng.choice([2, 5, 50]), (n, v), generator=g).to(dt)
        _, oi = O.topk(t, k)
        _, ii = _hip.topk(t.to(DEV), k, torch.int32)
        assert torch.equal(ii.cpu().long(), oi), ("topk", case)
        out = _hip.kl_fwd_topk(s.to(DEV), t.to(DEV), k, 1.0, "none", torch.int64)
        if out is not None:
            assert torch.equal(out[5].cpu(), oi), ("kl + topk indices", case)
        sm = _hip.softmax_fwd(s.to(DEV))
        assert _within(sm, O.softmax(s), dt, ulps=2.0), ("softmax", case)
        gy = torch.randn(n, v, generator=g).to(dt)
        smc = sm.cpu()
        sb = _hip.softmax_bwd(sm, gy.to(DEV))
        cancel = float((gy.float().abs().max() + 1) * smc.float().max())
        assert _within(sb, O.softmax_bwd(smc, gy), dt, ulps=2.0, cancel=cancel), ("softmax bwd", case)


def test_sweep_rows_kept_on_the_chip():
    """The one-pass losses and the softmax pair on rows of 7168 to 49152 vectors, the range in which a
    workgroup keeps the row (or the pair of rows) in its registers and LDS between the passes: widths
    around the points where the registers, the LDS share and the streamed remainder begin, a few
    elements either side, so that rows start at every alignment."""
    rng = random.Random(SEED + 5)
    g = torch.Generator().manual_seed(rng.randint(0, 1 << 30))
    for i in range(12):
        dt = rng.choice([BF16, F16, F32])
        epv = 4 if dt == F32 else 8
        v = rng.choice([7168, 8192, 12288, 15360, 16384, 24576, 32768, 49152]) * epv
        v += rng.choice([-17, -8, -1, 0, 1, 7, 9, 16, 33, rng.randint(-3000, 3000)])
        n = rng.randint(1, 3)
        T = rng.choice([1.0, 2.0])
        case = (i, n, v, dt, T)
        s = (3 * torch.randn(n, v, generator=g)).to(dt)
        t = (s.float() + 0.5 * torch.randn(n, v, generator=g)).to(dt)
        lab = torch.randint(0, v, (n,), generator=g)
        if n > 1:
            lab[n - 1] = -100
        sd, td, labd = s.to(DEV), t.to(DEV), lab.to(DEV)
        o64, _ = O.cross_entropy(s, lab, acc=torch.float64)
        _, og = O.cross_entropy(s, lab)
        nv = max(1, int((lab != -100).sum()))
        loss, dl, _, _ = _hip.ce_loss_grad(sd, labd, -100, "mean")
        assert abs(loss.item() - o64.item()) <= 1e-4 * abs(o64.item()) + 1e-6, ("ce one-pass loss", case)
        assert _within(dl, og, dt, cancel=1.0 / nv), ("ce one-pass grad", case)
        own = sd.clone()
        _, dl2, _, _ = _hip.ce_loss_grad(own, labd, -100, "mean", True)
        assert dl2.data_ptr() == own.data_ptr() and torch.equal(dl2, dl), ("ce one-pass in place", case)
        orow, _ = O.kl_div(s, t, "none", T, acc=torch.float64)
        _, ogk = O.kl_div(s, t, "mean", T)
        lm = 1.0 + float(torch.logsumexp(s.double() / T, -1).abs().max())
        _, g1, r1 = _hip.kl_loss_grad(sd, td, 1.0 / T, "mean", dt)
        assert _within(g1, ogk, dt, cancel=2 * lm / (T * n)), ("kl one-launch grad", case)
        assert torch.allclose(r1.cpu().double(), orow, rtol=3e-4, atol=3e-6), ("kl one-launch rows", case)
        own = sd.clone()
        _, g2, _ = _hip.kl_loss_grad(own, td, 1.0 / T, "mean", dt, True)
        assert g2.data_ptr() == own.data_ptr() and torch.equal(g2, g1), ("kl one-launch in place", case)
        sm = _hip.softmax_fwd(sd)
        assert _within(sm, O.softmax(s), dt, ulps=2.0), ("softmax", case)
        gy = torch.randn(n, v, generator=g).to(dt)
        smc = sm.cpu()
        sb = _hip.softmax_bwd(sm, gy.to(DEV))
        cancel = float((gy.float().abs().max() + 1) * smc.float().max())
        assert _within(sb, O.softmax_bwd(smc, gy), dt, ulps=2.0, cancel=cancel), ("softmax bwd", case)


def test_sweep_router():
    for i, rng, g in _cases(4):
        e = rng.choice([2, 3, 4, 8, 16, 32, 64, 100, 128, 256, 512])
        k, n = rng.randint(1, min(e, 8)), rng.randint(1, 3000)
        case = (i, n, e, k)
        lg = torch.round(torch.randn(n, e, generator=g) * 64) / 64       # a coarse grid: ties on most rows
        idx, wts, cnt, slot, order = O.router(lg, k)
        ri, rw, rc, rs, ro = _hip.route(lg.to(DEV), k)
        assert torch.equal(ri.cpu().long(), idx), ("route idx", case)
        assert torch.equal(rc.cpu().long(), cnt), ("route counts", case)
        assert torch.equal(rs.cpu().long(), slot) and torch.equal(ro.cpu().long(), order), ("route permutation", case)
        assert torch.allclose(rw.cpu(), wts, rtol=1e-5, atol=1e-7), ("route weights", case)
        gw = torch.randn(n, k, generator=g)
        ref = O.router_bwd(lg, k, gw, 0.01, 0.001)
        got = _hip.route_bwd(lg.to(DEV), ri, gw.to(DEV), rc, torch.tensor(0.01, device=DEV),
                             torch.tensor(0.001, device=DEV))
        # when k == e the renormalised weights are constants and the weight term cancels to zero:
        # what is left of it is the fp32 rounding of terms of the size of the upstream gradient
        bound = 1e-4 * ref.abs().max() + 8 * 2.0 ** -23 * gw.abs().max().double()
        assert (got.double().cpu() - ref).abs().max() <= bound, ("route bwd", case)

"""Parity of the HIP kernels with the CPU oracle, through the C ABI (the thin ctypes wrappers
of forgeminds_amd.kernels._hip pass raw device pointers to libfmhip.so and nothing else).

Bars: bit-exact for indices, counts and permutations; <= 1e-2 relative for bf16/fp16 tensors
(relative to the largest magnitude of the reference tensor, plus an elementwise bf16-ulp
check); <= 1e-4 relative for fp32 losses against fp32/fp64 math on the same input values.
Inputs are seeded on the CPU generator and moved to the GPU, so both sides see the same bits.
"""

import math

import numpy as np
import pytest
import torch

from forgeminds_amd.kernels import _hip
from oracle import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32


@pytest.fixture(scope="module", autouse=True)
def _need_gpu_and_library():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    assert _hip.loaded(), f"libfmhip.so must be built before GPU tests: {_hip.load_error()}"


def gen(seed):
    return torch.Generator(device="cpu").manual_seed(seed)


def rel_max(got, ref):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    return ((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()


def assert_close_lowp(got, ref, dt, what, ulps=2.0, cancel=0.0, cancel_lowp=0.0):
    """<= 1e-2 of the tensor's scale, and elementwise within a few ulps of the dtype.

    `cancel` is the magnitude of the fp32 terms the result is a difference of (g - xh*c in the
    norm backward, p_s - p_t in the KL gradient): each term carries ~2**-23 relative rounding
    (and ~2**-22 from the hardware exp2), so where the exact answer cancels towards 0 the
    honest absolute tolerance is a few 2**-23 of that magnitude, not of the tiny result."""
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    assert got.shape == ref.shape, what
    cancel = float(cancel)
    scale = ref.abs().max().clamp_min(max(1e-3 * cancel, 1e-30))
    assert ((got - ref).abs().max() / scale).item() <= 1e-2, what
    eps = {BF16: 2.0 ** -8, F16: 2.0 ** -11, F32: 2.0 ** -20}[dt]
    quantum = {BF16: 0.0, F16: 2.0 ** -24, F32: 0.0}[dt]      # fp16 subnormal spacing
    # cancel_lowp: same idea when the *reference* rounds its intermediate terms to the storage dtype
    bound = (ulps * eps * ref.abs() + 1e-6 * scale + 8 * 2.0 ** -23 * cancel + quantum
             + ulps * eps * float(cancel_lowp))
    bad = ((got - ref).abs() > bound)
    assert not bad.any(), f"{what}: {int(bad.sum())} elements beyond {ulps} ulp"


# ------------------------------------------------------------------ RMSNorm
NORM_CASES = [
    # n, d, x dtype, w dtype, eps      (first one: the RMSNorm benchmark shape at 1/8 of the rows)
    (1024, 1024, BF16, F32, 1e-6), (64, 8192, BF16, BF16, 1e-6), (33, 768, F16, F16, 1e-5),
    (17, 100, F32, F32, 1e-6), (5, 7, BF16, F32, 1e-6), (300, 5120, BF16, F32, 1e-6),
    (16, 64, BF16, BF16, 1e-6), (3, 1, F32, F32, 1e-6), (6, 8, F32, F32, 1e-6), (1, 3, F32, F32, 1e-6),
    (9, 16384, BF16, F32, 1e-6), (4, 40000, F16, F32, 1e-6), (130, 3072, F32, F32, 1e-6),
    (7, 12288, BF16, BF16, 1e-5), (2, 24576, BF16, F32, 1e-5),
    # rows past the register path: streamed 16-byte vectors (and, one row wider, scalars)
    (5, 40960, BF16, F32, 1e-6), (3, 65536, F16, F16, 1e-5), (6, 20480, F32, F32, 1e-6),
    (300, 32768, BF16, BF16, 1e-6), (2, 131080, BF16, F32, 1e-6), (3, 40961, BF16, F32, 1e-6),
    # 2049-4096 vectors (fp32: up to 8192): the backward is one persistent kernel with the column
    # sums in registers; more rows than workgroups, uneven chunks
    (700, 18432, BF16, F32, 1e-6), (513, 28672, F32, F32, 1e-6), (257, 32768, F16, F16, 1e-5),
    (300, 16392, BF16, BF16, 1e-6),
    # one tile per workgroup and a tile count the forward can deal by L2 (a multiple of eight
    # backward tiles): workgroups of 256, 512 and 1024 threads, one to many rounds
    (96, 4096, BF16, F32, 1e-6), (16, 16384, BF16, BF16, 1e-6), (48, 8192, F32, F32, 1e-6),
    (2048, 256, BF16, F32, 1e-6), (4096, 512, F16, F16, 1e-5),
]


@pytest.mark.parametrize("n,d,dt,wdt,eps", NORM_CASES)
def test_rmsnorm_fwd_bwd(n, d, dt, wdt, eps):
    g = gen(1001)
    x = torch.randn(n, d, generator=g).to(dt)
    w = (1 + 0.02 * torch.randn(d, generator=g)).to(wdt)
    dy = torch.randn(n, d, generator=g).to(dt)
    oy, orstd = O.rms_norm(x, w, eps)
    odx, odw = O.rms_norm_bwd(x, w, dy, eps)
    xd, wd, dyd = x.to(DEV), w.to(DEV), dy.to(DEV)
    y, rstd = _hip.rmsnorm_fwd(xd, wd, eps)
    dx, dw = _hip.rmsnorm_bwd(xd, wd, rstd, dyd)
    torch.cuda.synchronize()
    assert y.dtype == dt and dx.dtype == dt and dw.dtype == wdt
    assert_close_lowp(y, oy, dt, "y")
    natural = (dy.float().abs().max() * w.float().abs().max() * orstd.max()).item()
    assert_close_lowp(dx, odx, dt, "dx", ulps=3.0, cancel=natural)
    assert rel_max(rstd, orstd) < 1e-5
    # dw: fp32 accumulation on both sides; compare against the fp64 sum too
    _, odw64 = O.rms_norm_bwd(x, w.double(), dy, eps, acc=torch.float64)
    assert rel_max(dw, odw64) <= (1e-2 if wdt != F32 else 1e-4)
    assert rel_max(dw, odw) <= 1e-2
    # frozen weight: no dw, same dx
    dx2, none = _hip.rmsnorm_bwd(xd, wd, rstd, dyd, want_dw=False)
    assert none is None and torch.equal(dx2, dx)


def test_rmsnorm_is_deterministic_and_leaves_inputs_alone():
    g = gen(7)
    x = torch.randn(2048, 1024, generator=g).bfloat16().to(DEV)
    w = torch.randn(1024, generator=g).to(DEV)
    dy = torch.randn(2048, 1024, generator=g).bfloat16().to(DEV)
    keep = x.clone()
    y1, r1 = _hip.rmsnorm_fwd(x, w, 1e-6)
    dx1, dw1 = _hip.rmsnorm_bwd(x, w, r1, dy)
    y2, r2 = _hip.rmsnorm_fwd(x, w, 1e-6)
    dx2, dw2 = _hip.rmsnorm_bwd(x, w, r2, dy)
    assert torch.equal(y1, y2) and torch.equal(dx1, dx2) and torch.equal(dw1, dw2)   # bit for bit
    assert torch.equal(x, keep)


def test_rmsnorm_unaligned_views_take_the_any_width_path():
    g = gen(8)
    base = torch.randn(6 * 512 + 3, generator=g).bfloat16().to(DEV)
    x = base[3:].view(6, 512)                        # data pointer is 6 bytes off a 16-byte line
    w = torch.ones(512, device=DEV)
    y, _ = _hip.rmsnorm_fwd(x, w, 1e-6)
    oy, _ = O.rms_norm(x.cpu(), w.cpu(), 1e-6)
    assert_close_lowp(y, oy, BF16, "y on an unaligned view")


ADD_CASES = [(256, 8192, BF16, F32, 1e-5), (9, 24, F32, F32, 1e-6), (10, 33, BF16, BF16, 1e-6),
             (6, 8, F32, F32, 1e-6), (5, 7, F32, F32, 1e-6), (40, 4096, F16, F16, 1e-5),
             (12, 2048, BF16, F32, 1e-5), (7, 40960, BF16, F32, 1e-5), (5, 20480, F32, F32, 1e-6),
             (260, 24576, F16, F16, 1e-5),
             # tile counts the forward deals by L2
             (96, 4096, BF16, F32, 1e-5), (16, 16384, BF16, BF16, 1e-5), (4096, 512, F16, F16, 1e-5),
             (48, 8192, F32, F32, 1e-6)]


@pytest.mark.parametrize("n,d,dt,wdt,eps", ADD_CASES)
def test_add_rmsnorm_fwd_bwd(n, d, dt, wdt, eps):
    g = gen(1004)
    x = torch.randn(n, d, generator=g).to(dt)
    dl = torch.randn(n, d, generator=g).to(dt)
    w = (1 + 0.02 * torch.randn(d, generator=g)).to(wdt)
    gy = torch.randn(n, d, generator=g).to(dt)
    gxn = torch.randn(n, d, generator=g).to(dt)
    oxn, oy, orstd = O.add_rms_norm(x, dl, w, eps)
    odx, odw = O.add_rms_norm_bwd(oxn, w, gy, gxn, eps)
    odx0, _ = O.add_rms_norm_bwd(oxn, w, gy, None, eps)
    xn, y, rstd = _hip.add_rmsnorm_fwd(x.to(DEV), dl.to(DEV), w.to(DEV), eps)
    dx, dw = _hip.add_rmsnorm_bwd(xn, w.to(DEV), rstd, gy.to(DEV), gxn.to(DEV))
    dx0, dw0 = _hip.add_rmsnorm_bwd(xn, w.to(DEV), rstd, gy.to(DEV), None)
    torch.cuda.synchronize()
    assert torch.equal(xn.cpu(), oxn), "xn must be exactly x + delta in x's dtype"
    assert_close_lowp(y, oy, dt, "y")
    natural = (gy.float().abs().max() * w.float().abs().max() * orstd.max()).item()
    assert_close_lowp(dx, odx, dt, "dx", ulps=3.0, cancel=natural)
    assert_close_lowp(dx0, odx0, dt, "dx without a residual gradient", ulps=3.0, cancel=natural)
    assert rel_max(dw, odw) <= 1e-2 and torch.equal(dw, dw0)
    assert rel_max(rstd, orstd) < 1e-5


# ------------------------------------------------------------------ LayerNorm
LN_CASES = [
    (512, 1024, BF16, F32, 1e-5, True), (64, 8192, BF16, BF16, 1e-5, True), (33, 768, F16, F16, 1e-5, False),
    (17, 100, F32, F32, 1e-6, True), (5, 7, BF16, F32, 1e-5, True), (300, 5120, BF16, F32, 1e-5, False),
    (16, 64, BF16, BF16, 1e-5, True), (3, 1, F32, F32, 1e-5, True), (6, 8, F32, F32, 1e-5, True),
    (9, 16384, BF16, F32, 1e-5, True), (4, 40000, F16, F32, 1e-5, True), (130, 3072, F32, F32, 1e-5, True),
    (7, 12288, BF16, BF16, 1e-5, True), (2, 24576, BF16, F32, 1e-5, False), (40, 4096, BF16, F32, 1e-5, True),
    (5, 40960, BF16, F32, 1e-5, True), (3, 65536, F16, F16, 1e-5, False), (6, 20480, F32, F32, 1e-5, True),
    (270, 32768, BF16, BF16, 1e-5, True), (700, 18432, BF16, F32, 1e-5, True), (300, 24576, F32, F32, 1e-5, True),
    (260, 32768, F32, F32, 1e-5, True),
    # tile counts the forward deals by L2
    (96, 4096, BF16, F32, 1e-5, True), (48, 8192, F32, F32, 1e-5, True), (2048, 256, BF16, F32, 1e-5, False),
]


@pytest.mark.parametrize("n,d,dt,wdt,eps,bias", LN_CASES)
def test_layernorm_fwd_bwd(n, d, dt, wdt, eps, bias):
    g = gen(1031)
    x = (0.5 + torch.randn(n, d, generator=g)).to(dt)           # a mean the kernel has to remove
    w = (1 + 0.02 * torch.randn(d, generator=g)).to(wdt)
    b = (0.1 * torch.randn(d, generator=g)).to(wdt) if bias else None
    dy = torch.randn(n, d, generator=g).to(dt)
    oy, omean, orstd = O.layer_norm(x, w, b, eps)
    odx, odw, odb = O.layer_norm_bwd(x, w, dy, eps)
    xd, wd, dyd = x.to(DEV), w.to(DEV), dy.to(DEV)
    bd = None if b is None else b.to(DEV)
    _, y, mean, rstd = _hip.layernorm_fwd(xd, wd, bd, eps)
    dx, dw, db = _hip.layernorm_bwd(xd, wd, mean, rstd, dyd)
    torch.cuda.synchronize()
    assert y.dtype == dt and dx.dtype == dt and dw.dtype == wdt and db.dtype == wdt
    # y = xh*w + b: where it cancels towards 0 the honest bound is a few fp32 roundings of the terms
    yterms = 4.0 * w.float().abs().max().item() + (b.float().abs().max().item() if bias else 0.0)
    assert_close_lowp(y, oy, dt, "y", cancel=yterms)
    if d > 1:
        assert torch.allclose(mean.cpu(), omean, rtol=1e-5, atol=1e-6) and rel_max(rstd, orstd) < 1e-5
    natural = (dy.float().abs().max() * w.float().abs().max() * orstd.max()).item() * 4.0
    assert_close_lowp(dx, odx, dt, "dx", ulps=3.0, cancel=natural)
    _, odw64, odb64 = O.layer_norm_bwd(x, w.double(), dy, eps, acc=torch.float64)
    tol = 1e-2 if wdt != F32 else 1e-4
    if d > 1:                                                   # d == 1: xh is identically 0
        assert rel_max(dw, odw64) <= tol and rel_max(dw, odw) <= 1e-2
    assert rel_max(db, odb64) <= tol
    # frozen parameters: no dw / db, same dx; bias gradient alone
    dx2, none_w, none_b = _hip.layernorm_bwd(xd, wd, mean, rstd, dyd, None, False, False)
    assert none_w is None and none_b is None and torch.equal(dx2, dx)
    _, dw3, none_b = _hip.layernorm_bwd(xd, wd, mean, rstd, dyd, None, True, False)
    assert none_b is None and torch.equal(dw3, dw)


@pytest.mark.parametrize("n,d,dt,wdt", [(128, 8192, BF16, F32), (9, 24, F32, F32), (10, 33, BF16, BF16),
                                        (40, 4096, F16, F16), (12, 2048, BF16, F32), (6, 40960, BF16, F32),
                                        (4, 24576, F32, F32), (96, 4096, BF16, F32), (1024, 1024, BF16, BF16)])
def test_add_layernorm_fwd_bwd(n, d, dt, wdt):
    g = gen(1034)
    x = torch.randn(n, d, generator=g).to(dt)
    dl = (0.3 + torch.randn(n, d, generator=g)).to(dt)
    w = (1 + 0.02 * torch.randn(d, generator=g)).to(wdt)
    b = (0.1 * torch.randn(d, generator=g)).to(wdt)
    gy = torch.randn(n, d, generator=g).to(dt)
    gxn = torch.randn(n, d, generator=g).to(dt)
    oxn, oy, omean, orstd = O.add_layer_norm(x, dl, w, b, 1e-5)
    odx, odw, odb = O.layer_norm_bwd(oxn, w, gy, 1e-5, gxn=gxn)
    xn, y, mean, rstd = _hip.layernorm_fwd(x.to(DEV), w.to(DEV), b.to(DEV), 1e-5, dl.to(DEV))
    dx, dw, db = _hip.layernorm_bwd(xn, w.to(DEV), mean, rstd, gy.to(DEV), gxn.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(xn.cpu(), oxn), "xn must be exactly x + delta in x's dtype"
    assert_close_lowp(y, oy, dt, "y", cancel=4.0 * w.float().abs().max().item() + b.float().abs().max().item())
    natural = (gy.float().abs().max() * w.float().abs().max() * orstd.max()).item() * 4.0
    assert_close_lowp(dx, odx, dt, "dx", ulps=3.0, cancel=natural)
    assert rel_max(dw, odw) <= 1e-2 and rel_max(db, odb) <= 1e-2


def test_layernorm_determinism_unaligned_and_empty():
    g = gen(1035)
    x = torch.randn(2048, 1024, generator=g).bfloat16().to(DEV)
    w, b = torch.randn(1024, generator=g).to(DEV), torch.randn(1024, generator=g).to(DEV)
    dy = torch.randn(2048, 1024, generator=g).bfloat16().to(DEV)
    outs = []
    for _ in range(2):
        _, y, mean, rstd = _hip.layernorm_fwd(x, w, b, 1e-5)
        outs.append((y,) + _hip.layernorm_bwd(x, w, mean, rstd, dy))
    assert all(torch.equal(a, c) for a, c in zip(*outs))        # bit for bit
    base = torch.randn(6 * 512 + 3, generator=g).bfloat16().to(DEV)
    xv = base[3:].view(6, 512)                                  # 6 bytes off a 16-byte line
    _, y, _, _ = _hip.layernorm_fwd(xv, torch.ones(512, device=DEV), None, 1e-5)
    assert_close_lowp(y, O.layer_norm(xv.cpu(), torch.ones(512), None, 1e-5)[0], BF16, "unaligned", cancel=4.0)
    e = torch.empty(0, 64, device=DEV)
    _, y0, m0, _ = _hip.layernorm_fwd(e, torch.ones(64, device=DEV), None, 1e-5)
    dx0, dw0, db0 = _hip.layernorm_bwd(e, torch.ones(64, device=DEV), m0, m0, e)
    assert y0.shape == (0, 64) and not dw0.any() and not db0.any()


# ------------------------------------------------------------------ cross entropy
CE_CASES = [(512, 32000, BF16), (7, 50257, BF16), (5, 1000, F32), (4, 7, F16), (9, 16, F32),
            (3, 128256, BF16), (6, 32001, F32), (33, 4096, F16), (2, 1, F32), (64, 50257, F32),
            (1000, 100, BF16), (300, 257, F16), (50, 1024, F32), (70, 33, BF16), (129, 600, BF16),
            (300, 512, F32), (40, 513, F32),
            # rows that are whole aligned 16-byte vectors: every lane-group shape of the vector form
            (257, 24, BF16), (130, 64, BF16), (99, 128, F16), (65, 256, BF16), (300, 512, BF16),
            (50, 1024, BF16), (18, 1000, BF16), (37, 2048, BF16), (21, 4096, BF16), (37, 2048, F16),
            (21, 1536, F16), (33, 96, F32), (19, 2048, F32), (1025, 8, F32), (23, 2040, BF16)]


@pytest.mark.parametrize("n,v,dt", CE_CASES)
def test_ce_fwd_bwd(n, v, dt):
    g = gen(1002)
    lg = (2 * torch.randn(n, v, generator=g)).to(dt)
    y = torch.randint(0, v, (n,), generator=g)
    y[torch.rand(n, generator=g) < 0.2] = -100
    o32, ograd = O.cross_entropy(lg, y)
    o64, _ = O.cross_entropy(lg, y, acc=torch.float64)
    lgd, yd = lg.to(DEV), y.to(DEV)
    loss, lse, nv, rows = _hip.ce_fwd(lgd, yd, -100, "mean")
    go = torch.tensor(0.5, device=DEV)
    dl = _hip.ce_bwd(lgd, yd, lse, nv, go, -100)
    total, _, _, _ = _hip.ce_fwd(lgd, yd, -100, "sum")
    torch.cuda.synchronize()
    n_valid = max(1, int((y != -100).sum()))
    assert nv.item() == n_valid
    assert loss.item() == pytest.approx(o64.item(), rel=1e-4, abs=1e-7)
    assert loss.item() == pytest.approx(o32.item(), rel=1e-4, abs=1e-7)
    assert total.item() == pytest.approx(o64.item() * n_valid, rel=1e-4, abs=1e-6)
    assert_close_lowp(dl, ograd.float() * 0.5, dt, "dlogits", ulps=3.0, cancel=0.5 / n_valid)
    ign = (y == -100)
    assert not dl.cpu()[ign].any(), "ignored rows get exact zeros"
    if (~ign).any():                      # softmax - onehot sums to zero on every valid row
        assert dl.float().cpu()[~ign].sum(-1).abs().max() < (2e-2 if dt != F32 else 1e-5) * 0.5 / n_valid * 8
    lse_ref = torch.logsumexp(lg.double(), -1)
    assert torch.allclose(lse.cpu().double(), lse_ref, rtol=1e-5, atol=1e-5)


def test_ce_forward_with_and_without_a_backward_to_follow():
    """With an lse buffer the forward reads the last rows (what the memory-side cache holds) with cached
    loads for the backward to find, without one it streams every row: two kernels over two row ranges
    or one, the same numbers either way, also where the split falls inside the tensor."""
    g = gen(1019)
    for n, v, dt in ((9000, 32000, BF16), (300, 1000, F32), (5, 70001, F16)):
        lg = (2 * torch.randn(n, v, generator=g)).to(dt).to(DEV)
        y = torch.randint(0, v, (n,), generator=g)
        y[::7] = -100
        y = y.to(DEV)
        loss, lse, nv, rows = _hip.ce_fwd(lg, y, -100, "mean")
        loss2, lse2, nv2, rows2 = _hip.ce_fwd(lg, y, -100, "mean", for_backward=False)
        assert lse2 is None and torch.equal(rows, rows2) and loss.item() == loss2.item() and nv.item() == nv2.item()
        ref = torch.nn.functional.cross_entropy(lg.float(), y, ignore_index=-100)
        assert loss.item() == pytest.approx(ref.item(), rel=1e-4)
        ok = y != -100
        assert torch.allclose(lse[ok], torch.logsumexp(lg.float(), -1)[ok], rtol=1e-5, atol=1e-5)


CE1_CASES = CE_CASES + [(5, 140000, BF16), (3, 70000, F32), (4, 600, BF16), (3, 9000, F16),
                        # rows kept on the chip (registers + LDS of one workgroup per compute unit): aligned and
                        # odd widths, the widest that fits, and one past it (two sweeps)
                        (6, 128256, BF16), (5, 151937, F16), (4, 98000, F32), (4, 196560, BF16), (3, 196608, BF16),
                        (3, 262147, BF16), (2, 128256, F32), (2, 393300, F16)]


@pytest.mark.parametrize("n,v,dt", CE1_CASES)
@pytest.mark.parametrize("reduction", ["mean", "sum"])
def test_ce_loss_and_gradient_in_one_pass(n, v, dt, reduction):
    g = gen(1012)
    lg = (2 * torch.randn(n, v, generator=g)).to(dt)
    y = torch.randint(0, v, (n,), generator=g)
    y[torch.rand(n, generator=g) < 0.2] = -100
    o64, _ = O.cross_entropy(lg, y, acc=torch.float64)
    _, ograd = O.cross_entropy(lg.float(), y)        # unrounded: the sum form rescales it
    n_valid = max(1, int((y != -100).sum()))
    if reduction == "sum":
        o64, ograd = o64 * n_valid, ograd * n_valid
    lgd, yd = lg.to(DEV), y.to(DEV)
    keep = lgd.clone()
    loss, dl, nv, rows = _hip.ce_loss_grad(lgd, yd, -100, reduction)
    torch.cuda.synchronize()
    assert torch.equal(lgd, keep), "the input is left alone unless in-place is asked for"
    assert nv.item() == n_valid
    assert loss.item() == pytest.approx(o64.item(), rel=1e-4, abs=1e-6)
    cancel = 1.0 / n_valid if reduction == "mean" else 1.0
    assert_close_lowp(dl, ograd.float(), dt, "dlogits", ulps=3.0, cancel=cancel)
    ign = (y == -100)
    assert not dl.cpu()[ign].any() and not rows.cpu()[ign].any()
    # the same call writing over the logits gives the same bits
    loss2, dl2, _, _ = _hip.ce_loss_grad(lgd, yd, -100, reduction, inplace=True)
    torch.cuda.synchronize()
    assert dl2.data_ptr() == lgd.data_ptr()             # rows of any width, aligned or not
    assert torch.equal(dl2, dl) and loss2.item() == loss.item()
    # and it agrees with the two-pass kernels to the last bit of the loss and a rounding of the grad
    loss3, lse, nv3, _ = _hip.ce_fwd(keep, yd, -100, reduction)
    dl3 = _hip.ce_bwd(keep, yd, lse, nv3 if reduction == "mean" else None, None, -100)
    assert loss3.item() == pytest.approx(loss.item(), rel=1e-6, abs=1e-7)
    assert_close_lowp(dl, dl3.float().cpu(), dt, "vs two-pass", ulps=2.0, cancel=cancel)


@pytest.mark.parametrize("n,v,dt", [(600, 66000, BF16), (300, 70001, F16), (530, 33032, F32)])
def test_ce_one_pass_many_wide_rows_with_ignored_ones(n, v, dt):
    """More rows than the chip has compute units, at widths kept on the chip (one workgroup per
    compute unit at a time), with ignored rows first, last, 256 apart and two in a row. Checked
    against the two-pass kernels (which the other tests pin to the oracle) and, on a sample of
    rows, against the oracle itself."""
    g = gen(1051)
    lg = (2 * torch.randn(n, v, generator=g)).to(dt)
    y = torch.randint(0, v, (n,), generator=g)
    y[torch.rand(n, generator=g) < 0.15] = -100
    y[3] = -100
    y[5::256] = -100                # every row a compute unit would get in turn
    y[7 + 256] = -100
    y[9] = -100
    y[9 + 256] = -100
    y[n - 1] = -100                 # the last row of all
    y[10] = v - 1                   # labels at both ends of the row
    y[11] = 0
    lgd, yd = lg.to(DEV), y.to(DEV)
    keep = lgd.clone()
    for reduction in ("mean", "sum"):
        loss, dl, nv, rows = _hip.ce_loss_grad(lgd, yd, -100, reduction)
        torch.cuda.synchronize()
        assert torch.equal(lgd, keep)
        n_valid = int((y != -100).sum())
        assert nv.item() == n_valid
        cancel = 1.0 / n_valid if reduction == "mean" else 1.0
        loss3, lse, nv3, _ = _hip.ce_fwd(keep, yd, -100, reduction)
        dl3 = _hip.ce_bwd(keep, yd, lse, nv3 if reduction == "mean" else None, None, -100)
        assert loss3.item() == pytest.approx(loss.item(), rel=1e-6, abs=1e-7)
        assert_close_lowp(dl, dl3.float().cpu(), dt, "vs two-pass", ulps=2.0, cancel=cancel)
        ign = (y == -100)
        assert not dl.cpu()[ign].any() and not rows.cpu()[ign].any()
        sample = torch.tensor([0, 3, 5, 9, 10, 11, 255, 256, 257, 261, 263, 265, 299, n - 2, n - 1])
        _, og = O.cross_entropy(lg[sample].float(), y[sample])
        ov = max(1, int((y[sample] != -100).sum()))
        want = og * ov * (1.0 / n_valid if reduction == "mean" else 1.0)
        assert_close_lowp(dl[sample.to(DEV)], want.float(), dt, "sampled rows vs oracle", ulps=3.0, cancel=cancel)
        loss2, dl2, _, _ = _hip.ce_loss_grad(lgd.clone(), yd, -100, reduction, inplace=True)
        assert torch.equal(dl2, dl) and loss2.item() == loss.item()


def test_ce_kl_vector_rows_agree_with_the_scalar_form():
    """Narrow rows of whole aligned vectors take 16-byte loads; the same rows one element per
    load (the form for other widths and alignments, reached here by buffers that start one element
    off a 16-byte line) must give the same answers, special values included."""
    g = gen(1040)
    for dt, v in ((BF16, 512), (F16, 1024), (F32, 256), (BF16, 2048)):
        n = 37
        lg = (2 * torch.randn(n, v, generator=g)).to(dt)
        lg[0, 5] = float("nan")
        lg[1] = float("-inf")
        lg[1, 7] = 1.0
        lg[2, 3] = float("inf")
        y = torch.randint(0, v, (n,), generator=g)
        y[3] = -100
        y[4] = v + 5                       # out of range: the loss of that row is NaN, as in torch
        y[1] = 7
        t = (lg.float() + 0.5 * torch.randn(n, v, generator=g)).to(dt)
        yd = y.to(DEV)
        res = []
        for shift in (0, 1):
            def place(x):       # the tensor, or a copy of it that starts `shift` elements into an allocation
                buf = torch.empty(x.numel() + shift, device=DEV, dtype=x.dtype)
                buf[shift:] = x.reshape(-1).to(DEV)
                return buf[shift:].view(x.shape)
            lgd, td = place(lg), place(t)
            loss, lse, nv, rows = _hip.ce_fwd(lgd, yd, -100, "sum")
            dl = _hip.ce_bwd(lgd, yd, lse, nv, None, -100)
            l1, d1, _, r1 = _hip.ce_loss_grad(lgd, yd, -100, "mean")
            kl, krows, ls, lt = _hip.kl_fwd(lgd, td, 0.5, "none")
            kg = _hip.kl_bwd(lgd, td, ls, lt, None, False, dt, 0.5, 1.0)
            torch.cuda.synchronize()
            res.append([x.float().cpu() for x in (lse, rows, dl, d1, r1, krows, ls, lt, kg)])
        names = ("lse", "rows", "dl", "d1", "r1", "krows", "ls", "lt", "kg")
        for name, a, b in zip(names, *res):
            assert torch.equal(a.isnan(), b.isnan()), (dt, v, name)
            assert torch.allclose(a.nan_to_num(0.0, 1e30, -1e30), b.nan_to_num(0.0, 1e30, -1e30),
                                  rtol=2e-2 if dt != F32 else 1e-5, atol=1e-6), (dt, v, name)
        assert res[0][1][4].isnan() and res[0][1][3] == 0 and not res[0][2][3].any()
    # 16 bytes further into a buffer the rows are still aligned; 2 bytes further they are not
    base = (2 * torch.randn(9 * 512 + 9, generator=g)).to(BF16).to(DEV)
    yb = torch.randint(0, 512, (9,), generator=g)
    for off in (8, 1):
        view = base[off:off + 9 * 512].view(9, 512)
        loss, dl, _, _ = _hip.ce_loss_grad(view, yb.to(DEV), -100, "mean")
        ref, rgrad = O.cross_entropy(view.cpu(), yb)
        assert loss.item() == pytest.approx(ref.item(), rel=1e-4)
        assert_close_lowp(dl, rgrad, BF16, f"offset {off}", ulps=3.0, cancel=1.0 / 9)


def test_ce_loss_grad_unaligned_and_scale_inplace():
    g = gen(1013)
    base = (2 * torch.randn(5 * 3001 + 1, generator=g)).bfloat16().to(DEV)
    lg = base[1:].view(5, 3001)                                      # base pointer off by 2 bytes
    y = torch.randint(0, 3001, (5,), generator=g).to(DEV)
    loss, dl, nv, _ = _hip.ce_loss_grad(lg, y, -100, "mean")
    o64, _ = O.cross_entropy(lg.cpu(), y.cpu(), acc=torch.float64)
    _, ograd = O.cross_entropy(lg.cpu(), y.cpu())
    assert loss.item() == pytest.approx(o64.item(), rel=1e-4)
    assert_close_lowp(dl, ograd.float(), BF16, "dlogits", ulps=3.0, cancel=0.2)
    # scale_inplace: a factor of 1 leaves every bit alone, any other factor multiplies once
    for dt, cnt in ((BF16, 100003), (F32, 4099), (F16, 7)):
        x = torch.randn(cnt, generator=g).to(dt).to(DEV)
        before = x.clone()
        _hip.scale_inplace(x, torch.tensor(1.0, device=DEV))
        assert torch.equal(x, before)
        _hip.scale_inplace(x, torch.tensor(0.375, device=DEV))
        assert torch.equal(x, (before.float() * 0.375).to(dt))
    x = torch.randn(33, device=DEV)[1:]                              # unaligned start
    before = x.clone()
    _hip.scale_inplace(x, torch.tensor(-2.0, device=DEV))
    assert torch.equal(x, before * -2.0)


def test_ce_known_answers_on_gpu():
    # all ignored -> 0.0 and a zero gradient; reference tests/test_edge_cases.py:21-28
    lg = torch.randn(6, 16, device=DEV)
    y = torch.full((6,), -100, device=DEV)
    loss, lse, nv, _ = _hip.ce_fwd(lg, y, -100, "mean")
    dl = _hip.ce_bwd(lg, y, lse, nv, None, -100)
    assert loss.item() == 0.0 and nv.item() == 1.0 and not dl.any()
    # uniform logits -> log(V)
    loss, *_ = _hip.ce_fwd(torch.zeros(3, 10, device=DEV), torch.tensor([0, 5, 9], device=DEV), -100, "mean")
    assert loss.item() == pytest.approx(math.log(10), rel=1e-6)
    # a different ignore_index
    y2 = torch.tensor([1, 2, 3, 2, 2, 0], device=DEV)
    loss2, *_ = _hip.ce_fwd(lg, y2, 2, "mean")
    ref, _ = O.cross_entropy(lg.cpu(), y2.cpu(), ignore_index=2)
    assert loss2.item() == pytest.approx(ref.item(), rel=1e-5)


# ------------------------------------------------------------------ KL
KL_CASES = [(64, 128256, BF16, 2.0), (6, 5000, F32, 1.0), (3, 1, F32, 1.0), (5, 50257, BF16, 1.0),
            (4, 7, F32, 1.0), (4, 64, F32, 1.0), (4, 1000, F32, 1.0), (9, 32000, F16, 1.5),
            (2, 5000, F32, 4.0),
            # narrow rows: lane groups, several rows per workgroup
            (1000, 100, BF16, 2.0), (300, 257, F16, 1.0), (50, 1024, F32, 2.0), (70, 33, BF16, 1.0),
            (129, 600, BF16, 1.5), (1030, 8, F32, 1.0), (77, 16, BF16, 3.0),
            # whole aligned vectors: every lane-group shape of the vector form
            (257, 24, BF16, 1.0), (130, 64, BF16, 2.0), (99, 128, F16, 1.0), (65, 256, BF16, 1.0),
            (300, 512, BF16, 2.0), (50, 1024, BF16, 1.0), (37, 2048, BF16, 1.5), (21, 2040, F16, 1.0),
            (33, 96, F32, 1.0), (19, 1024, F32, 2.0), (40, 520, F32, 1.0)]


@pytest.mark.parametrize("n,v,dt,T", KL_CASES)
def test_kl_fwd_bwd(n, v, dt, T):
    g = gen(1005)
    s = (3 * torch.randn(n, v, generator=g)).to(dt)
    t = (s.float() + 0.5 * torch.randn(n, v, generator=g)).to(dt)
    o64, _ = O.kl_div(s, t, "mean", T, acc=torch.float64)
    orow, _ = O.kl_div(s, t, "none", T, acc=torch.float64)
    _, ograd = O.kl_div(s, t, "mean", T)
    sd, td = s.to(DEV), t.to(DEV)
    loss, rows, ls, lt = _hip.kl_fwd(sd, td, 1.0 / T, "mean")
    total, *_ = _hip.kl_fwd(sd, td, 1.0 / T, "sum")
    gs = _hip.kl_bwd(sd, td, ls, lt, None, False, dt, 1.0 / T, 1.0 / n)
    torch.cuda.synchronize()
    assert loss.item() == pytest.approx(o64.item(), rel=1e-4, abs=2e-7)
    assert total.item() == pytest.approx(o64.item() * n, rel=1e-4, abs=2e-6)
    assert torch.allclose(rows.cpu().double(), orow, rtol=2e-4, atol=2e-6)
    # p = exp(z / T - lse): each of the two terms carries its own fp32 rounding, so the honest
    # absolute error of a probability near 1 (narrow rows) grows with |lse|
    lse_mag = 1.0 + float(torch.logsumexp(s.double() / T, -1).abs().max())
    assert_close_lowp(gs, ograd, dt, "dstudent", ulps=3.0, cancel=lse_mag / (T * n))
    assert torch.allclose(ls.cpu().double(), torch.logsumexp(s.double() / T, -1), rtol=1e-5, atol=1e-5)
    assert torch.allclose(lt.cpu().double(), torch.logsumexp(t.double() / T, -1), rtol=1e-5, atol=1e-5)
    # per-row upstream gradients and an fp32 gradient buffer
    up = torch.rand(n, generator=g)
    gs32 = _hip.kl_bwd(sd, td, ls, lt, up.to(DEV), True, F32, 1.0 / T, 1.0)
    _, g_none = O.kl_div(s.float(), t.float(), "none", T)
    want = g_none * up[:, None]
    tol = (1e-2 if dt != F32 else 1e-4) * want.abs().max().item() + 1e-6 / T
    assert (gs32.cpu() - want).abs().max().item() <= tol


KL1_CASES = [(64, 32000, BF16, 2.0, BF16), (6, 5000, F32, 1.0, F32), (3, 1, F32, 1.0, F32),
             (5, 32768, BF16, 1.0, F32), (4, 7, F32, 1.0, F32), (9, 32000, F16, 1.5, F16),
             (7, 4099, BF16, 1.0, BF16), (3, 50257, BF16, 1.0, BF16), (4, 16000, F32, 4.0, F32),
             (5, 600, F16, 1.0, F32), (6, 2048, BF16, 2.0, BF16),
             (1000, 100, BF16, 2.0, BF16), (300, 257, F16, 1.0, F32), (50, 1024, F32, 2.0, F32),
             (70, 33, BF16, 1.0, F32), (1030, 8, BF16, 1.0, BF16),
             (257, 24, BF16, 1.0, F32), (130, 64, BF16, 2.0, BF16), (99, 128, F16, 1.0, F16),
             (65, 256, BF16, 1.0, BF16), (300, 512, BF16, 2.0, F32), (50, 1024, F16, 1.0, F32),
             (37, 2048, BF16, 1.5, F32), (33, 96, F32, 1.0, F32), (19, 1024, F32, 2.0, F32),
             # rows past the register path: two sweeps in one launch
             (4, 70000, BF16, 2.0, BF16), (3, 40000, F32, 1.0, F32), (3, 128256, BF16, 2.0, F32),
             (5, 65537, F16, 1.0, F16),
             # rows that stay on the chip between the passes (registers + LDS of one workgroup per
             # compute unit): aligned and odd widths, in place, and rows past what the chip holds
             (3, 128256, BF16, 1.0, BF16), (2, 151937, F16, 2.0, F16), (2, 140000, F32, 1.0, F32),
             (2, 196608, BF16, 1.0, BF16), (3, 28673, F32, 2.0, F32),
             # the same with more rows than the chip holds workgroups (one to three per compute unit
             # by row width): a workgroup then walks two or three rows and loads the next one from
             # inside this one's gradient pass (even and odd widths, rows of fewer slots than a thread
             # holds, the last row of a workgroup)
             (600, 20000, BF16, 2.0, BF16), (300, 17001, F16, 2.0, F32), (530, 9001, F32, 1.0, F32),
             (257, 40008, BF16, 1.0, BF16), (520, 16392, BF16, 1.0, BF16),
             (1700, 16400, BF16, 2.0, BF16), (1100, 36880, BF16, 2.0, BF16), (300, 70000, BF16, 2.0, BF16)]


@pytest.mark.parametrize("n,v,dt,T,gdt", KL1_CASES)
@pytest.mark.parametrize("reduction", ["mean", "sum"])
def test_kl_loss_and_gradient_in_one_pass(n, v, dt, T, gdt, reduction):
    g = gen(1025)
    s = (3 * torch.randn(n, v, generator=g)).to(dt)
    t = (s.float() + 0.5 * torch.randn(n, v, generator=g)).to(dt)
    o64, _ = O.kl_div(s, t, reduction, T, acc=torch.float64)
    orow, _ = O.kl_div(s, t, "none", T, acc=torch.float64)
    _, ograd = O.kl_div(s.float() if gdt == F32 else s, t.float() if gdt == F32 else t, reduction, T)
    sd, td = s.to(DEV), t.to(DEV)
    keep = sd.clone()
    loss, grad, rows = _hip.kl_loss_grad(sd, td, 1.0 / T, reduction, gdt)
    torch.cuda.synchronize()
    assert torch.equal(sd, keep) and grad.dtype == gdt
    assert loss.item() == pytest.approx(o64.item(), rel=1e-4, abs=2e-6 if reduction == "sum" else 2e-7)
    assert torch.allclose(rows.cpu().double(), orow, rtol=2e-4, atol=2e-6)
    cancel = 1.0 / (T * n) if reduction == "mean" else 1.0 / T
    assert_close_lowp(grad, ograd.float(), gdt, "dstudent", ulps=3.0, cancel=cancel)
    # against the two-pass kernels
    loss2, rows2, ls, lt = _hip.kl_fwd(sd, td, 1.0 / T, reduction)
    g2 = _hip.kl_bwd(sd, td, ls, lt, None, False, gdt, 1.0 / T, 1.0 / n if reduction == "mean" else 1.0)
    assert loss2.item() == pytest.approx(loss.item(), rel=1e-4, abs=5e-7)
    assert_close_lowp(grad, g2.float().cpu(), gdt, "vs two-pass", ulps=2.0, cancel=cancel)
    # written over the student when the dtypes agree (rows of any width)
    loss3, g3, _ = _hip.kl_loss_grad(sd, td, 1.0 / T, reduction, gdt, inplace=True)
    torch.cuda.synchronize()
    assert (g3.data_ptr() == sd.data_ptr()) == (gdt == dt)
    assert torch.equal(g3, grad) and loss3.item() == loss.item()


def test_kl_known_answers_on_gpu():
    s = torch.randn(5, 777, device=DEV)
    loss, rows, ls, lt = _hip.kl_fwd(s, s.clone(), 1.0, "mean")
    gs = _hip.kl_bwd(s, s.clone(), ls, lt, None, False, F32, 1.0, 0.2)
    assert abs(loss.item()) < 1e-6 and gs.abs().max().item() < 1e-7   # identical -> 0
    t = torch.randn(5, 777, device=DEV)
    _, rows, _, _ = _hip.kl_fwd(s, t, 1.0, "none")
    assert (rows > 0).all()                                           # Gibbs
    keep = s.clone()
    assert torch.equal(s, keep)


# ------------------------------------------------------------------ KL + teacher top-k, one pass
KLTOPK_CASES = [(16, 128256, 64, BF16, 2.0), (6, 32000, 64, BF16, 1.0), (4, 50257, 33, BF16, 2.0),
                (3, 4096, 8, F32, 1.0), (2, 80000, 64, F32, 2.0), (5, 20000, 100, F16, 1.0),
                (3, 700, 5, BF16, 1.0), (2, 1025, 512, BF16, 2.0), (4, 1, 1, F32, 1.0),
                (2, 9000, 512, F32, 1.0),
                # rows whose teacher prefixes take more than 64 KB of LDS (one workgroup per compute unit)
                (2, 262144, 64, BF16, 2.0), (2, 170001, 40, F16, 1.0), (1, 131072, 64, F32, 1.0)]


@pytest.mark.parametrize("n,v,k,dt,T", KLTOPK_CASES)
def test_kl_fwd_topk_matches_the_two_kernels(n, v, k, dt, T):
    g = gen(1015)
    s = (3 * torch.randn(n, v, generator=g)).to(dt)
    t = (s.float() + 0.5 * torch.randn(n, v, generator=g)).to(dt)
    o64, _ = O.kl_div(s, t, "mean", T, acc=torch.float64)
    orow, _ = O.kl_div(s, t, "none", T, acc=torch.float64)
    ov, oi = O.topk(t, k)
    sd, td = s.to(DEV), t.to(DEV)
    for bits in (torch.int32, torch.int64):
        out = _hip.kl_fwd_topk(sd, td, k, 1.0 / T, "mean", bits, want_values=True, want_probs=True)
        assert out is not None
        loss, rows, ls, lt, vals, idx, probs = out
        loss2, rows2, ls2, lt2 = _hip.kl_fwd(sd, td, 1.0 / T, "mean")
        torch.cuda.synchronize()
        assert idx.dtype == bits and torch.equal(idx.cpu().long(), oi)      # bit-exact selection
        assert torch.equal(vals.cpu(), ov)
        assert loss.item() == pytest.approx(o64.item(), rel=1e-4, abs=2e-7)
        assert torch.allclose(rows.cpu().double(), orow, rtol=2e-4, atol=2e-6)
        assert torch.allclose(rows, rows2, rtol=2e-4, atol=2e-6)
        assert torch.allclose(ls, ls2, rtol=1e-6, atol=2e-6) and torch.allclose(lt, lt2, rtol=1e-6, atol=2e-6)
        want = torch.gather(torch.softmax(t.double() / T, -1), -1, oi)
        assert torch.allclose(probs.cpu().double(), want, rtol=1e-4, atol=1e-9)
    # the same launch also writing the student's gradient: every other output keeps its bits
    keep = sd.clone()
    full = _hip.kl_fwd_topk(sd, td, k, 1.0 / T, "mean", torch.int64, want_values=True, want_probs=True,
                            want_grad=True)
    torch.cuda.synchronize()
    assert torch.equal(sd, keep)
    for a, b in zip(full[:7], out):
        assert torch.equal(a, b)
    _, ograd = O.kl_div(s, t, "mean", T)
    lse_mag = 1.0 + float(torch.logsumexp(s.double() / T, -1).abs().max())
    assert_close_lowp(full[7], ograd, dt, "dstudent", ulps=3.0, cancel=lse_mag / (T * n))
    summed = _hip.kl_fwd_topk(sd, td, k, 1.0 / T, "sum", torch.int32, want_grad=True)
    _, ograd_sum = O.kl_div(s, t, "sum", T)
    assert_close_lowp(summed[7], ograd_sum, dt, "dstudent (sum)", ulps=3.0, cancel=lse_mag / T)


def test_kl_fwd_topk_ties_unaligned_and_unsupported():
    g = gen(1016)
    # three distinct teacher values: the exact path runs inside the fused kernel
    t = torch.randint(0, 3, (4, 40000), generator=g).to(BF16)
    s = torch.randn(4, 40000, generator=g).to(BF16)
    out = _hip.kl_fwd_topk(s.to(DEV), t.to(DEV), 300, 1.0, "none", torch.int32)
    assert torch.equal(out[5].cpu().long(), O.topk(t, 300)[1])
    orow, _ = O.kl_div(s, t, "none", 1.0, acc=torch.float64)
    assert torch.allclose(out[1].cpu().double(), orow, rtol=2e-4, atol=2e-6)
    # rows that start off a 16-byte boundary
    base_s = (3 * torch.randn(3 * 9001 + 1, generator=g)).bfloat16().to(DEV)
    base_t = (3 * torch.randn(3 * 9001 + 1, generator=g)).bfloat16().to(DEV)
    s2, t2 = base_s[1:].view(3, 9001), base_t[1:].view(3, 9001)
    out = _hip.kl_fwd_topk(s2, t2, 20, 0.5, "none", torch.int64)
    assert torch.equal(out[5].cpu(), O.topk(t2.cpu(), 20)[1])
    orow, _ = O.kl_div(s2.cpu(), t2.cpu(), "none", 2.0, acc=torch.float64)
    assert torch.allclose(out[1].cpu().double(), orow, rtol=2e-4, atol=2e-6)
    # NaN in the teacher: selected first, KL of that row is NaN, other rows untouched
    t3 = torch.randn(2, 5000, generator=g)
    t3[0, 77] = float("nan")
    s3 = torch.randn(2, 5000, generator=g)
    out = _hip.kl_fwd_topk(s3.to(DEV), t3.to(DEV), 4, 1.0, "none", torch.int64)
    assert torch.equal(out[5].cpu(), O.topk(t3, 4)[1]) and out[5][0, 0].item() == 77
    assert math.isnan(out[1][0].item()) and math.isfinite(out[1][1].item())
    # rows wider than the fused kernel's LDS budget: the binding says so
    wide = torch.zeros(1, 66561 * 8, dtype=BF16, device=DEV)
    assert _hip.kl_fwd_topk(wide, wide, 4, 1.0, "none", torch.int64) is None


# ------------------------------------------------------------------ top-k
TOPK_CASES = [(32, 128256, 64, BF16), (8, 4096, 64, F32), (4, 64, 8, F32), (3, 5000, 512, BF16),
              (4, 20000, 100, F16), (2, 300000, 17, BF16), (3, 9000, 5, F32), (2, 100, 99, F32),
              (1, 512, 512, F32), (5, 1, 1, F32), (2, 600, 4, F32), (4, 5000, 512, F32),
              (2, 1025, 3, BF16), (3, 70000, 512, F32), (6, 50257, 64, BF16), (2, 140000, 64, F32),
              (1000, 64, 8, F32), (333, 128, 2, BF16), (77, 200, 200, F16), (50, 1024, 512, BF16),
              (41, 1000, 64, F32), (9, 7, 7, BF16), (130, 513, 100, F16), (5, 1024, 1, F32),
              (6, 4096, 256, BF16), (5, 8192, 512, F32), (4, 8192, 256, F16), (3, 16384, 512, F32),
              # rows whose vector prefixes need more than 64 KB of LDS, and one past even that
              (3, 262144, 64, BF16), (2, 500000, 300, BF16), (2, 262144, 64, F32), (2, 262147, 100, F16),
              (1, 600000, 8, BF16)]


@pytest.mark.parametrize("n,v,k,dt", TOPK_CASES)
def test_topk_is_bit_exact(n, v, k, dt):
    g = gen(1006)
    x = (3 * torch.randn(n, v, generator=g)).to(dt)
    ov, oi = O.topk(x, k)
    vals, idx = _hip.topk(x.to(DEV), k, torch.int32)
    vals64, idx64 = _hip.topk(x.to(DEV), k, torch.int64)
    torch.cuda.synchronize()
    assert idx.dtype == torch.int32 and idx64.dtype == torch.int64
    assert torch.equal(idx.cpu().long(), oi) and torch.equal(idx64.cpu(), oi)
    assert torch.equal(vals.cpu(), ov) and torch.equal(vals64.cpu(), ov)


def test_topk_ties_nans_zeros_and_degenerate_rows():
    def run(t, k):
        _, i = _hip.topk(t.to(DEV), k, torch.int64)
        return i.cpu()
    # reference tests/test_topk.py:68-85
    assert run(torch.tensor([[1.0, 3.0, 3.0, 2.0, 3.0]]), 3).tolist() == [[1, 2, 4]]
    assert run(torch.tensor([[float("nan"), 1.0, 2.0, float("nan"), 0.0]]), 3).tolist() == [[0, 3, 2]]
    assert run(torch.tensor([[float("inf"), float("nan"), 0.0, -0.0, 0.0]]), 5).tolist() == [[1, 0, 2, 3, 4]]
    # long runs of equal values force the exact path (every element is a candidate)
    for dt in (BF16, F32):
        for v, k in ((5000, 7), (131000, 64), (2049, 512)):
            z = torch.zeros(3, v, dtype=dt)
            assert torch.equal(run(z, k), torch.arange(k).expand(3, k))
    g = gen(11)
    x = torch.randint(0, 3, (4, 40000), generator=g).to(BF16)         # three distinct values
    assert torch.equal(run(x, 300), O.topk(x, 300)[1])
    x = torch.randint(0, 50, (4, 70000), generator=g).float()
    x[:, ::7] = float("nan")
    x[:, 5::11] = float("-inf")
    assert torch.equal(run(x, 512), O.topk(x, 512)[1])
    # fp16 values that differ only in their last three mantissa bits, in long runs: the exact
    # path must order them by value, not by position
    steps = torch.randint(0, 8, (3, 6000), generator=g).float()
    x = (1.0 + steps * 2.0 ** -10).to(F16) * torch.where(torch.rand(3, 6000, generator=g) < 0.5, 1.0, -1.0).to(F16)
    for k in (5, 100, 512):
        assert torch.equal(run(x, k), O.topk(x, k)[1])
    # k close to the row width: the per-wave threshold admits everything, the exact path decides
    for dt, v, k in ((BF16, 2048, 256), (F32, 1500, 300), (F16, 4096, 512), (BF16, 1100, 512)):
        x = (3 * torch.randn(5, v, generator=g)).to(dt)
        assert torch.equal(run(x, k), O.topk(x, k)[1])
    # short rows (a wave per row): ties, NaNs, -inf and signed zeros
    x = torch.randint(0, 4, (300, 700), generator=g).to(BF16)
    x[::3, ::5] = float("nan")
    x[1::3, 1::7] = float("-inf")
    x[2::3, ::2] = -0.0
    for k in (1, 17, 64, 300, 512):
        assert torch.equal(run(x, k), O.topk(x, k)[1])
    z = torch.zeros(5, 64)
    assert torch.equal(run(z, 64), torch.arange(64).expand(5, 64))
    # the same kernel with 16-byte loads (aligned rows): all-equal rows, few distinct values,
    # k up to the row width, and fp16 values one ulp apart
    for dt in (BF16, F16, F32):
        for v, ks in ((8, (1, 8)), (100, (1, 5, 100)), (1024, (1, 64, 100, 512)), (2048, (7, 64, 257, 512))):
            z = torch.full((3, v), -1.5, dtype=dt)
            x = torch.randint(0, 5, (6, v), generator=g).to(dt)
            x[::2, ::9] = float("nan")
            x[1::2, 3::4] = float("-inf")
            for k in ks:
                assert torch.equal(run(z, k), torch.arange(k).expand(3, k)), (dt, v, k)
                assert torch.equal(run(x, k), O.topk(x, k)[1]), (dt, v, k)
    steps = torch.randint(0, 8, (40, 2048), generator=g).float()
    x = (1.0 + steps * 2.0 ** -10).to(F16) * torch.where(torch.rand(40, 2048, generator=g) < 0.5, 1.0, -1.0).to(F16)
    for k in (3, 64, 200):
        assert torch.equal(run(x, k), O.topk(x, k)[1])
    x = (3 * torch.randn(50, 2048, generator=g)).to(BF16)
    assert torch.equal(run(x, 2048 // 4), O.topk(x, 512)[1])
    x = (3 * torch.randn(9, 300, generator=g))
    assert torch.equal(run(x, 300), O.topk(x, 300)[1])
    # negative NaN payloads and a row of -inf
    x = torch.full((2, 3000), float("-inf"))
    x[0, 17] = -torch.tensor(float("nan"))
    assert torch.equal(run(x, 4), O.topk(x, 4)[1])


def test_topk_lane_group_rows():
    """Rows of at most 512 elements with k <= 8 take lane groups (several rows per wave): every
    group width, widths that are not whole vectors, ties, NaNs, signed zeros, -inf, unaligned
    buffers, and more rows than one workgroup holds."""
    g = gen(1050)

    def check(x, k):
        ov, oi = O.topk(x, k)
        for bits in (torch.int32, torch.int64):
            vals, idx = _hip.topk(x.to(DEV), k, bits)
            assert torch.equal(idx.cpu().long(), oi), (tuple(x.shape), x.dtype, k)
            assert torch.equal(vals.cpu().nan_to_num(7.0), ov.nan_to_num(7.0)), (tuple(x.shape), x.dtype, k)
    for dt in (BF16, F16, F32):
        for v in (1, 2, 7, 8, 16, 60, 64, 65, 100, 128, 129, 200, 256, 257, 384, 500, 512):
            n = 333 if v <= 64 else 77
            x = (3 * torch.randn(n, v, generator=g)).to(dt)
            for k in sorted({1, min(v, 2), min(v, 5), min(v, 8)}):
                check(x, k)
            t = torch.randint(0, 3, (n, v), generator=g).to(dt)         # heavy ties
            t[::5, ::3] = float("nan")
            t[1::5, 1::2] = float("-inf")
            t[2::5, ::2] = -0.0
            for k in sorted({1, min(v, 2), min(v, 8)}):
                check(t, k)
    z = torch.zeros(1000, 64)
    check(z, 8)
    base = (3 * torch.randn(1 + 50 * 128, generator=g)).to(BF16).to(DEV)
    x = base[1:].view(50, 128)                                          # rows 2 bytes off 16-byte alignment
    _, idx = _hip.topk(x, 4, torch.int32)
    assert torch.equal(idx.cpu().long(), O.topk(x.cpu(), 4)[1])


def test_topk_two_wave_rows():
    """Rows of 2-24 K elements with k <= 72 take the 128-thread form (512 candidate slots, half
    the work list): random rows around its bounds, then inputs that overflow its slots or its
    work list and fall to the exact path, NaN / -inf rows, and unaligned rows."""
    g = gen(1012)

    def run(t, k):
        _, i = _hip.topk(t.to(DEV), k, torch.int64)
        return i.cpu()
    for dt, n, v, ks in ((BF16, 40, 2049, (1, 64, 72, 73)), (F16, 9, 8191, (8, 72)), (BF16, 7, 24576, (1, 33, 72)),
                         (F32, 12, 2304, (2, 72)), (F32, 6, 12288, (64, 72, 73)), (BF16, 5, 24584, (72,)),
                         (F32, 4, 12290, (64,)), (BF16, 300, 4096, (64,))):
        x = (3 * torch.randn(n, v, generator=g)).to(dt)
        for k in ks:
            vals, idx = _hip.topk(x.to(DEV), k, torch.int32)
            ov, oi = O.topk(x, k)
            assert torch.equal(idx.cpu().long(), oi) and torch.equal(vals.cpu(), ov), (dt, v, k)
    # every element equal, few distinct values, one vector in each group of eight holding the
    # maximum (the work list sees every vector), a row of NaNs, -inf with a few finite values
    for dt in (BF16, F32):
        for v in (4096, 9000, 20000):
            z = torch.full((3, v), 0.25, dtype=dt)
            assert torch.equal(run(z, 72), torch.arange(72).expand(3, 72))
            x = torch.randint(0, 4, (5, v), generator=g).to(dt)
            assert torch.equal(run(x, 64), O.topk(x, 64)[1]), (dt, v)
            x = torch.randn(4, v, generator=g).to(dt)
            x[:, ::8] = 9.0
            assert torch.equal(run(x, 50), O.topk(x, 50)[1]), (dt, v)
            x = torch.randn(4, v, generator=g).to(dt)
            x[0] = float("nan")
            x[1] = float("-inf")
            x[1, 5::1000] = 1.0
            x[2, 3::5] = float("nan")
            x[3, ::2] = -0.0
            x[3, 1::2] = 0.0
            for k in (1, 20, 72):
                assert torch.equal(run(x, k), O.topk(x, k)[1]), (dt, v, k)
    base = (3 * torch.randn(1 + 6 * 5003, generator=g)).to(BF16).to(DEV)
    x = base[1:].view(6, 5003)                                        # rows start 2 bytes off 16-byte alignment
    assert torch.equal(run(x, 40), O.topk(x.cpu(), 40)[1])


def test_topk_rows_with_signed_zeros_negative_nans_and_denormals():
    """Rows wide enough for the streaming forms, which fold each 16-byte vector to an integer key
    (16-bit for bf16 / fp16, 32-bit for fp32): inputs where that key and the float order could
    part ways."""
    g = gen(1013)

    def ints(dt):
        return torch.int32 if dt == F32 else torch.int16

    def check(x, k):
        vals, idx = _hip.topk(x.to(DEV), k, torch.int64)
        oi = O.topk(x, k)[1]
        assert torch.equal(idx.cpu(), oi), (x.dtype, tuple(x.shape), k)
        # the selected elements themselves, bit for bit (NaN payloads and the sign of zero included)
        want = x.view(ints(x.dtype)).gather(1, oi)
        assert torch.equal(vals.cpu().view(ints(x.dtype)), want), (x.dtype, tuple(x.shape), k)
    for dt in (BF16, F16, F32):
        for v in (5000, 40000, 131072):
            # the k-th value is zero; most zeros are -0.0, whole vectors hold nothing above -0.0
            x = -(torch.randn(3, v, generator=g).abs() + 0.5).to(dt)
            x[:, ::3] = -0.0
            x[:, 1000::997] = 0.0
            for k in (1, 64, 300):
                check(x, k)
            # NaNs of both signs among ordinary values, fewer and more of them than k
            x = (3 * torch.randn(3, v, generator=g)).to(dt)
            bits = x.view(ints(dt))
            neg_nan = {BF16: -64, F16: -512, F32: -4194304}[dt]     # 0xFFC0 / 0xFE00 / 0xFFC00000
            bits[0, 7::501] = neg_nan
            bits[1, 3::1999] = -1                                # all ones
            bits[1, 11::2003] = 0x7FFFFFFF if dt == F32 else 0x7FFF
            bits[2, 5::97] = -3
            for k in (5, 64, 512):
                check(x, k)
            # only negative values, and the infinities
            x = -(torch.randn(3, v, generator=g).abs() * 100 + 1e-3).to(dt)
            x[1, 17::333] = float("-inf")
            x[2, 19::4001] = float("inf")
            for k in (3, 64, 257):
                check(x, k)
            # denormals of both signs around zero (fp16: below 6.1e-5; bf16 / fp32: below 1.2e-38)
            tiny = {F16: 2.0 ** -24, BF16: 2.0 ** -133, F32: 2.0 ** -149}[dt]
            x = (torch.randint(-40, 41, (3, v), generator=g).double() * tiny).to(dt)
            for k in (8, 64, 400):
                check(x, k)
            # few distinct negative values: long tie runs below zero
            x = (-torch.randint(1, 4, (2, v), generator=g).float()).to(dt)
            check(x, 100)
        # values that differ only in their last mantissa bit (below the 16 bits the LDS keeps of an
        # fp32 key): the threshold must not cut between them
        step = torch.finfo(dt).eps
        x = (1.0 + torch.randint(0, 3, (3, 30000), generator=g).double() * step).to(dt)
        x[1] = -x[1]
        for k in (10, 200):
            check(x, k)
    # the largest finite values and one step below (fp16 65504, 65472)
    x = torch.full((2, 30000), 65472.0).to(F16)
    x[:, 5::7] = 65504.0
    x[1] = -x[1]
    check(x, 64)
    check(x, 512)


def test_topk_unaligned_rows():
    g = gen(12)
    for dt, v in ((BF16, 50257), (F32, 32001), (F16, 4099)):
        x = (3 * torch.randn(5, v, generator=g)).to(dt)
        _, idx = _hip.topk(x.to(DEV), 33, torch.int32)
        assert torch.equal(idx.cpu().long(), O.topk(x, 33)[1])
    base = (3 * torch.randn(3 * 9000 + 1, generator=g)).bfloat16().to(DEV)
    x = base[1:].view(3, 9000)                                        # base pointer off by 2 bytes
    _, idx = _hip.topk(x, 20, torch.int32)
    assert torch.equal(idx.cpu().long(), O.topk(x.cpu(), 20)[1])
    x = base[1:1 + 12 * 2048].view(12, 2048)                          # the same for wave-per-row rows
    _, idx = _hip.topk(x, 20, torch.int32)
    assert torch.equal(idx.cpu().long(), O.topk(x.cpu(), 20)[1])


# ------------------------------------------------------------------ softmax
@pytest.mark.parametrize("n,v,dt", [(4, 64, F32), (5, 1000, F32), (3, 4096, F32), (7, 1, F32),
                                     (8, 50257, BF16), (6, 300, F16), (2, 128256, BF16),
                                     (1000, 64, F32), (77, 16, BF16), (3, 4, F32), (33, 512, BF16),
                                     (130, 8, F16), (9, 8192, BF16), (5, 32768, F16), (3, 65536, BF16),
                                     (257, 2048, F32), (4, 32000, BF16), (1000, 33, BF16), (77, 7, F32),
                                     (300, 257, F16), (65, 1023, BF16), (40, 100, F32), (9, 513, F32),
                                     # rows kept on the chip between the passes (registers + LDS): odd widths,
                                     # the widest that fits and one past it
                                     (3, 151937, F16), (2, 98000, F32), (2, 196592, BF16), (2, 196608, BF16),
                                     (3, 65543, BF16)])
def test_softmax(n, v, dt):
    x = torch.randn(n, v, generator=gen(21)).to(dt)
    y = _hip.softmax_fwd(x.to(DEV))
    ref = O.softmax(x)
    assert_close_lowp(y, ref, dt, "softmax", ulps=2.0)
    assert torch.allclose(y.float().sum(-1).cpu(), torch.ones(n), atol=1e-2)


@pytest.mark.parametrize("n,v,dt", [(4, 64, F32), (5, 1000, F32), (7, 1, F32), (8, 50257, BF16), (6, 300, F16),
                                     (2, 128256, BF16), (1000, 64, F32), (77, 16, BF16), (33, 512, BF16),
                                     (9, 8192, BF16), (5, 32768, F16), (3, 65536, BF16), (257, 2048, F32),
                                     (4, 32000, BF16), (1000, 33, BF16), (65, 1023, BF16), (9, 513, F32),
                                     (3, 40000, F32), (6, 16384, F32),
                                     # both rows kept on the chip: 16-bit rows near the 16384 vectors it holds,
                                     # fp32 rows from 8192 vectors on, odd widths, one past the capacity
                                     (3, 128257, F16), (2, 131056, BF16), (2, 131072, BF16), (3, 65530, F32),
                                     (2, 120000, BF16)])
def test_softmax_bwd(n, v, dt):
    g = gen(22)
    y = torch.softmax(2 * torch.randn(n, v, generator=g), -1).to(dt)
    dy = torch.randn(n, v, generator=g).to(dt)
    dx = _hip.softmax_bwd(y.to(DEV), dy.to(DEV))
    ref = O.softmax_bwd(y, dy)
    # (dy - dot) * y: the subtraction cancels up to |dy| + |dot| before it is scaled by y
    cancel = float((dy.float().abs().max() + 1) * y.float().max())
    assert_close_lowp(dx, ref, dt, "softmax_bwd", ulps=2.0, cancel=cancel)
    ref64 = O.softmax_bwd(y.double(), dy.double(), acc=torch.float64)
    assert rel_max(dx, ref64) <= (1e-2 if dt != F32 else 1e-5)


def test_softmax_bwd_unaligned_base_and_determinism():
    g = gen(23)
    for v in (9000, 700):
        base = torch.softmax(torch.randn(3, v, generator=g), -1).bfloat16().reshape(-1)
        pad = torch.zeros(1, dtype=BF16)
        y = torch.cat((pad, base)).to(DEV)[1:].view(3, v)                 # base pointer off by 2 bytes
        dy = torch.randn(3, v, generator=g).bfloat16().to(DEV)
        dx = _hip.softmax_bwd(y, dy)
        assert_close_lowp(dx, O.softmax_bwd(y.cpu(), dy.cpu()), BF16, "softmax_bwd", ulps=2.0, cancel=4.0)
        assert torch.equal(dx, _hip.softmax_bwd(y, dy))


def test_softmax_nan_and_neg_inf_rows():
    y = _hip.softmax_fwd(torch.tensor([[float("nan"), 1.0, 2.0]], device=DEV))
    assert math.isnan(y[0, 0].item())
    y = _hip.softmax_fwd(torch.full((1, 3), float("-inf"), device=DEV))
    assert all(math.isnan(v) for v in y[0].tolist())


# ------------------------------------------------------------------ router
def router_inputs(n, e, seed, dtype=F32):
    """Logits on a 2**-12 grid (distinct values differ by far more than any exp rounding), 1% of
    the rows with four copies of the row maximum and four copies of another value."""
    g = gen(seed)
    lg = torch.round(torch.randn(n, e, generator=g) * 4096) / 4096
    rows = torch.randperm(n, generator=g)[: max(1, n // 100)]
    for r in rows.tolist():
        cols = torch.randperm(e, generator=g)[: min(8, e)]
        lg[r, cols[: len(cols) // 2]] = lg[r].max().clone()
        lg[r, cols[len(cols) // 2:]] = lg[r, cols[-1]].clone()
    return lg.to(dtype)


ROUTE_CASES = [(16384, 64, 2), (1000, 8, 2), (513, 128, 4), (100, 300, 8), (1, 64, 2), (70000, 16, 1),
               (257, 512, 8), (4099, 64, 6), (3, 2, 2),
               # many tiles x many experts: the histograms are scanned by a kernel of their own
               (40000, 64, 2), (9000, 256, 8), (5000, 500, 3), (300000, 8, 1),
               # expert counts around the lane-group sizes, not multiples of eight
               (700, 65, 2), (700, 129, 3), (700, 257, 8), (900, 60, 4), (64, 7, 7),
               # nine to sixteen picks (sorted heads, at least sixteen lanes a row)
               (4000, 512, 10), (700, 128, 16), (300, 16, 16), (900, 24, 12), (2000, 384, 12),
               (513, 200, 9), (70000, 64, 10)]


@pytest.mark.parametrize("n,e,k", ROUTE_CASES)
def test_route_is_bit_exact(n, e, k):
    lg = router_inputs(n, e, 1003)
    oi, ow, oc, oslot, oorder = O.router(lg, k)
    idx, w, counts, slot, order = _hip.route(lg.to(DEV), k)
    torch.cuda.synchronize()
    assert idx.dtype == torch.int32 and counts.dtype == torch.int32
    assert torch.equal(idx.cpu().long(), oi), "expert indices"
    assert torch.equal(counts.cpu().long(), oc), "per-expert counts"
    assert torch.equal(slot.cpu().long(), oslot), "token -> slot permutation"
    assert torch.equal(order.cpu().long(), oorder), "slot -> token permutation"
    assert torch.allclose(w.cpu(), ow, rtol=1e-5, atol=0)
    i2, w2, c2, none_a, none_b = _hip.route(lg.to(DEV), k, want_permutation=False)
    assert none_a is None and none_b is None and torch.equal(i2, idx) and torch.equal(c2, counts)
    # the sums behind the auxiliary losses (forgemind/moe.py:92-95), from the same pass
    *_, stats = _hip.route(lg.to(DEV), k, want_stats=True)
    probs = torch.softmax(lg.double(), -1)
    assert torch.allclose(stats[:e].cpu().double(), probs.sum(0), rtol=1e-4, atol=1e-6)
    lse2 = torch.logsumexp(lg.double(), -1).pow(2).sum()
    assert stats[e].item() == pytest.approx(lse2.item(), rel=1e-4)
    aux, z = O.router_aux(lg, oi)
    got_aux = e * ((counts.cpu().float() / (n * k)) * (stats[:e].cpu() / n)).sum()
    assert got_aux.item() == pytest.approx(aux.item(), rel=1e-4) and (stats[e] / n).item() == pytest.approx(z.item(), rel=1e-4)
    assert stats.shape == (e + 3,)                                   # and finished, as the last two entries
    assert stats[e + 1].item() == pytest.approx(aux.item(), rel=1e-4) and stats[e + 2].item() == pytest.approx(z.item(), rel=1e-4)


ROUTE_BWD_CASES = [(16384, 64, 2, F32), (1000, 8, 2, F32), (513, 128, 4, BF16), (100, 300, 8, F32), (1, 64, 2, F32),
                   (257, 512, 8, F16), (4099, 60, 6, F32), (3, 2, 2, F32), (700, 65, 2, BF16), (900, 256, 8, F32),
                   (600, 512, 10, F32), (300, 40, 16, BF16), (900, 160, 12, F32)]


@pytest.mark.parametrize("n,e,k,dt", ROUTE_BWD_CASES)
def test_route_bwd_matches_the_oracle(n, e, k, dt):
    """The router's gradient (reference: autograd through moe.py:86-95) from one kernel: through
    the weights, the load-balance loss and the z-loss, separately and together."""
    lg = router_inputs(n, e, 1007, dt)
    g = gen(1008)
    gw = torch.randn(n, k, generator=g)
    idx, w, counts, _, _ = _hip.route(lg.to(DEV), k)
    lgd = lg.to(DEV)
    for use_w, ga, gz in ((True, None, None), (False, 0.7, None), (False, None, -1.3), (True, 0.01, 0.001)):
        want = O.router_bwd(lg, k, gw if use_w else None, ga, gz)
        got = _hip.route_bwd(lgd, idx, gw.to(DEV) if use_w else None, counts,
                             None if ga is None else torch.tensor(ga, device=DEV),
                             None if gz is None else torch.tensor(gz, device=DEV))
        assert got.dtype == dt and got.shape == (n, e)
        # the terms that cancel inside (g_p - sum g_p p) p set the absolute error, not the result
        terms = (gw.abs().max().item() if use_w else 0.0) + abs(ga or 0.0) * e / n + abs(gz or 0.0) * 2 / n * 20
        scale = want.abs().max().item()
        tol = (1e-2 if dt != F32 else 2e-5) * scale + 1e-6 * terms
        assert (got.double().cpu() - want).abs().max().item() <= tol, (use_w, ga, gz)
    # nothing upstream: zeros
    assert not _hip.route_bwd(lgd, idx, None, None, None, None).any()


def test_route_half_precision_logits_and_all_equal_rows():
    lg = router_inputs(300, 64, 5, BF16)
    oi, ow, oc, oslot, oorder = O.router(lg, 2)
    idx, w, counts, slot, order = _hip.route(lg.to(DEV), 2)
    assert torch.equal(idx.cpu().long(), oi) and torch.equal(order.cpu().long(), oorder)
    for dt, e, k in ((F16, 128, 4), (BF16, 320, 8), (F16, 24, 3)):
        lg = router_inputs(777, e, 6, dt)
        oi, ow, oc, oslot, oorder = O.router(lg, k)
        idx, w, counts, slot, order = _hip.route(lg.to(DEV), k)
        assert torch.equal(idx.cpu().long(), oi) and torch.equal(order.cpu().long(), oorder), (dt, e, k)
        assert torch.equal(counts.cpu().long(), oc) and torch.allclose(w.cpu(), ow, rtol=1e-5, atol=0)
    # a buffer that starts 4 bytes off a 16-byte line takes the element-wise loads
    base = torch.zeros(500 * 64 + 1, device=DEV)
    lg = router_inputs(500, 64, 7)
    base[1:] = lg.reshape(-1).to(DEV)
    idx, w, counts, slot, order = _hip.route(base[1:].view(500, 64), 2)
    oi, ow, oc, oslot, oorder = O.router(lg, 2)
    assert torch.equal(idx.cpu().long(), oi) and torch.equal(slot.cpu().long(), oslot)
    z = torch.zeros(130, 64, device=DEV)
    idx, w, counts, slot, order = _hip.route(z, 2)
    assert torch.equal(idx.cpu(), torch.tensor([[0, 1]], dtype=torch.int32).expand(130, 2))
    assert counts.cpu().tolist() == [130, 130] + [0] * 62
    assert torch.allclose(w.cpu(), torch.full((130, 2), 0.5))
    assert order.cpu().tolist() == list(range(0, 260, 2)) + list(range(1, 260, 2))


def test_route_pick_forms_on_special_rows():
    """The router picks by scanning a lane's eight keys per pick (few picks), from lane-sorted keys
    (more picks), or, for 129-256 experts and five picks or more, by sorting the experts that reach a
    lower bound of the k-th key across the lanes: all against the oracle on rows of equal logits
    (every expert is a candidate: the list is taken in several rounds), rows with a single finite
    logit (the other picks tie at probability zero), few distinct values, runs of equal logits of
    every length around the row width, and NaN / +inf rows (all probabilities NaN: lowest experts
    win)."""
    if True:
        for e in (8, 60, 64, 130, 136, 200, 256, 512):
            lg = router_inputs(400, e, 1021)
            lg[0] = 0.25
            lg[1] = float("-inf")
            lg[1, e // 2] = 1.0
            lg[2] = torch.randint(0, 3, (e,), generator=gen(e)).float()
            lg[3, e - 1] = float("nan")
            lg[4, 1] = float("inf")
            lg[5] = float("-inf")
            lg[5, [0, e - 1]] = 2.0
            # rows 6..: the m largest logits are equal, for m around 8, 24, 32, 56 and the row width
            runs = [m for m in (7, 8, 9, 23, 24, 25, 31, 32, 33, 55, 56, 57, e - 1, e) if m <= e]
            for i, m in enumerate(runs):
                perm = torch.randperm(e, generator=gen(100 + i))
                lg[6 + i, perm[:m]] = 9.0
            finite = torch.ones(400, dtype=torch.bool)
            finite[3] = finite[4] = False
            for k in (1, 2, 4, 5, 8):
                if k > e:
                    continue
                out = _hip.route(lg.to(DEV), k, want_stats=True)
                idx, w = out[0].cpu().long(), out[1].cpu()
                oi, ow = O.router(lg[finite], k)[:2]
                assert torch.equal(idx[finite], oi), (e, k)
                assert torch.allclose(w[finite], ow, rtol=1e-5, atol=0), (e, k)
                assert idx[3].tolist() == list(range(k)) and idx[4].tolist() == list(range(k)), (e, k)
                assert torch.isnan(w[3]).all() and torch.isnan(w[4]).all()
                assert torch.equal(out[2].cpu().long(), torch.bincount(idx.flatten(), minlength=e)), (e, k)


def test_route_statistics_from_one_or_two_kernels():
    """Small problems (up to 127 experts, 256 tiles) fold the statistics inside the kernel that
    finishes the auxiliary losses, larger ones in a kernel of their own: both against the oracle."""
    for n, e, k in ((16384, 64, 2), (1000, 8, 2), (513, 127, 4), (3, 2, 2), (9000, 100, 8), (1, 64, 1),
                    (4000, 128, 2), (70000, 200, 6)):
        lg = router_inputs(n, e, 1031)
        idx, w, counts, slot, order, stats = _hip.route(lg.to(DEV), k, True, True)
        oi = O.router(lg, k)[0]
        assert torch.equal(idx.cpu().long(), oi), (n, e, k)
        aux, z = O.router_aux(lg, oi)
        probs = torch.softmax(lg.double(), -1)
        assert torch.allclose(stats[:e].double().cpu(), probs.sum(0), rtol=2e-5, atol=1e-6), (n, e, k)
        assert stats[e + 1].item() == pytest.approx(aux.item(), rel=2e-5), (n, e, k)
        assert stats[e + 2].item() == pytest.approx(z.item(), rel=2e-5), (n, e, k)


# ------------------------------------------------------------------ gather / combine around the permutation
@pytest.mark.parametrize("n,e,k,d,dt", [(1000, 8, 2, 1024, BF16), (257, 16, 4, 100, F32), (64, 4, 1, 7, F16),
                                         (2048, 64, 2, 4096, BF16), (33, 8, 8, 256, F32),
                                         (500, 64, 10, 1024, BF16), (129, 16, 16, 100, F32), (77, 32, 12, 7, F16)])
def test_moe_gather_and_combine(n, e, k, d, dt):
    g = gen(1007)
    lg = router_inputs(n, e, 77)
    idx, w, counts, slot, order = O.router(lg, k)
    x = torch.randn(n, d, generator=g).to(dt)
    ys = torch.randn(n * k, d, generator=g).to(dt)
    o32, s32 = order.to(torch.int32).to(DEV), slot.to(torch.int32).to(DEV)
    xs = _hip.moe_gather(x.to(DEV), o32, k)
    assert torch.equal(xs.cpu(), O.moe_gather(x, order, k))                    # a pure copy: bit-exact
    assert torch.equal(_hip.moe_scatter(x.to(DEV), s32, k), xs)                # the same move from the token's side
    out = _hip.moe_combine(ys.to(DEV), w.to(DEV), s32, n, k)
    ref = O.moe_combine(ys, w, order, k, n)
    # the reference rounds each w*y product and each partial sum to the activation dtype
    assert_close_lowp(out, ref, dt, "combine", ulps=2.0, cancel_lowp=k * float(ys.float().abs().max()))
    # unit weights undo the gather: k copies of each token (exact for k <= 2: x and 2x need no rounding)
    back = _hip.moe_combine(xs, None, s32, n, k)
    if k <= 2:
        assert torch.equal(back.float().cpu(), (x.float() * k).to(dt).float())
    else:
        assert torch.allclose(back.float().cpu(), x.float() * k, rtol=2.0 ** -7 if dt != F32 else 1e-6)
    # the two backward uses: weighted gather and the weight gradient
    dout = torch.randn(n, d, generator=g).to(dt)
    dys = _hip.moe_gather(dout.to(DEV), o32, k, w.reshape(-1).to(DEV))
    want = (dout.float()[(order // k)] * w.reshape(-1)[order][:, None]).to(dt)
    assert_close_lowp(dys, want, dt, "combine backward wrt ys", ulps=2.0)
    assert torch.equal(_hip.moe_scatter(dout.to(DEV), s32, k, w.reshape(-1).to(DEV)), dys)
    dw = _hip.moe_combine_dw(ys.to(DEV), dout.to(DEV), s32, n, k)
    want_dw = (ys.float()[slot].view(n, k, d) * dout.float()[:, None, :]).sum(-1)
    assert torch.allclose(dw.cpu(), want_dw, rtol=1e-4, atol=1e-4 * float(want_dw.abs().max()))


# ------------------------------------------------------------------ SwiGLU epilogues
@pytest.mark.parametrize("shape,dt", [((37,), F32), ((4096,), F32), ((300, 11008), BF16), ((7, 33), F16),
                                       ((2, 5, 64), BF16)])
def test_swiglu_fwd_bwd(shape, dt):
    g = gen(31)
    a, b, dy = (torch.randn(*shape, generator=g).to(dt) for _ in range(3))
    ar, br = a.float().requires_grad_(True), b.float().requires_grad_(True)
    ref = torch.nn.functional.silu(ar) * br
    b = b.detach()
    ref.backward(dy.float())
    y = _hip.swiglu_fwd(a.to(DEV), b.to(DEV))
    da, db = _hip.swiglu_bwd(a.to(DEV), b.to(DEV), dy.to(DEV))
    assert_close_lowp(y, ref.detach(), dt, "swiglu", ulps=2.0)
    assert_close_lowp(da, ar.grad, dt, "dgate", ulps=3.0, cancel=float(dy.float().abs().max() * b.float().abs().max()))
    assert_close_lowp(db, br.grad, dt, "dup", ulps=3.0)


@pytest.mark.parametrize("rows,h,dt", [(6, 8, F32), (5, 6, F32), (3, 32, BF16), (200, 11008, BF16), (9, 1, F32),
                                        (4, 100, F16)])
def test_swiglu_split_fwd_bwd(rows, h, dt):
    g = gen(32)
    x = torch.randn(rows, 2 * h, generator=g).to(dt)
    dy = torch.randn(rows, h, generator=g).to(dt)
    xr = x.float().requires_grad_(True)
    ref = torch.nn.functional.silu(xr[:, :h]) * xr[:, h:]
    ref.backward(dy.float())
    y = _hip.swiglu_split_fwd(x.to(DEV))
    dx = _hip.swiglu_split_bwd(x.to(DEV), dy.to(DEV))
    assert_close_lowp(y, ref.detach(), dt, "swiglu_split", ulps=2.0)
    assert_close_lowp(dx, xr.grad, dt, "dx", ulps=3.0, cancel=float(dy.float().abs().max() * x.detach().float().abs().max()))


# ------------------------------------------------------------------ per-head RMSNorm + RoPE
@pytest.mark.parametrize("b,t,h,hd,dt,wdt", [(2, 5, 3, 4, F32, F32), (1, 7, 2, 8, F32, F32), (2, 3, 4, 6, F32, F32),
                                              (2, 64, 8, 64, BF16, F32), (1, 33, 4, 32, F16, F16), (2, 16, 2, 256, BF16, BF16),
                                              # heads of four or eight vectors (one vector per lane, partner by lane
                                              # permute): 1, 2 and 4 heads per lane group, several tiles
                                              (2, 9, 6, 32, BF16, F32), (1, 5, 3, 32, BF16, BF16), (2, 7, 8, 16, BF16, F32),
                                              (3, 4, 5, 16, F32, F32), (2, 300, 8, 32, BF16, F32), (1, 130, 2, 8, F32, F32),
                                              # halves of 5, 6, 3, 7 and 12 vectors (head sizes 80, 96, 48, 112, 192; 24 in
                                              # fp32): lane groups of exactly that width, idle lanes at the end of a wave,
                                              # odd and even head counts, several tiles
                                              (2, 37, 8, 40, BF16, F32), (1, 301, 3, 48, BF16, BF16), (2, 9, 4, 24, F16, F16),
                                              (1, 50, 6, 56, BF16, F32), (2, 11, 2, 96, BF16, F32), (3, 21, 5, 12, F32, F32)])
def test_qk_norm_rope_fwd_bwd(b, t, h, hd, dt, wdt):
    # shapes of reference tests/kernel_interp_check.py:82-89, then realistic head sizes
    g = gen(41)
    d = 2 * hd
    x = torch.randn(b, t, h, d, generator=g).to(dt)
    w = (1 + 0.1 * torch.randn(d, generator=g)).to(wdt)
    cos, sin = torch.randn(t, hd, generator=g), torch.randn(t, hd, generator=g)
    do = torch.randn(b, t, h, d, generator=g).to(dt)
    xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
    r = torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + 1e-6)
    y = xr * r * wr
    y1, y2 = y.chunk(2, -1)
    c, s = cos.view(1, t, 1, hd), sin.view(1, t, 1, hd)
    ref = torch.cat((y1 * c - y2 * s, y1 * s + y2 * c), -1)
    ref.backward(do.float())
    out, rstd = _hip.qk_norm_rope_fwd(x.to(DEV), w.to(DEV), cos.to(DEV), sin.to(DEV), 1e-6)
    dx, dw = _hip.qk_norm_rope_bwd(x.to(DEV), w.to(DEV), cos.to(DEV), sin.to(DEV), rstd, do.to(DEV))
    scale = float(ref.detach().abs().max())
    assert_close_lowp(out, ref.detach(), dt, "qk_norm_rope", ulps=3.0, cancel=scale)
    assert_close_lowp(dx, xr.grad, dt, "dx", ulps=4.0, cancel=float(xr.grad.abs().max()) * 4)
    assert rel_max(dw, wr.grad) <= (1e-2 if wdt != F32 else 1e-4)


def test_router_where_probabilities_leave_the_normal_range():
    """A pick whose probability is below 2^-126 (its logit more than 87.3 under the row maximum):
    the hardware exponential flushes it to zero, so such picks tie and go to the lowest expert
    index, where a CPU softmax still tells denormals apart (and rounds them to a grid of 1.4e-45,
    so its own order there is an artefact of the rounding as well). Pinned here: rows whose k-th
    largest logit is within 86 of the maximum match the oracle bit for bit; beyond 88 the picks
    follow the flush-to-zero model exactly (the deviation is confined to that window and to the
    places after the last normal probability)."""
    g = torch.Generator().manual_seed(5150)
    n, e, k = 512, 64, 4
    for gap, exact in ((60.0, True), (80.0, True), (86.0, True), (88.0, False), (95.0, False), (120.0, False)):
        lg = -torch.round(torch.rand(n, e, generator=g) * 256) / 256   # the field: (-1, 0] on a 1/256 grid
        top2 = torch.stack([torch.randperm(e, generator=g)[:2] for _ in range(n)])
        lg.scatter_(1, top2, torch.tensor([gap, gap - 0.5]).expand(n, 2).contiguous())   # picks 3, 4 sit gap .. gap + 1 below the maximum
        idx, w, counts, slot, order = _hip.route(lg.to(DEV), k)
        oi, ow, oc, oslot, oorder = O.router(lg, k)
        if exact:
            assert torch.equal(idx.cpu().long(), oi), gap
            assert torch.allclose(w.cpu(), ow, rtol=1e-5, atol=1e-37)
        else:
            # flush-to-zero model: probabilities below 2^-126 are zero, ties to the lowest index
            p = torch.softmax(lg.double(), -1)
            p = torch.where(p < 2.0 ** -126, torch.zeros_like(p), p).float()
            mi = O.topk(p, k)[1]
            assert torch.equal(idx.cpu().long(), mi), gap
            assert torch.equal(idx.cpu().long()[:, :2], oi[:, :2])          # the normal picks agree with the oracle
        flat = idx.reshape(-1).long().cpu()
        assert torch.equal(counts.cpu().long(), torch.bincount(flat, minlength=e))
        assert torch.equal(order.cpu().long(), torch.from_numpy(np.argsort(flat.numpy(), kind="stable")))

"""Pins the CPU oracle before anything is compared against it.

Each oracle function is checked against (a) the library routine the reference's own tests use
as their yardstick, (b) the reference's known-answer tests, re-typed here as data, (c) closed
forms / invariants, and (d) brute-force loops on tiny inputs -- chosen so that a dropped term,
a wrong sign, a transposed operand or a wrong divisor fails at least one check.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O

F64 = torch.float64


# ------------------------------------------------------------------ rms_norm
@pytest.mark.parametrize("d", [1, 3, 4, 8, 16, 100])
@pytest.mark.parametrize("eps", [1e-6, 1e-5])
def test_rms_norm_is_torch_rms_norm(d, eps):
    # reference tests/test_kernels.py:37-46 and tests/test_edge_cases.py:115-120 (d == 1)
    torch.manual_seed(d)
    x, w = torch.randn(5, d), torch.randn(d)
    y, rstd = O.rms_norm(x, w, eps)
    assert torch.allclose(y, F.rms_norm(x, (d,), w, eps), atol=2e-6, rtol=1e-5)
    assert torch.allclose(rstd, torch.rsqrt(x.pow(2).mean(-1) + eps), rtol=1e-6)


def test_rms_norm_closed_forms():
    x = torch.randn(7, 64, dtype=F64)
    y, rstd = O.rms_norm(x, torch.ones(64, dtype=F64), 0.0, acc=F64)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(7, dtype=F64), atol=1e-12)   # unit RMS
    z, rz = O.rms_norm(torch.zeros(2, 8), torch.ones(8), 1e-6)
    assert torch.equal(z, torch.zeros(2, 8)) and torch.allclose(rz, torch.full((2,), 1e3))
    # scaling the input leaves the output unchanged when eps == 0
    y2, _ = O.rms_norm(3.0 * x, torch.ones(64, dtype=F64), 0.0, acc=F64)
    assert torch.allclose(y, y2, atol=1e-12)


def test_rms_norm_half_inputs_round_once():
    torch.manual_seed(0)
    x = torch.randn(9, 48).bfloat16()
    w = (1 + 0.02 * torch.randn(48))
    y, _ = O.rms_norm(x, w, 1e-6)
    ref = F.rms_norm(x.float(), (48,), w, 1e-6).bfloat16()
    assert y.dtype == torch.bfloat16
    # same fp32 math up to association; at most one bf16 ulp apart, almost always equal
    assert (y.float() - ref.float()).abs().max() <= 2 ** -7 * ref.float().abs().max()
    assert (y != ref).float().mean() < 0.02


def test_rms_norm_backward_is_autograd_of_torch_rms_norm():
    # reference tests/test_kernels.py:49-60, fp64 like tests/test_nn_blocks.py:66-77
    torch.manual_seed(1)
    x = torch.randn(6, 8, dtype=F64, requires_grad=True)
    w = torch.randn(8, dtype=F64, requires_grad=True)
    g = torch.randn(6, 8, dtype=F64)
    F.rms_norm(x, (8,), w, 1e-6).backward(g)
    dx, dw = O.rms_norm_bwd(x.detach(), w.detach(), g, 1e-6, acc=F64)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dw, w.grad, atol=1e-12)
    # dx is orthogonal to x when eps == 0
    dx0, _ = O.rms_norm_bwd(x.detach(), w.detach(), g, 0.0, acc=F64)
    assert (dx0 * x.detach()).sum(-1).abs().max() < 1e-12


def test_rms_norm_non_contiguous_input():
    # reference tests/test_edge_cases.py:106-111
    x = torch.randn(4, 8).t().contiguous().t()
    w = torch.randn(8)
    assert not x.is_contiguous()
    assert torch.allclose(O.rms_norm(x, w)[0], F.rms_norm(x, (8,), w, 1e-6), atol=2e-6)


# ------------------------------------------------------------------ add_rms_norm
def test_add_rms_norm_rounding_points():
    # reference tests/test_kernels.py:63-69: xn == x + delta with atol 0, y == rms_norm(xn)
    torch.manual_seed(0)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        x, d = torch.randn(4, 8).to(dt), torch.randn(4, 8).to(dt)
        w = torch.randn(8)
        xn, y, _ = O.add_rms_norm(x, d, w)
        assert torch.equal(xn, x + d)
        assert torch.equal(y, O.rms_norm(x + d, w)[0])


def test_add_rms_norm_backward_is_autograd():
    # reference tests/test_nn_blocks.py:101-106: dx == ddelta, both from autograd
    torch.manual_seed(2)
    x = torch.randn(5, 12, dtype=F64, requires_grad=True)
    dl = torch.randn(5, 12, dtype=F64, requires_grad=True)
    w = torch.randn(12, dtype=F64, requires_grad=True)
    gy, gxn = torch.randn(5, 12, dtype=F64), torch.randn(5, 12, dtype=F64)
    xn = x + dl
    y = F.rms_norm(xn, (12,), w, 1e-5)
    torch.autograd.backward([xn, y], [gxn, gy])
    dx, dw = O.add_rms_norm_bwd(xn.detach(), w.detach(), gy, gxn, 1e-5, acc=F64)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dx, dl.grad, atol=1e-12)
    assert torch.allclose(dw, w.grad, atol=1e-12)
    dx0, _ = O.add_rms_norm_bwd(xn.detach(), w.detach(), gy, None, 1e-5, acc=F64)
    assert torch.allclose(dx0, dx - gxn, atol=1e-12)


# ------------------------------------------------------------------ layer_norm
@pytest.mark.parametrize("d", [1, 3, 8, 100])
@pytest.mark.parametrize("bias", [True, False])
def test_layer_norm_is_torch_layer_norm(d, bias):
    torch.manual_seed(d)
    x, w = 2 + torch.randn(5, d), torch.randn(d)
    b = torch.randn(d) if bias else None
    y, mean, rstd = O.layer_norm(x, w, b, 1e-5)
    assert torch.allclose(y, F.layer_norm(x, (d,), w, b, 1e-5), atol=2e-6, rtol=1e-5)
    assert torch.allclose(mean, x.mean(-1), atol=1e-6)
    assert torch.allclose(rstd, torch.rsqrt(x.var(-1, unbiased=False) + 1e-5), rtol=1e-5)


def test_layer_norm_closed_forms():
    x = 5 + torch.randn(7, 64, dtype=F64)
    y, _, _ = O.layer_norm(x, torch.ones(64, dtype=F64), None, 0.0, acc=F64)
    assert y.mean(-1).abs().max() < 1e-12 and torch.allclose(y.var(-1, unbiased=False),
                                                             torch.ones(7, dtype=F64), atol=1e-12)
    # invariant under shift and positive scaling of the input when eps == 0
    y2, _, _ = O.layer_norm(3.0 * x - 11.0, torch.ones(64, dtype=F64), None, 0.0, acc=F64)
    assert torch.allclose(y, y2, atol=1e-10)
    # a constant row: zero centred values, output is the bias
    b = torch.randn(8)
    yc, mc, rc = O.layer_norm(torch.full((2, 8), 3.0), torch.ones(8), b, 1e-5)
    assert torch.equal(yc, b.expand(2, 8)) and torch.equal(mc, torch.full((2,), 3.0))
    assert torch.allclose(rc, torch.full((2,), 1e-5 ** -0.5))


def test_layer_norm_backward_is_autograd_of_torch_layer_norm():
    torch.manual_seed(3)
    x = torch.randn(6, 10, dtype=F64, requires_grad=True)
    w = torch.randn(10, dtype=F64, requires_grad=True)
    b = torch.randn(10, dtype=F64, requires_grad=True)
    g = torch.randn(6, 10, dtype=F64)
    F.layer_norm(x, (10,), w, b, 1e-5).backward(g)
    dx, dw, db = O.layer_norm_bwd(x.detach(), w.detach(), g, 1e-5, acc=F64)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dw, w.grad, atol=1e-12)
    assert torch.allclose(db, b.grad, atol=1e-12)
    assert dx.sum(-1).abs().max() < 1e-12                       # dx has no mean component
    dx0, _, _ = O.layer_norm_bwd(x.detach(), w.detach(), g, 0.0, acc=F64)
    xc = x.detach() - x.detach().mean(-1, keepdim=True)
    assert (dx0 * xc).sum(-1).abs().max() < 1e-11               # nor one along the centred row


def test_add_layer_norm_rounding_points_and_backward():
    torch.manual_seed(4)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        x, d = torch.randn(4, 8).to(dt), torch.randn(4, 8).to(dt)
        w, b = torch.randn(8), torch.randn(8)
        xn, y, _, _ = O.add_layer_norm(x, d, w, b)
        assert torch.equal(xn, x + d) and torch.equal(y, O.layer_norm(x + d, w, b)[0])
    x = torch.randn(5, 12, dtype=F64, requires_grad=True)
    dl = torch.randn(5, 12, dtype=F64, requires_grad=True)
    w = torch.randn(12, dtype=F64, requires_grad=True)
    gy, gxn = torch.randn(5, 12, dtype=F64), torch.randn(5, 12, dtype=F64)
    xn = x + dl
    torch.autograd.backward([xn, F.layer_norm(xn, (12,), w, None, 1e-5)], [gxn, gy])
    dx, dw, _ = O.layer_norm_bwd(xn.detach(), w.detach(), gy, 1e-5, gxn=gxn, acc=F64)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dx, dl.grad, atol=1e-12)
    assert torch.allclose(dw, w.grad, atol=1e-12)


# ------------------------------------------------------------------ cross entropy
def test_ce_is_torch_cross_entropy():
    # reference tests/test_edge_cases.py:39-47
    torch.manual_seed(0)
    lg = torch.randn(9, 16, dtype=F64, requires_grad=True)
    y = torch.randint(0, 16, (9,))
    y[2] = -100
    ref = F.cross_entropy(lg, y, ignore_index=-100, reduction="mean")
    ref.backward()
    loss, grad = O.cross_entropy(lg.detach(), y, acc=F64)
    assert loss.item() == pytest.approx(ref.item(), rel=1e-12)
    assert torch.allclose(grad, lg.grad, atol=1e-14)


def test_ce_known_answers():
    # all labels ignored -> 0.0, gradient all zero (reference tests/test_edge_cases.py:21-28)
    loss, grad = O.cross_entropy(torch.randn(6, 16), torch.full((6,), -100))
    assert loss.item() == 0.0 and not grad.any()
    # empty batch -> 0.0 (tests/test_edge_cases.py:31-36)
    loss, grad = O.cross_entropy(torch.randn(0, 16), torch.zeros(0, dtype=torch.long))
    assert loss.item() == 0.0 and grad.shape == (0, 16)
    # uniform logits: loss == log(V)
    loss, _ = O.cross_entropy(torch.zeros(3, 10), torch.tensor([0, 5, 9]))
    assert loss.item() == pytest.approx(math.log(10), rel=1e-6)
    # 3-D logits reduce like the flattened ones (tests/test_edge_cases.py:50-56)
    lg, y = torch.randn(2, 5, 16), torch.randint(0, 16, (2, 5))
    a, _ = O.cross_entropy(lg, y)
    b, _ = O.cross_entropy(lg.reshape(10, 16), y.reshape(10))
    assert a.item() == pytest.approx(b.item(), rel=1e-6)


def test_ce_brute_force_and_invariants():
    torch.manual_seed(3)
    lg = torch.randn(4, 7, dtype=F64)
    y = torch.tensor([3, -100, 0, 6])
    loss, grad = O.cross_entropy(lg, y, acc=F64)
    total, n = 0.0, 0
    for i in range(4):
        if y[i] == -100:
            continue
        row = [lg[i, j].item() for j in range(7)]
        total += math.log(sum(math.exp(v) for v in row)) - row[y[i]]
        n += 1
    assert loss.item() == pytest.approx(total / n, rel=1e-12)
    assert grad[1].abs().max() == 0                                   # ignored row
    assert grad[[0, 2, 3]].sum(-1).abs().max() < 1e-15                # softmax - onehot sums to 0
    assert (grad[0, 3] < 0) and (grad[0, [0, 1, 2, 4, 5, 6]] > 0).all()  # sign of the onehot term
    assert (grad[[0, 2, 3]] * n).abs().max() <= 1.0


def test_ce_bf16_logits_use_fp32_math():
    torch.manual_seed(4)
    lg = (2 * torch.randn(64, 1000)).bfloat16()
    y = torch.randint(0, 1000, (64,))
    loss, grad = O.cross_entropy(lg, y)
    ref = F.cross_entropy(lg.float(), y, reduction="sum") / 64
    assert loss.dtype == torch.float32 and grad.dtype == torch.bfloat16
    assert loss.item() == pytest.approx(ref.item(), rel=1e-6)


# ------------------------------------------------------------------ KL
def test_kl_is_torch_kl_div():
    # reference tests/test_kernels.py:115-129
    torch.manual_seed(0)
    s, t = torch.randn(6, 40, dtype=F64), torch.randn(6, 40, dtype=F64)
    loss, grad = O.kl_div(s, t, "mean", acc=F64)
    ref = F.kl_div(F.log_softmax(s, -1), F.softmax(t, -1), reduction="sum") / 6
    assert loss.item() == pytest.approx(ref.item(), rel=1e-12)
    assert torch.allclose(grad, (F.softmax(s, -1) - F.softmax(t, -1)) / 6, atol=1e-15)


def test_kl_reductions_and_known_answers():
    torch.manual_seed(1)
    s, t = torch.randn(5, 33), torch.randn(5, 33)
    rows, g_none = O.kl_div(s, t, "none")
    assert rows.shape == (5,) and (rows >= 0).all()                     # Gibbs
    assert O.kl_div(s, t, "sum")[0].item() == pytest.approx(rows.sum().item(), rel=1e-6)
    assert O.kl_div(s, t, "mean")[0].item() == pytest.approx(rows.mean().item(), rel=1e-6)
    assert torch.allclose(O.kl_div(s, t, "mean")[1] * 5, g_none, atol=1e-7)
    assert g_none.sum(-1).abs().max() < 1e-6                            # p_s - p_t sums to 0
    z, gz = O.kl_div(s, s.clone(), "mean")
    assert abs(z.item()) < 1e-7 and gz.abs().max() < 1e-7               # identical -> 0
    # V == 1 -> 0 (reference tests/test_edge_cases.py:123-126)
    assert O.kl_div(torch.randn(3, 1), torch.randn(3, 1))[0].item() == pytest.approx(0.0, abs=1e-6)
    with pytest.raises(ValueError):
        O.kl_div(s, t, "bogus")


def test_kl_temperature_is_a_rescaling_of_the_logits():
    torch.manual_seed(2)
    s = torch.randn(4, 50, dtype=F64, requires_grad=True)
    t = torch.randn(4, 50, dtype=F64)
    T = 2.0
    ref = F.kl_div(F.log_softmax(s / T, -1), F.softmax(t / T, -1), reduction="sum") / 4
    ref.backward()
    loss, grad = O.kl_div(s.detach(), t, "mean", temperature=T, acc=F64)
    assert loss.item() == pytest.approx(ref.item(), rel=1e-12)
    assert torch.allclose(grad, s.grad, atol=1e-15)


# ------------------------------------------------------------------ softmax
def test_softmax_matches_torch():
    # reference tests/test_softmax.py:32-40, 60-71
    for shape in [(4, 64), (5, 1000), (2, 300, 97), (7, 1)]:
        x = torch.randn(*shape)
        assert torch.allclose(O.softmax(x), torch.softmax(x, -1), rtol=1e-5, atol=1e-6)
    y = O.softmax(torch.tensor([[float("nan"), 1.0, 2.0]]))
    assert math.isnan(y[0, 0])
    y = O.softmax(torch.tensor([[float("-inf")] * 3]))
    assert all(math.isnan(v) for v in y[0].tolist())


def test_softmax_bwd_matches_autograd():
    # pinned by torch's own derivative of softmax and by what the mathematics fixes: gradient
    # rows sum to zero, a constant upstream gradient gives zero, a one-hot y gives zero
    for shape in [(4, 64), (5, 1000), (2, 3, 97), (7, 1)]:
        x = torch.randn(*shape, dtype=torch.float64, requires_grad=True)
        g = torch.randn(*shape, dtype=torch.float64)
        y = torch.softmax(x, -1)
        y.backward(g)
        got = O.softmax_bwd(y.detach(), g, acc=torch.float64)
        assert torch.allclose(got, x.grad, rtol=1e-12, atol=1e-14)
        assert got.sum(-1).abs().max() < 1e-12
    y = torch.softmax(torch.randn(3, 50), -1)
    assert O.softmax_bwd(y, torch.full((3, 50), 2.5)).abs().max() < 1e-6
    onehot = torch.zeros(2, 9)
    onehot[:, 4] = 1.0
    assert O.softmax_bwd(onehot, torch.randn(2, 9)).abs().max() == 0
    yb = torch.softmax(torch.randn(4, 300), -1).bfloat16()
    gb = torch.randn(4, 300).bfloat16()
    assert O.softmax_bwd(yb, gb).dtype == torch.bfloat16
    ref = O.softmax_bwd(yb.double(), gb.double(), acc=torch.float64)
    assert torch.allclose(O.softmax_bwd(yb, gb).double(), ref, rtol=2 ** -7, atol=1e-6)


# ------------------------------------------------------------------ top-k
def _canonical(v, idx):
    k = v.shape[-1]
    v2, i2 = v.reshape(-1, k), idx.reshape(-1, k)
    for r in range(v2.shape[0]):
        for j in range(k - 1):
            a, b = v2[r, j], v2[r, j + 1]
            assert a >= b or torch.isnan(a)
            if a == b and not torch.isnan(a):
                assert i2[r, j] < i2[r, j + 1]


@pytest.mark.parametrize("shape,k", [
    ((4, 64), 8), ((2, 100), 1), ((2, 100), 99), ((1, 512), 512), ((3, 4096), 64),
    ((2, 5000), 100), ((4, 128), 17), ((5, 1), 1), ((2, 600), 4), ((4, 5000), 512),
    ((2, 300, 97), 12),
])
def test_topk_multiset_matches_torch(shape, k):
    # the eleven cases of reference tests/test_topk.py:53-65
    torch.manual_seed(0)
    x = torch.randn(*shape)
    v, idx = O.topk(x, k)
    tv, _ = torch.topk(x, k, dim=-1)
    assert torch.equal(v.sort(-1).values, tv.sort(-1).values)
    assert torch.equal(torch.gather(x, -1, idx), v)
    assert idx.dtype == torch.int64
    _canonical(v, idx)


def test_topk_known_answers():
    # reference tests/test_topk.py:68-74
    v, idx = O.topk(torch.tensor([[1.0, 3.0, 3.0, 2.0, 3.0]]), 3)
    assert v[0].tolist() == [3.0, 3.0, 3.0] and idx[0].tolist() == [1, 2, 4]
    # reference tests/test_topk.py:77-85
    v, idx = O.topk(torch.tensor([[float("nan"), 1.0, 2.0, float("nan"), 0.0]]), 3)
    assert math.isnan(v[0, 0]) and math.isnan(v[0, 1]) and idx[0, :2].tolist() == [0, 3]
    assert v[0, 2].item() == 2.0
    # NaN outranks +inf; the two zeros tie and keep index order
    _, idx = O.topk(torch.tensor([[float("inf"), float("nan"), 0.0, -0.0, 0.0]]), 5)
    assert idx[0].tolist() == [1, 0, 2, 3, 4]
    # reference tests/test_topk.py:88-95
    with pytest.raises(RuntimeError, match="selected index k out of range"):
        O.topk(torch.randn(4, 8), 9)
    with pytest.raises(RuntimeError, match="selected index k out of range"):
        O.topk(torch.randn(4, 8), 0)


def test_topk_brute_force_with_heavy_ties():
    g = torch.Generator().manual_seed(5)
    x = torch.randint(0, 4, (6, 23), generator=g).float()
    _, idx = O.topk(x, 9)
    for r in range(6):
        pairs = sorted(((-x[r, j].item(), j) for j in range(23)))
        assert idx[r].tolist() == [j for _, j in pairs[:9]]


# ------------------------------------------------------------------ router
def test_router_integer_closed_forms_and_invariants():
    torch.manual_seed(0)
    n, e, k = 257, 16, 3
    logits = torch.round(torch.randn(n, e) * 8) / 8          # coarse grid: plenty of exact ties
    idx, w, counts, slot, order = O.router(logits, k)
    flat = idx.reshape(-1).numpy()
    assert np.array_equal(counts.numpy(), np.bincount(flat, minlength=e)) and counts.sum() == n * k
    assert np.array_equal(order.numpy(), np.argsort(flat, kind="stable"))
    assert np.array_equal(slot.numpy()[order.numpy()], np.arange(n * k))
    grouped = flat[order.numpy()]
    assert (np.diff(grouped) >= 0).all()
    for ex in range(e):                                    # ascending positions inside an expert
        seg = order.numpy()[grouped == ex]
        assert (np.diff(seg) > 0).all()
    assert torch.allclose(w.sum(-1), torch.ones(n), atol=1e-6)
    assert (w[:, :-1] >= w[:, 1:]).all()
    assert all(len(set(r)) == k for r in idx.tolist())


def test_router_brute_force_small():
    logits = torch.tensor([[0.0, 1.0, 1.0, -1.0], [2.0, 2.0, 2.0, 2.0], [0.5, -0.5, 0.25, 0.5]])
    idx, w, counts, slot, order = O.router(logits, 2)
    assert idx.tolist() == [[1, 2], [0, 1], [0, 3]]         # ties -> lowest expert first
    p = [[math.exp(v) for v in row] for row in logits.tolist()]
    p = [[v / sum(row) for v in row] for row in p]
    for r, (a, b) in enumerate(idx.tolist()):
        tot = p[r][a] + p[r][b]
        assert w[r].tolist() == pytest.approx([p[r][a] / tot, p[r][b] / tot], rel=1e-6)
    assert counts.tolist() == [2, 2, 1, 1]
    # flat = [1,2, 0,1, 0,3] -> stable argsort
    assert order.tolist() == [2, 4, 0, 3, 1, 5]
    assert slot.tolist() == [2, 4, 0, 3, 1, 5]


def test_router_bwd_matches_autograd_of_the_reference_expression():
    """Router.forward of the reference (moe.py:86-95) typed out in float64 and differentiated by
    torch.autograd: weights, load-balance loss and z-loss, separately and together; a dropped
    term, a wrong sign or a 1/n in the wrong place fails here."""
    g = torch.Generator().manual_seed(77)
    for n, e, k in ((9, 8, 2), (33, 64, 6), (5, 3, 3), (17, 130, 1)):
        logits = torch.round(torch.randn(n, e, generator=g) * 64) / 64
        idx, *_ = O.router(logits, k)
        gw = torch.randn(n, k, generator=g)
        for use_w, ga, gz in ((True, None, None), (False, 0.7, None), (False, None, -1.3), (True, 0.01, 0.001)):
            lf = logits.double().requires_grad_(True)
            probs = lf.softmax(-1)
            w, _ = probs.gather(1, idx), None
            w = w / w.sum(-1, keepdim=True)
            with torch.no_grad():
                frac = torch.bincount(idx.reshape(-1), minlength=e).double() / idx.numel()
            aux = e * (frac * probs.mean(0)).sum()
            z = lf.logsumexp(-1).pow(2).mean()
            total = lf.sum() * 0
            if use_w:
                total = total + (w * gw.double()).sum()
            if ga is not None:
                total = total + ga * aux
            if gz is not None:
                total = total + gz * z
            (want,) = torch.autograd.grad(total, lf)
            got = O.router_bwd(logits, k, gw if use_w else None, ga, gz)
            assert torch.allclose(got, want, rtol=1e-10, atol=1e-12), (n, e, k, use_w, ga, gz)
    # rows of the weight gradient sum to zero (softmax), and a constant gw gives no gradient
    # (the renormalised weights sum to one)
    logits = torch.randn(11, 16, generator=g)
    assert O.router_bwd(logits, 4, torch.randn(11, 4, generator=g)).sum(-1).abs().max() < 1e-12
    assert O.router_bwd(logits, 4, torch.full((11, 4), 3.0)).abs().max() < 1e-12


def test_router_aux_matches_the_reference_expression():
    # forgemind/moe.py:92-95 written out with library calls
    torch.manual_seed(1)
    logits = torch.randn(64, 8)
    idx, *_ = O.router(logits, 2)
    aux, z = O.router_aux(logits, idx)
    probs = logits.softmax(-1)
    c = torch.zeros(8, dtype=torch.int64).scatter_add_(0, idx.reshape(-1), torch.ones(128, dtype=torch.int64))
    assert aux.item() == pytest.approx((8 * ((c / 128) * probs.mean(0)).sum()).item(), rel=1e-6)
    assert z.item() == pytest.approx(logits.logsumexp(-1).pow(2).mean().item(), rel=1e-6)


# ------------------------------------------------------------------ gather / combine
def test_moe_gather_combine_brute_force():
    g = torch.Generator().manual_seed(9)
    n, k, e, d = 7, 2, 4, 5
    x = torch.randn(n, d, generator=g)
    idx, w, counts, slot, order = O.router(torch.randn(n, e, generator=g), k)
    xs = O.moe_gather(x, order, k)
    flat = idx.reshape(-1)
    for s in range(n * k):                       # grouped position s holds the token of assignment order[s]
        assert torch.equal(xs[s], x[order[s] // k])
        assert flat[order[s]] == torch.sort(flat).values[s]
    ys = torch.randn(n * k, d, generator=g)
    out = O.moe_combine(ys, w, order, k, n)
    for t in range(n):
        want = sum(w[t, j] * ys[slot[t * k + j]] for j in range(k))
        assert torch.allclose(out[t], want, atol=1e-6)
    # unit weights after a gather return k copies of every token
    assert torch.allclose(O.moe_combine(xs, torch.ones(n, k), order, k, n), k * x, atol=1e-6)

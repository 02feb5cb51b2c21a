"""Committed vectors (tests/golden/hotpath_vectors.npz): the oracle must keep reproducing them on
CPU, and the HIP kernels must match them on a GPU, without either side seeing the other."""

import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_vectors.npz")


@pytest.fixture(scope="module")
def gv():
    return np.load(PATH, allow_pickle=False)


def bf(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_oracle_reproduces_the_vectors(gv):
    x, dl, w = bf(gv["norm_x"]), bf(gv["norm_delta"]), torch.from_numpy(gv["norm_w"])
    dy, gxn = bf(gv["norm_dy"]), bf(gv["norm_gxn"])
    y, rstd = O.rms_norm(x, w, 1e-6)
    dx, dw = O.rms_norm_bwd(x, w, dy, 1e-6)
    assert torch.equal(y, bf(gv["norm_y"])) and torch.equal(dx, bf(gv["norm_dx"]))
    assert np.allclose(dw.numpy(), gv["norm_dw"], rtol=1e-6) and np.allclose(rstd.numpy(), gv["norm_rstd"], rtol=1e-6)
    xn, y2, _ = O.add_rms_norm(x, dl, w, 1e-5)
    dx2, dw2 = O.add_rms_norm_bwd(xn, w, dy, gxn, 1e-5)
    assert torch.equal(xn, bf(gv["add_xn"])) and torch.equal(y2, bf(gv["add_y"])) and torch.equal(dx2, bf(gv["add_dx"]))
    loss, _ = O.cross_entropy(bf(gv["ce_logits"]), torch.from_numpy(gv["ce_labels"]), acc=torch.float64)
    assert loss.item() == pytest.approx(float(gv["ce_loss"]), rel=1e-12)
    kl, _ = O.kl_div(bf(gv["kl_s"]), bf(gv["kl_t"]), "mean", 2.0, acc=torch.float64)
    assert kl.item() == pytest.approx(float(gv["kl_loss"]), rel=1e-12)
    assert np.array_equal(O.topk(bf(gv["topk_x"]), 64)[1].numpy(), gv["topk_idx"])
    assert np.array_equal(O.topk(torch.from_numpy(gv["topk_kat_tie"]), 3)[1].numpy(), gv["topk_kat_tie_idx"])
    assert np.array_equal(O.topk(torch.from_numpy(gv["topk_kat_nan"]), 3)[1].numpy(), gv["topk_kat_nan_idx"])
    ri, rw, rc, rs, ro = O.router(torch.from_numpy(gv["route_logits"]), 2)
    assert np.array_equal(ri.numpy(), gv["route_idx"]) and np.array_equal(ro.numpy(), gv["route_order"])
    assert np.array_equal(rs.numpy(), gv["route_slot"]) and np.array_equal(rc.numpy(), gv["route_counts"])
    rg = O.router_bwd(torch.from_numpy(gv["route_logits"]), 2, torch.from_numpy(gv["route_gw"]), 0.01, 0.001)
    assert np.allclose(rg.numpy(), gv["route_grad"], rtol=1e-12, atol=1e-15)


@pytest.mark.gpu
def test_kernels_match_the_vectors(gv):
    from forgeminds_amd.kernels import _hip
    dev = "cuda:0"

    def close(got, want_bits, ulps=3):
        a, b = got.float().cpu(), bf(want_bits).float()
        return bool(((a - b).abs() <= ulps * 2.0 ** -8 * b.abs() + 1e-6 * b.abs().max()).all())

    x, dl, w = bf(gv["norm_x"]).to(dev), bf(gv["norm_delta"]).to(dev), torch.from_numpy(gv["norm_w"]).to(dev)
    dy, gxn = bf(gv["norm_dy"]).to(dev), bf(gv["norm_gxn"]).to(dev)
    y, rstd = _hip.rmsnorm_fwd(x, w, 1e-6)
    dx, dw = _hip.rmsnorm_bwd(x, w, rstd, dy)
    assert close(y, gv["norm_y"]) and close(dx, gv["norm_dx"])
    assert np.allclose(dw.cpu().numpy(), gv["norm_dw"], rtol=1e-4, atol=1e-4)
    xn, y2, rstd2 = _hip.add_rmsnorm_fwd(x, dl, w, 1e-5)
    dx2, dw2 = _hip.add_rmsnorm_bwd(xn, w, rstd2, dy, gxn)
    assert torch.equal(xn.cpu(), bf(gv["add_xn"])) and close(y2, gv["add_y"]) and close(dx2, gv["add_dx"])
    assert np.allclose(dw2.cpu().numpy(), gv["add_dw"], rtol=1e-4, atol=1e-4)
    lg, lab = bf(gv["ce_logits"]).to(dev), torch.from_numpy(gv["ce_labels"]).to(dev)
    loss, lse, nv, _ = _hip.ce_fwd(lg, lab, -100, "mean")
    assert loss.item() == pytest.approx(float(gv["ce_loss"]), rel=1e-4)
    assert close(_hip.ce_bwd(lg, lab, lse, nv, None, -100), gv["ce_grad"])
    s, t = bf(gv["kl_s"]).to(dev), bf(gv["kl_t"]).to(dev)
    kl, rows, ls, lt = _hip.kl_fwd(s, t, 0.5, "mean")
    assert kl.item() == pytest.approx(float(gv["kl_loss"]), rel=1e-4)
    assert np.allclose(rows.cpu().numpy(), gv["kl_rows"], rtol=2e-4, atol=1e-6)
    g = _hip.kl_bwd(s, t, ls, lt, None, False, torch.bfloat16, 0.5, 1.0 / 6)
    a, b = g.float().cpu(), bf(gv["kl_grad"]).float()
    assert ((a - b).abs() <= 3 * 2.0 ** -8 * b.abs() + 1e-6).all()
    assert np.array_equal(_hip.topk(bf(gv["topk_x"]).to(dev), 64, torch.int32)[1].cpu().numpy(), gv["topk_idx"])
    for name in ("tie", "nan"):
        got = _hip.topk(torch.from_numpy(gv[f"topk_kat_{name}"]).to(dev), 3, torch.int32)[1].cpu().numpy()
        assert np.array_equal(got, gv[f"topk_kat_{name}_idx"])
    idx, wts, counts, slot, order = _hip.route(torch.from_numpy(gv["route_logits"]).to(dev), 2)
    assert np.array_equal(idx.cpu().numpy(), gv["route_idx"]) and np.array_equal(counts.cpu().numpy(), gv["route_counts"])
    assert np.array_equal(slot.cpu().numpy(), gv["route_slot"]) and np.array_equal(order.cpu().numpy(), gv["route_order"])
    assert np.allclose(wts.cpu().numpy(), gv["route_w"], rtol=1e-5)
    rg = _hip.route_bwd(torch.from_numpy(gv["route_logits"]).to(dev), idx, torch.from_numpy(gv["route_gw"]).to(dev),
                        counts, torch.tensor(0.01, device=dev), torch.tensor(0.001, device=dev))
    assert np.abs(rg.cpu().numpy() - gv["route_grad"]).max() <= 2e-5 * np.abs(gv["route_grad"]).max() + 1e-9

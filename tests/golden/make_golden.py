"""Writes tests/golden/hotpath_vectors.npz: small seeded inputs and the oracle's outputs.

    python tests/golden/make_golden.py

The expected values come from oracle/oracle.py (pinned by tests/test_oracle.py), not from the
reference's code; the known-answer vectors of the reference's own tests (top-k ties and NaNs,
tests/test_topk.py:68-85 there) are included as data. bf16 tensors are stored as their uint16
bit patterns. Re-running this script must reproduce the file bit for bit.
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hotpath_vectors.npz")


def bits(t):
    return t.view(torch.int16).numpy().view(np.uint16) if t.dtype == torch.bfloat16 else t.numpy()


def main():
    g = torch.Generator().manual_seed(20240)
    d = {}
    # RMSNorm / add-RMSNorm, bf16 activations, fp32 weight
    x = torch.randn(12, 256, generator=g).bfloat16()
    dl = torch.randn(12, 256, generator=g).bfloat16()
    w = 1 + 0.02 * torch.randn(256, generator=g)
    dy = torch.randn(12, 256, generator=g).bfloat16()
    gxn = torch.randn(12, 256, generator=g).bfloat16()
    y, rstd = O.rms_norm(x, w, 1e-6)
    dx, dw = O.rms_norm_bwd(x, w, dy, 1e-6)
    xn, y2, rstd2 = O.add_rms_norm(x, dl, w, 1e-5)
    dx2, dw2 = O.add_rms_norm_bwd(xn, w, dy, gxn, 1e-5)
    d.update(norm_x=bits(x), norm_delta=bits(dl), norm_w=w.numpy(), norm_dy=bits(dy), norm_gxn=bits(gxn),
             norm_y=bits(y), norm_rstd=rstd.numpy(), norm_dx=bits(dx), norm_dw=dw.numpy(),
             add_xn=bits(xn), add_y=bits(y2), add_rstd=rstd2.numpy(), add_dx=bits(dx2), add_dw=dw2.numpy())
    # cross entropy, bf16 logits, some ignored labels
    lg = (2 * torch.randn(10, 1000, generator=g)).bfloat16()
    lab = torch.randint(0, 1000, (10,), generator=g)
    lab[[1, 7]] = -100
    loss, grad = O.cross_entropy(lg, lab, acc=torch.float64)
    _, grad32 = O.cross_entropy(lg, lab)
    d.update(ce_logits=bits(lg), ce_labels=lab.numpy(), ce_loss=np.float64(loss.item()), ce_grad=bits(grad32))
    # KL, temperature 2
    s = (3 * torch.randn(6, 777, generator=g)).bfloat16()
    t = (s.float() + 0.5 * torch.randn(6, 777, generator=g)).bfloat16()
    kl, _ = O.kl_div(s, t, "mean", 2.0, acc=torch.float64)
    rows, _ = O.kl_div(s, t, "none", 2.0, acc=torch.float64)
    _, kgrad = O.kl_div(s, t, "mean", 2.0)
    d.update(kl_s=bits(s), kl_t=bits(t), kl_loss=np.float64(kl.item()), kl_rows=rows.numpy(), kl_grad=bits(kgrad))
    # top-k: heavy ties (coarse grid), plus the reference's two known-answer rows
    xt = (torch.round(torch.randn(5, 3000, generator=g) * 4) / 4).bfloat16()
    _, ti = O.topk(xt, 64)
    d.update(topk_x=bits(xt), topk_idx=ti.numpy().astype(np.int32),
             topk_kat_tie=np.array([[1.0, 3.0, 3.0, 2.0, 3.0]], np.float32), topk_kat_tie_idx=np.array([[1, 2, 4]], np.int32),
             topk_kat_nan=np.array([[np.nan, 1.0, 2.0, np.nan, 0.0]], np.float32), topk_kat_nan_idx=np.array([[0, 3, 2]], np.int32))
    # router: 2**-12 grid and forced ties
    lr = torch.round(torch.randn(300, 64, generator=g) * 4096) / 4096
    lr[::50, 3] = lr[::50].max(-1).values
    lr[::50, 40] = lr[::50, 3]
    ri, rw, rc, rs, ro = O.router(lr, 2)
    d.update(route_logits=lr.numpy(), route_idx=ri.numpy().astype(np.int32), route_w=rw.numpy(),
             route_counts=rc.numpy().astype(np.int32), route_slot=rs.numpy().astype(np.int32),
             route_order=ro.numpy().astype(np.int32))
    # the router's gradient: through the weights, the load-balance loss and the z-loss
    gw = torch.randn(300, 2, generator=g)
    d.update(route_gw=gw.numpy(), route_grad=O.router_bwd(lr, 2, gw, 0.01, 0.001, acc=torch.float64).numpy())
    np.savez_compressed(OUT, **d)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(d), "arrays")


if __name__ == "__main__":
    main()

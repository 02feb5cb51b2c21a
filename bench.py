#!/usr/bin/env python3
"""Benchmark of the packed-kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extras] [--no-cpu]

NAME: ce (headline), ce_one_pass, rmsnorm, add_rmsnorm, add_layernorm, kl, kl_one_launch, kl_topk, kl_topk_one_launch, topk,
route, route_256x8, route_train, moe_dispatch, swiglu, qk_norm_rope.

A step is one pass of the hot path (forward + backward) over one batch of synthetic,
seeded input that is already resident in HBM, launched straight through the C ABI of
libfmhip.so with pre-allocated outputs (no allocator, no autograd in the timed region).
The headline workload is the fused cross entropy of the reference's loss path at
logits bf16 [8192, 32000]; `value` is algorithmic bytes per step / time per step.

Prints ONE JSON line of a few KB (numbers only; `--detail PATH` writes the long form with the
descriptions, warm-cache, graph-replay, torch-eager and CPU columns to a file). The line carries
  checked       one step's output compared with the CPU oracle on a bounded row sample before
                anything is timed (per workload too);
  roofline      the dominant kernel of the headline workload against the 8 TB/s HBM peak, timed
                with HIP events around that kernel's launches (each behind the forward that precedes
                it in every step, as in the timed region), on the bytes it has to move;
                `traffic` = that kernel's HBM bytes from the committed profiler counter runs,
                looked up by the name of the kernel that actually ran (null when unknown);
                `configs` = one row per BASELINE configuration (cfg1 RMSNorm, cfg2 CE, cfg3 router,
                cfg4 add-RMSNorm, cfg5 KL, cfg5b top-k): ms per step, fraction of the 8 TB/s peak
                on the algorithmic bytes, rows/s, the dominant kernel with its average and minimum
                launch time, and `floor_ms` = the best bare sweep (fm_stream_probe_mix: same
                buffers, same read / write mix per launch, no arithmetic), `of_floor` = floor / ms;
  cpu_baseline  the CPU oracle (the reference's torch expression) on the host's cores -- a
                reported baseline, never a target;
  workloads     ms / GB/s / fraction for the other shapes of the hot path;
  kbench        the reference's own protocol (public API, clones + autograd timed), ms per op.

Inputs follow one recipe: torch.Generator(device="cpu").manual_seed(1000 + config number), values
drawn on the CPU in row chunks, converted to the storage type and moved to the GPU.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X HBM3E, published
METRIC = "HBM GB/s & % roofline: RMSNorm, CE/KL fwd+bwd; MoE top-k rows/s"

# HBM traffic per launch, keyed by the kernel's full name as fm_last_kernel() reports it:
# (FETCH_SIZE KiB, WRITE_SIZE KiB) per dispatch from two `rocprofv3 --pmc` runs of this file
# (profiles/all_workloads_hbm_traffic_pmc.txt). Each counter is scaled by what it reads for the
# library's own 1 GiB copy (probe_copy_kernel, `bench.py --copy-probe 1024` under the same counters).
# A kernel that is not in the table (a retune changed its template arguments) reports null.
TRAFFIC_SCALE = (1048576.0 / 524299.5, 1048576.0 / 1049433.3)
TRAFFIC_KIB = {
    "ce_bwd_kernel<bf16_t, 1024, 4>": (244221.5, 512256.4),
    "ce_fwd_kernel<bf16_t, 512, 4, false>": (125276.5, 250.2),
    "ce_fwd_kernel<bf16_t, 512, 4, true>": (131369.4, 266.4),
    "ce_loss_grad_held_kernel<bf16_t>": (487092.0, 1028560.3),
    "ce_loss_grad_kernel<bf16_t, 512, 8>": (243962.6, 512526.3),
    "colsum16_kernel<bf16_t>": (4111.0, 8.0),
    "colsum16_kernel<float>": (1039.0, 4.0),
    "colsum_kernel<float>": (8208.0, 64.0),
    "combine_kernel<bf16_t, true, 8>": (133142.6, 131072.0),
    "kl_bwd_kernel<bf16_t, bf16_t, 1024, 8>": (1026898.0, 1026058.2),
    "kl_fwd_kernel<bf16_t, 512, 4>": (1026880.6, 385.0),
    "kl_fwd_topk_kernel<bf16_t, 512, 2, false>": (1054177.5, 2433.6),
    "kl_fwd_topk_kernel<bf16_t, 512, 2, true>": (2057727.9, 1028505.4),
    "kl_loss_grad_held_kernel<bf16_t, bf16_t, 512, 22, 9>": (1026391.4, 1026433.1),
    "norm_bwd_kernel<bf16_t, bf16_t, 256, 2, false, true>": (65831.7, 69632.3),
    "norm_bwd_kernel<bf16_t, float, 512, 2, false, true>": (393631.7, 270336.0),
    "norm_bwd_kernel<bf16_t, float, 512, 2, true, true>": (393894.8, 278528.0),
    "norm_bwd_kernel<bf16_t, float, 64, 2, false, true>": (16461.6, 17409.4),
    "norm_fwd_kernel<bf16_t, bf16_t, 256, 2, false, false, true>": (32821.0, 65842.9),
    "norm_fwd_kernel<bf16_t, bf16_t, 256, 2, true, false, false>": (65592.6, 131367.7),
    "norm_fwd_kernel<bf16_t, float, 512, 2, true, false, false>": (262296.8, 524857.6),
    "norm_fwd_kernel<bf16_t, float, 512, 2, true, true, false>": (262429.8, 525351.4),
    "norm_fwd_kernel<bf16_t, float, 64, 2, false, false, true>": (8227.1, 16427.0),
    "permute_kernel": (1585.1, 10651.3),
    "probe_read_kernel": (524298.8, 0.0),
    "rope_vec_kernel<bf16_t, float, 8, false, 2>": (105921.2, 213461.3),
    "rope_vec_kernel<bf16_t, float, 8, true, 2>": (216510.7, 214218.1),
    "route_bwd_kernel<float, 8, true>": (2221.5, 4096.0),
    "route_group_kernel<float, 32, true, 2, 8>": (32845.1, 6179.1),
    "route_group_kernel<float, 8, true, 0, 8>": (2106.0, 328.5),
    "route_scan_stats_kernel": (1893.5, 1026.0),
    "scatter_kernel<bf16_t, true, 8>": (66084.3, 262270.8),
    "softmax_bwd_rows_kernel<bf16_t, 16, 1>": (2061.5, 2048.0),
    "softmax_bwd_rows_kernel<bf16_t, 256, 2>": (65553.0, 65550.5),
    "softmax_rows_kernel<bf16_t, 16, 1>": (1039.6, 2048.0),
    "softmax_rows_kernel<bf16_t, 256, 2>": (32788.6, 65609.7),
    "swiglu_bwd_kernel<bf16_t, true>": (264214.2, 352258.0),
    "swiglu_fwd_kernel<bf16_t, true>": (176147.3, 176128.0),
    "swiglu_split_kernel<bf16_t, true, false>": (458770.2, 458752.1),
    "swiglu_split_kernel<bf16_t, true, true>": (688148.5, 917505.8),
    "topk_lds_kernel<bf16_t, 512, 4, 0>": (539853.8, 1024.0),
}
TRAFFIC_SOURCE = "profiles/all_workloads_hbm_traffic_pmc.txt"


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` from the committed counter runs, or None."""
    kib = TRAFFIC_KIB.get(kernel)
    if kib is None:
        return None
    return int(round((kib[0] * TRAFFIC_SCALE[0] + kib[1] * TRAFFIC_SCALE[1]) * 1024))


WORKLOADS = ["ce", "ce_one_pass", "ce_one_pass_128k", "rmsnorm", "add_rmsnorm", "add_layernorm", "kl", "kl_one_launch", "kl_topk",
             "kl_topk_one_launch", "topk", "route", "route_256x8", "route_train", "moe_dispatch", "swiglu", "qk_norm_rope"]


def parse():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="ce",
                    choices=WORKLOADS)
    ap.add_argument("--no-extras", action="store_true", help="only the headline workload")
    ap.add_argument("--only", default="", metavar="A,B", help="besides the headline, only these workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--detail", default="", metavar="PATH",
                    help="also write the long form (descriptions, warm / graph / eager / CPU columns) here")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="only run a plain device copy of this many MiB (counter calibration)")
    return ap.parse_args()


# ---------------------------------------------------------------------------- workloads
class Workload:
    """Pre-allocated tensors plus closures that enqueue the launches of one step."""

    name = ""
    desc = ""
    unit = "GB/s"
    dominant = ""          # kernel the roofline object is about

    def step(self):        # forward + backward of the hot path
        raise NotImplementedError

    def dominant_launch(self):
        raise NotImplementedError


def _check(rc, what):
    if rc != 0:
        from forgeminds_amd.kernels import _hip
        raise RuntimeError(f"{what}: status {rc}: {_hip.lib().fm_last_error().decode()}")


_SHARED = {}        # big inputs that several workloads use (the KL pair): drawn once


def make_workload(name, torch, L, dev):
    from forgeminds_amd.kernels import _hip
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device="cpu")
    BF, F32c = _hip.BF16, _hip.F32
    w = Workload()
    w.name = name

    def rn(*shape, scale=1.0, dtype=torch.bfloat16, base=None):
        """scale * N(0,1) (+ base, added in fp32) drawn from the CPU generator in row chunks,
        rounded once to `dtype`, resident on the GPU."""
        out = torch.empty(*shape, device=dev, dtype=dtype)
        flat = out.view(shape[0], -1) if len(shape) > 1 else out.view(1, -1)
        rows, width = flat.shape
        step = max(1, (1 << 25) // max(1, width))
        for r0 in range(0, rows, step):
            r1 = min(rows, r0 + step)
            c = torch.randn(r1 - r0, width, generator=g)
            if scale != 1.0:
                c.mul_(scale)
            if base is None:
                flat[r0:r1] = c.to(dtype)
            else:
                bf = base.view(rows, width)[r0:r1].float()
                flat[r0:r1] = (bf + c.to(dev)).to(dtype)
        return out

    if name == "rmsnorm":
        n, d = 8192, 1024
        g.manual_seed(1001)
        sets = 8     # rotate through > 256 MB so the Infinity Cache cannot serve a step
        xs = [rn(n, d) for _ in range(sets)]
        dys = [rn(n, d) for _ in range(sets)]
        ys = [torch.empty_like(xs[0]) for _ in range(sets)]
        dxs = [torch.empty_like(xs[0]) for _ in range(sets)]
        wt = 1 + 0.02 * rn(d, dtype=torch.float32)
        rstd = torch.empty(n, device=dev)
        dw = torch.empty_like(wt)
        nb = L.fm_rmsnorm_bwd_workspace(n, d, BF)
        ws = torch.empty(nb, device=dev, dtype=torch.uint8)
        state = {"i": 0}

        def fwd(i):
            _check(L.fm_rmsnorm_fwd(xs[i].data_ptr(), wt.data_ptr(), ys[i].data_ptr(), rstd.data_ptr(),
                                    n, d, BF, F32c, 1e-6, st), "fm_rmsnorm_fwd")

        def bwd(i):
            _check(L.fm_rmsnorm_bwd(xs[i].data_ptr(), wt.data_ptr(), rstd.data_ptr(), dys[i].data_ptr(),
                                    dxs[i].data_ptr(), dw.data_ptr(), ws.data_ptr(), nb, n, d, BF, F32c,
                                    st), "fm_rmsnorm_bwd")

        def step():
            i = state["i"] = (state["i"] + 1) % sets
            fwd(i)
            bwd(i)

        def warm_step():
            fwd(0)
            bwd(0)

        def check():
            from oracle import oracle as O
            step()
            torch.cuda.synchronize()
            i = state["i"]
            xc, dyc, wc = xs[i].cpu(), dys[i].cpu(), wt.cpu()
            oy, _ = O.rms_norm(xc, wc, 1e-6)
            odx, odw = O.rms_norm_bwd(xc, wc, dyc, 1e-6)
            return _close(ys[i], oy) and _close(dxs[i], odx) and _close(dw, odw)

        def cpu():
            from oracle import oracle as O
            xc, dyc, wc = xs[0].cpu(), dys[0].cpu(), wt.cpu()
            return (lambda: (O.rms_norm(xc, wc, 1e-6), O.rms_norm_bwd(xc, wc, dyc, 1e-6))), 1.0, f"all {n} rows"

        def eager():
            from forgeminds_amd.kernels import _fallback as fb
            x_, w_ = xs[0].detach().requires_grad_(True), wt.detach().requires_grad_(True)
            fb.rms_norm(x_, w_, 1e-6).backward(dys[0])

        w.check, w.cpu, w.eager = check, cpu, eager
        w.graph_steps = [(lambda i=i: (fwd(i), bwd(i))) for i in range(sets)]
        w.step, w.warm_step = step, warm_step
        def next_forward():       # the step's own order: the next buffer set, forward, then the backward timed
            state["i"] = (state["i"] + 1) % sets
            fwd(state["i"])

        w.dominant_launch, w.dominant_before = (lambda: bwd(state["i"])), next_forward
        w.dominant = "norm_bwd_kernel<bf16,f32,64,2> + colsum_kernel"
        w.dominant_bytes = n * d * 6
        w.bytes = n * d * 10
        w.desc = f"RMSNorm fwd+bwd x bf16 [{n},{d}], w fp32, eps 1e-6 (rotating {sets} buffer sets)"
        w.rows = n
        w.sets = sets
        w.floor = [lambda i: ((xs[i],), (ys[i],)), lambda i: ((xs[i], dys[i]), (dxs[i],))]
        return w

    if name == "add_rmsnorm":
        n, d = 16384, 8192
        g.manual_seed(1004)
        x, dl, gy, gxn = rn(n, d), rn(n, d), rn(n, d), rn(n, d)
        wt = 1 + 0.02 * rn(d, dtype=torch.float32)
        xn, y, dx = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
        rstd = torch.empty(n, device=dev)
        dw = torch.empty_like(wt)
        nb = L.fm_rmsnorm_bwd_workspace(n, d, BF)
        ws = torch.empty(nb, device=dev, dtype=torch.uint8)

        def fwd():
            _check(L.fm_add_rmsnorm_fwd(x.data_ptr(), dl.data_ptr(), wt.data_ptr(), xn.data_ptr(),
                                        y.data_ptr(), rstd.data_ptr(), n, d, BF, F32c, 1e-5, st),
                   "fm_add_rmsnorm_fwd")

        def bwd():
            _check(L.fm_add_rmsnorm_bwd(xn.data_ptr(), wt.data_ptr(), rstd.data_ptr(), gy.data_ptr(),
                                        gxn.data_ptr(), dx.data_ptr(), None, dw.data_ptr(), ws.data_ptr(),
                                        nb, n, d, BF, F32c, st), "fm_add_rmsnorm_bwd")

        def step():
            fwd()
            bwd()

        def check(rows=64):
            from oracle import oracle as O
            step()
            torch.cuda.synchronize()
            xc, dc, wc = x[:rows].cpu(), dl[:rows].cpu(), wt.cpu()
            oxn, oy, _ = O.add_rms_norm(xc, dc, wc, 1e-5)
            odx, _ = O.add_rms_norm_bwd(oxn, wc, gy[:rows].cpu(), gxn[:rows].cpu(), 1e-5)
            return bool(torch.equal(xn[:rows].cpu(), oxn)) and _close(y[:rows], oy) and _close(dx[:rows], odx)

        def cpu(rows=2048):
            from oracle import oracle as O
            xc, dc, wc, gyc, gxc = x[:rows].cpu(), dl[:rows].cpu(), wt.cpu(), gy[:rows].cpu(), gxn[:rows].cpu()

            def run():
                oxn, _, _ = O.add_rms_norm(xc, dc, wc, 1e-5)
                O.add_rms_norm_bwd(oxn, wc, gyc, gxc, 1e-5)
            return run, n / rows, f"{rows} of {n} rows, time scaled by {n // rows}"

        def eager():
            from forgeminds_amd.kernels import _fallback as fb
            x_, d_, w_ = (t.detach().requires_grad_(True) for t in (x, dl, wt))
            oxn, oy = fb.add_rms_norm(x_, d_, w_, 1e-5)
            torch.autograd.backward([oxn, oy], [gxn, gy])

        w.check, w.cpu, w.eager = check, cpu, eager
        w.step = step
        w.dominant_launch, w.dominant_before = bwd, fwd
        w.dominant = "norm_bwd_kernel<bf16,f32,512,2> + colsum_kernel"
        w.dominant_bytes = n * d * 8
        w.bytes = n * d * 16
        w.desc = f"add-RMSNorm fwd+bwd x,delta bf16 [{n},{d}], w fp32, eps 1e-5, with residual grad"
        w.rows = n
        w.floor = [lambda i: ((x, dl), (xn, y)), lambda i: ((xn, gy, gxn), (dx,))]
        return w

    if name == "add_layernorm":
        n, d = 16384, 8192
        g.manual_seed(1034)
        x, dl, gy, gxn = rn(n, d), rn(n, d), rn(n, d), rn(n, d)
        wt = 1 + 0.02 * rn(d, dtype=torch.float32)
        bs = 0.1 * rn(d, dtype=torch.float32)
        xn, y, dx = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
        mean, rstd = torch.empty(n, device=dev), torch.empty(n, device=dev)
        dw, db = torch.empty_like(wt), torch.empty_like(wt)
        nb = L.fm_layernorm_bwd_workspace(n, d, BF)
        ws = torch.empty(nb, device=dev, dtype=torch.uint8)

        def fwd():
            _check(L.fm_add_layernorm_fwd(x.data_ptr(), dl.data_ptr(), wt.data_ptr(), bs.data_ptr(),
                                          xn.data_ptr(), y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), n, d,
                                          BF, F32c, 1e-5, st), "fm_add_layernorm_fwd")

        def bwd():
            _check(L.fm_layernorm_bwd(xn.data_ptr(), wt.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                                      gy.data_ptr(), gxn.data_ptr(), dx.data_ptr(), dw.data_ptr(), db.data_ptr(),
                                      ws.data_ptr(), nb, n, d, BF, F32c, st), "fm_layernorm_bwd")

        def step():
            fwd()
            bwd()

        def check(rows=64):
            from oracle import oracle as O
            step()
            torch.cuda.synchronize()
            wc, bc = wt.cpu(), bs.cpu()
            oxn, oy, _, _ = O.add_layer_norm(x[:rows].cpu(), dl[:rows].cpu(), wc, bc, 1e-5)
            odx, _, _ = O.layer_norm_bwd(oxn, wc, gy[:rows].cpu(), 1e-5, gxn=gxn[:rows].cpu())
            return bool(torch.equal(xn[:rows].cpu(), oxn)) and _close(y[:rows], oy) and _close(dx[:rows], odx)

        w.check = check
        w.step = step
        w.dominant_launch, w.dominant_before = bwd, fwd
        w.floor = [lambda i: ((x, dl), (xn, y)), lambda i: ((xn, gy, gxn), (dx,))]
        w.dominant = "norm_bwd_kernel<bf16,f32,512,2,LN> + colsum_kernel"
        w.dominant_bytes = n * d * 8
        w.bytes = n * d * 16
        w.desc = f"add-LayerNorm fwd+bwd x,delta bf16 [{n},{d}], w,b fp32, eps 1e-5, with residual grad"
        w.rows = n
        return w

    if name in ("ce", "ce_one_pass", "ce_one_pass_128k"):
        wide = name == "ce_one_pass_128k"    # the vocabulary of config 5: rows of 250 KB, kept on the chip
        n, v = (4096, 128256) if wide else (8192, 32000)
        g.manual_seed(1002)
        if wide:
            if "kl_st" not in _SHARED:       # the student logits of the KL workloads serve
                g.manual_seed(1005)
                s_ = rn(n, v, scale=3.0)
                _SHARED["kl_st"] = (s_, rn(n, v, scale=0.5, base=s_))
            lg = _SHARED["kl_st"][0]
            g.manual_seed(1002)
        else:
            lg = rn(n, v, scale=2.0)
        loss_rows = 256 if wide else 2048
        y = torch.randint(0, v, (n,), generator=g)
        y[torch.rand(n, generator=g) < 0.05] = -100
        y = y.to(dev)
        lse, rl = torch.empty(n, device=dev), torch.empty(n, device=dev)
        sc = torch.empty(2, device=dev)
        dlg = torch.empty_like(lg)

        def fwd():
            _check(L.fm_ce_fwd(lg.data_ptr(), y.data_ptr(), lse.data_ptr(), rl.data_ptr(), sc.data_ptr(),
                               sc.data_ptr() + 4, n, v, BF, -100, 2, st), "fm_ce_fwd")

        def bwd():
            _check(L.fm_ce_bwd(lg.data_ptr(), y.data_ptr(), lse.data_ptr(), sc.data_ptr() + 4, None,
                               dlg.data_ptr(), n, v, BF, -100, st), "fm_ce_bwd")

        n_valid = int((y != -100).sum().item())

        def check(rows=64):
            from oracle import oracle as O
            w.step()
            torch.cuda.synchronize()
            yc = y[:rows].cpu()
            _, og = O.cross_entropy(lg[:rows].cpu(), yc)        # mean over the sample's valid rows
            og = og.float() * (max(1, int((yc != -100).sum())) / max(1, n_valid))
            ol, _ = O.cross_entropy(lg[:loss_rows].cpu(), y[:loss_rows].cpu())   # loss: the first rows against their own row losses
            got = rl[:loss_rows].sum().item() / max(1, int((y[:loss_rows] != -100).sum().item()))
            return _close(dlg[:rows], og) and abs(got - ol.item()) <= 1e-4 * abs(ol.item())

        def cpu():
            from oracle import oracle as O
            rows_ = 512 if wide else n
            lc, yc = lg[:rows_].cpu(), y[:rows_].cpu()
            return (lambda: O.cross_entropy(lc, yc)), n / rows_, (f"{rows_} rows x {n // rows_}" if wide else f"all {n} rows")

        def eager():
            from forgeminds_amd.kernels import _fallback as fb
            l_ = lg.detach().requires_grad_(True)
            fb.cross_entropy(l_, y, -100, "mean").backward()

        w.check, w.cpu, w.eager = check, cpu, eager
        # bytes the dataflow has to move: rows whose label is ignored are never read
        w.valid_rows = n_valid

        if name in ("ce_one_pass", "ce_one_pass_128k"):
            one = torch.ones((), device=dev)

            def both():
                _check(L.fm_ce_loss_grad(lg.data_ptr(), y.data_ptr(), lse.data_ptr(), rl.data_ptr(),
                                         sc.data_ptr(), sc.data_ptr() + 4, dlg.data_ptr(), n, v, BF, -100, 2,
                                         st), "fm_ce_loss_grad")

            def step():
                both()      # forward: loss and gradient from one read of the logits
                _check(L.fm_scale_inplace(dlg.data_ptr(), one.data_ptr(), n * v, BF, st),
                       "fm_scale_inplace")   # backward: upstream gradient 1, nothing to move

            w.step = step
            w.dominant_launch = both
            w.dominant = "ce_loss_grad_held_kernel<bf16>" if wide else "ce_loss_grad_kernel<bf16,512,8>"
            w.dominant_bytes = w.bytes = n * v * 4
            w.required_bytes = w.dominant_required_bytes = n_valid * v * 2 + n * v * 2
            w.desc = (f"fused CE loss + gradient in one pass, logits bf16 [{n},{v}], 5% ignore_index, mean; "
                      "dataflow read + write = 4 B/logit")
            w.rows = n
            w.tensors = (lg, y)
            w.floor = [lambda i: ((lg,), (dlg,))]
            return w

        def step():
            fwd()
            bwd()

        w.step = step
        w.dominant_launch, w.dominant_before = bwd, fwd
        w.dominant = "ce_bwd_kernel<bf16,1024,4>"
        w.dominant_bytes = n * v * 4
        w.bytes = n * v * 6
        w.dominant_required_bytes = n_valid * v * 2 + n * v * 2      # read valid rows, write all rows
        w.required_bytes = 2 * n_valid * v * 2 + n * v * 2           # + the forward's read of the valid rows
        w.desc = (f"fused CE fwd+bwd logits bf16 [{n},{v}], 5% ignore_index, mean; "
                  "dataflow fwd(read) + bwd(read, write) = 6 B/logit")
        w.rows = n
        w.tensors = (lg, y)
        w.floor = [lambda i: ((lg,), ()), lambda i: ((lg,), (dlg,))]
        return w

    if name in ("kl", "kl_one_launch", "kl_topk", "kl_topk_one_launch", "topk"):
        n, v = 4096, 128256
        if "kl_st" not in _SHARED:
            g.manual_seed(1005)
            s_ = rn(n, v, scale=3.0)
            _SHARED["kl_st"] = (s_, rn(n, v, scale=0.5, base=s_))
        s, t = _SHARED["kl_st"]
        if name == "topk":
            idx = torch.empty(n, 64, device=dev, dtype=torch.int32)

            def step():
                _check(L.fm_topk(t.data_ptr(), None, idx.data_ptr(), n, v, 64, BF, 32, st), "fm_topk")

            def check(rows=32):
                from oracle import oracle as O
                step()
                torch.cuda.synchronize()
                return bool(torch.equal(idx[:rows].cpu().long(), O.topk(t[:rows].cpu(), 64)[1]))

            def cpu(rows=256):
                from oracle import oracle as O
                tc = t[:rows].cpu()
                return (lambda: O.topk(tc, 64)), n / rows, f"{rows} of {n} rows, time scaled by {n // rows}"

            w.check, w.cpu = check, cpu
            w.eager = lambda: torch.topk(t, 64)
            w.step = step
            w.dominant_launch = step
            w.dominant = "topk_lds_kernel<bf16,1024,4>"
            w.dominant_bytes = w.bytes = n * v * 2
            w.desc = f"top-64 of teacher logits bf16 [{n},{v}], int32 indices (separate launch)"
            w.rows = n
            w.floor = [lambda i: ((t,), ())]
            return w
        b3 = torch.empty(3, n, device=dev)
        ls = torch.empty((), device=dev)
        gs = torch.empty_like(s)

        def fwd():
            _check(L.fm_kl_fwd(s.data_ptr(), t.data_ptr(), b3[0].data_ptr(), b3[1].data_ptr(),
                               b3[2].data_ptr(), ls.data_ptr(), n, v, BF, 0.5, 2, st), "fm_kl_fwd")

        def bwd():
            _check(L.fm_kl_bwd(s.data_ptr(), t.data_ptr(), b3[0].data_ptr(), b3[1].data_ptr(), None, 0,
                               gs.data_ptr(), n, v, BF, BF, 0.5, 1.0 / n, st), "fm_kl_bwd")

        def check(rows=16):
            from oracle import oracle as O
            w.step()
            torch.cuda.synchronize()
            sc_, tc_ = s[:rows].cpu(), t[:rows].cpu()
            ol, og = O.kl_div(sc_, tc_, "none", 2.0)
            ok = _close(gs[:rows], og.float() / n) and _close(b3[2][:rows], ol)
            if name in ("kl_topk", "kl_topk_one_launch"):
                ok = ok and bool(torch.equal(idx[:rows].cpu().long(), O.topk(tc_, 64)[1]))
            return ok

        def cpu(rows=512):
            from oracle import oracle as O
            sc_, tc_ = s[:rows].cpu(), t[:rows].cpu()
            return (lambda: O.kl_div(sc_, tc_, "mean", 2.0)), n / rows, f"{rows} of {n} rows, time scaled by {n // rows}"

        def eager():
            from forgeminds_amd.kernels import _fallback as fb
            s_ = s.detach().requires_grad_(True)
            fb.kl_div_logits(s_, t, "mean", 2.0).backward()

        w.check = check
        if name == "kl":
            w.cpu, w.eager = cpu, eager

        if name == "kl_one_launch":
            one = torch.ones((), device=dev)

            def both():
                _check(L.fm_kl_loss_grad(s.data_ptr(), t.data_ptr(), b3[0].data_ptr(), b3[1].data_ptr(),
                                         b3[2].data_ptr(), ls.data_ptr(), gs.data_ptr(), n, v, BF, BF, 0.5, 2,
                                         st), "fm_kl_loss_grad")

            def step():
                both()      # forward: loss and gradient, the row pair read once
                _check(L.fm_scale_inplace(gs.data_ptr(), one.data_ptr(), n * v, BF, st),
                       "fm_scale_inplace")   # backward: upstream gradient 1, nothing to move

            w.step = step
            w.dominant_launch = both
            w.dominant = "kl_loss_grad_held_kernel<bf16,bf16,512,22,9>"
            w.dominant_bytes = w.bytes = n * v * 6
            w.desc = (f"KL loss + gradient in one launch bf16 [{n},{v}], T=2, mean; algorithmic 6 B/logit pair "
                      "(read s,t + write g). The pair of rows stays in the registers and LDS of one workgroup per "
                      "compute unit between the two passes (which loads its next row under this row's "
                      "gradient): it is read once, and the L2-side counters show the algorithmic bytes")
            w.rows = n
            w.floor = [lambda i: ((s, t), (gs,))]
            return w

        if name == "kl_topk_one_launch":
            one = torch.ones((), device=dev)
            idx = torch.empty(n, 64, device=dev, dtype=torch.int32)
            pr = torch.empty(n, 64, device=dev)

            def both():
                _check(L.fm_kl_loss_grad_topk(s.data_ptr(), t.data_ptr(), b3[0].data_ptr(), b3[1].data_ptr(),
                                              b3[2].data_ptr(), ls.data_ptr(), gs.data_ptr(), None, idx.data_ptr(),
                                              pr.data_ptr(), n, v, 64, BF, 32, 0.5, 2, st), "fm_kl_loss_grad_topk")

            def step():
                both()
                _check(L.fm_scale_inplace(gs.data_ptr(), one.data_ptr(), n * v, BF, st), "fm_scale_inplace")

            w.step = step
            w.dominant_launch = both
            w.dominant = "kl_fwd_topk_kernel<bf16,512,2>"
            w.dominant_bytes = w.bytes = n * v * 6
            w.desc = (f"KL loss + gradient + teacher top-64 in one launch bf16 [{n},{v}], T=2, mean; algorithmic "
                      "6 B/logit pair; two sweeps per row inside the launch: the L2-side counters show 10 B/pair "
                      "(both sweeps fetched)")
            w.l2_bytes = n * v * 10
            w.rows = n
            return w

        if name == "kl_topk":
            idx = torch.empty(n, 64, device=dev, dtype=torch.int32)
            pr = torch.empty(n, 64, device=dev)

            def fwd():  # noqa: F811 -- the fused forward replaces the plain one
                _check(L.fm_kl_fwd_topk(s.data_ptr(), t.data_ptr(), b3[0].data_ptr(), b3[1].data_ptr(),
                                        b3[2].data_ptr(), ls.data_ptr(), None, idx.data_ptr(),
                                        pr.data_ptr(), n, v, 64, BF, 32, 0.5, 2, st), "fm_kl_fwd_topk")

        def step():
            fwd()
            bwd()

        w.step = step
        w.dominant_launch, w.dominant_before = bwd, fwd
        w.dominant = "kl_bwd_kernel<bf16,bf16,1024,8>"
        w.dominant_bytes = n * v * 6
        w.bytes = n * v * 10
        w.desc = f"KL(teacher||student) fwd+bwd bf16 [{n},{v}], T=2, mean"
        if name == "kl_topk":
            w.desc += "; the forward also returns the teacher's top-64 (int32 indices, fp32 probabilities)"
        w.rows = n
        w.floor = [lambda i: ((s, t), ()), lambda i: ((s, t), (gs,))]
        return w

    if name == "swiglu":
        rows, h = 16384, 14336
        g.manual_seed(1041)
        x = rn(rows, 2 * h)
        dy = rn(rows, h)
        y = torch.empty(rows, h, device=dev, dtype=torch.bfloat16)
        dx = torch.empty_like(x)

        def fwd():
            _check(L.fm_swiglu_split_fwd(x.data_ptr(), y.data_ptr(), rows, h, BF, st), "fm_swiglu_split_fwd")

        def bwd():
            _check(L.fm_swiglu_split_bwd(x.data_ptr(), dy.data_ptr(), dx.data_ptr(), rows, h, BF, st),
                   "fm_swiglu_split_bwd")

        def step():
            fwd()
            bwd()

        def check(r=32):
            from forgeminds_amd.kernels import _fallback as fb
            step()
            torch.cuda.synchronize()
            xc = x[:r].cpu().float().requires_grad_(True)
            ref = fb.swiglu_split(xc)
            ref.backward(dy[:r].cpu().float())
            return _close(y[:r], ref) and _close(dx[:r], xc.grad)

        w.check = check
        w.step = step
        w.dominant_launch = bwd
        w.dominant = "swiglu_split_bwd_kernel<bf16>"
        xa, xb = x.view(-1)[:rows * h], x.view(-1)[rows * h:]      # streams of the size of gate and up
        da, db_ = dx.view(-1)[:rows * h], dx.view(-1)[rows * h:]
        w.floor = [lambda i: ((xa, xb), (y,)), lambda i: ((xa, xb, dy), (da, db_))]
        w.dominant_bytes = rows * h * 2 * 5          # gate, up, dy in; dgate, dup out
        w.bytes = rows * h * 2 * 8                   # + gate, up in; y out
        w.desc = f"SwiGLU on a fused projection fwd+bwd, x bf16 [{rows},{2 * h}] -> y [{rows},{h}]"
        w.rows = rows
        return w

    if name == "qk_norm_rope":
        b, t, hh, d = 8, 4096, 32, 128
        g.manual_seed(1042)
        x = rn(b, t, hh, d)
        do = rn(b, t, hh, d)
        wt = 1 + 0.02 * rn(d, dtype=torch.float32)
        ang = (torch.rand(t, d // 2, generator=g) * 6.28).to(dev)
        cs, sn = torch.cos(ang), torch.sin(ang)
        out, dx = torch.empty_like(x), torch.empty_like(x)
        rstd = torch.empty(b * t * hh, device=dev)
        dw = torch.empty_like(wt)
        nb = L.fm_qk_norm_rope_bwd_workspace(b, t, hh, d)
        ws = torch.empty(max(nb, 16), device=dev, dtype=torch.uint8)

        def fwd():
            _check(L.fm_qk_norm_rope_fwd(x.data_ptr(), wt.data_ptr(), cs.data_ptr(), sn.data_ptr(), out.data_ptr(),
                                         rstd.data_ptr(), b, t, hh, d, BF, F32c, 1e-6, st), "fm_qk_norm_rope_fwd")

        def bwd():
            _check(L.fm_qk_norm_rope_bwd(x.data_ptr(), wt.data_ptr(), cs.data_ptr(), sn.data_ptr(), rstd.data_ptr(),
                                         do.data_ptr(), dx.data_ptr(), dw.data_ptr(), ws.data_ptr(), nb, b, t, hh,
                                         d, BF, F32c, st), "fm_qk_norm_rope_bwd")

        def step():
            fwd()
            bwd()

        def check(tt=16):
            from forgeminds_amd.kernels import _fallback as fb
            step()
            torch.cuda.synchronize()
            xc = x[:1, :tt].cpu().float().requires_grad_(True)
            ref = fb.qk_norm_rope(xc, wt.cpu(), cs[:tt].cpu()[:, None, :], sn[:tt].cpu()[:, None, :], 1e-6)
            ref.backward(do[:1, :tt].cpu().float())
            return _close(out[:1, :tt], ref) and _close(dx[:1, :tt], xc.grad)

        w.check = check
        w.step = step
        w.dominant_launch = bwd
        w.floor = [lambda i: ((x,), (out,)), lambda i: ((x, do), (dx,))]
        w.dominant = "qk_norm_rope_bwd_kernel<bf16,f32>"
        w.dominant_bytes = b * t * hh * d * 2 * 3
        w.bytes = b * t * hh * d * 2 * 5
        w.desc = f"per-head RMSNorm + RoPE fwd+bwd, x bf16 [{b},{t},{hh},{d}], w fp32"
        w.rows = b * t * hh
        return w

    if name in ("route", "route_256x8"):
        big = name == "route_256x8"     # the common MoE shape of today: 256 experts, eight picks, with statistics
        n, e, k = (65536, 256, 8) if big else (16384, 64, 2)
        g.manual_seed(1013 if big else 1003)
        # 80 x 4 MiB (8 x 64 MiB) of logits: a step's input is never in the 256 MB memory-side cache
        sets = 8 if big else 80
        lgs = []
        for i in range(sets):
            lg = torch.round(torch.randn(n, e, generator=g) * 4096) / 4096
            if i == 0:
                # 1 % of the rows get ties at the top and a second group of equal values
                rows = torch.randperm(n, generator=g)[: n // 100]
                cols = torch.stack([torch.randperm(e, generator=g)[:8] for _ in range(rows.numel())])
                top = lg[rows].max(dim=1, keepdim=True).values
                lg[rows[:, None], cols[:, :4]] = top
                lg[rows[:, None], cols[:, 4:]] = lg[rows, cols[:, 4]][:, None]
            lgs.append(lg.to(dev))
        idx = torch.empty(n, k, device=dev, dtype=torch.int32)
        wt = torch.empty(n, k, device=dev)
        cnt = torch.empty(e, device=dev, dtype=torch.int32)
        sl = torch.empty(n * k, device=dev, dtype=torch.int32)
        od = torch.empty(n * k, device=dev, dtype=torch.int32)
        nb = L.fm_route_workspace(n, e, k)
        ws = torch.empty(max(nb, 16), device=dev, dtype=torch.uint8)
        stats = torch.empty(e + 3, device=dev) if big else None
        state = {"i": 0}

        def run(i):
            _check(L.fm_route(lgs[i].data_ptr(), idx.data_ptr(), wt.data_ptr(), cnt.data_ptr(), sl.data_ptr(),
                              od.data_ptr(), None if stats is None else stats.data_ptr(), ws.data_ptr(), nb, n, e, k,
                              F32c, st), "fm_route")

        def step():
            i = state["i"] = (state["i"] + 1) % sets
            run(i)

        def check():
            from oracle import oracle as O
            run(0)                      # the set with the forced ties
            torch.cuda.synchronize()
            oi, ow, oc, oslot, oorder = O.router(lgs[0].cpu(), k)
            return (bool(torch.equal(idx.cpu().long(), oi)) and bool(torch.equal(cnt.cpu().long(), oc))
                    and bool(torch.equal(sl.cpu().long(), oslot)) and bool(torch.equal(od.cpu().long(), oorder))
                    and bool(torch.allclose(wt.cpu(), ow, rtol=1e-5, atol=0)))

        def cpu():
            from oracle import oracle as O
            lc = lgs[0].cpu()
            return (lambda: O.router(lc, k)), 1.0, f"all {n} rows"

        def eager():        # the aten sequence of the reference, moe.py:86-91, 52-60, 232-236
            probs = torch.softmax(lgs[0].float(), dim=-1)
            w_, i_ = torch.topk(probs, k, dim=-1)
            w_ = w_ / w_.sum(dim=-1, keepdim=True)
            flat = i_.reshape(-1)
            torch.zeros(e, dtype=torch.int64, device=dev).scatter_add_(0, flat, torch.ones_like(flat))
            torch.sort(flat, stable=True)

        w.check, w.cpu, w.eager = check, cpu, eager
        w.step = step
        w.warm_step = lambda: run(0)
        w.graph_steps = [(lambda i=i: run(i)) for i in range(sets)]
        w.dominant_launch = step
        w.dominant = "route_group_kernel + permute_kernel"
        w.dominant_bytes = w.bytes = n * (e * 4 + k * 4 * 4)
        w.desc = (f"router softmax + top-{k} + counts + stable permutation" + (" + statistics and auxiliary losses" if big else "")
                  + f", logits fp32 [{n},{e}], 1% tie rows (rotating {sets} logit sets: cold)")
        w.unit = "rows/s"
        w.rows = n
        w.sets = sets
        w.floor = [lambda i: ((lgs[i],), ()), lambda i: ((idx.view(-1),), (sl,))]
        return w

    if name == "route_train":
        # what a training step runs around the router: routing with the statistics and the two
        # auxiliary losses, then the gradient wrt the logits in one kernel
        n, e, k = 16384, 64, 2
        g.manual_seed(1003)
        lg = (torch.round(torch.randn(n, e, generator=g) * 4096) / 4096).to(dev)
        idx = torch.empty(n, k, device=dev, dtype=torch.int32)
        wt = torch.empty(n, k, device=dev)
        cnt = torch.empty(e, device=dev, dtype=torch.int32)
        sl = torch.empty(n * k, device=dev, dtype=torch.int32)
        od = torch.empty(n * k, device=dev, dtype=torch.int32)
        stats = torch.empty(e + 3, device=dev)
        gw = torch.randn(n, k, generator=g).to(dev)
        ga, gz = torch.tensor(0.01, device=dev), torch.tensor(0.001, device=dev)
        dl = torch.empty_like(lg)
        nb = L.fm_route_workspace(n, e, k)
        ws = torch.empty(max(nb, 16), device=dev, dtype=torch.uint8)

        def bwd():
            _check(L.fm_route_bwd(lg.data_ptr(), idx.data_ptr(), gw.data_ptr(), cnt.data_ptr(), ga.data_ptr(),
                                  gz.data_ptr(), dl.data_ptr(), n, e, k, F32c, st), "fm_route_bwd")

        def step():
            _check(L.fm_route(lg.data_ptr(), idx.data_ptr(), wt.data_ptr(), cnt.data_ptr(), sl.data_ptr(),
                              od.data_ptr(), stats.data_ptr(), ws.data_ptr(), nb, n, e, k, F32c, st), "fm_route")
            bwd()

        def check():
            from oracle import oracle as O
            step()
            torch.cuda.synchronize()
            lc = lg.cpu()
            oi, ow, oc, oslot, oorder = O.router(lc, k)
            ref = O.router_bwd(lc, k, gw.cpu(), float(ga), float(gz))
            return (bool(torch.equal(idx.cpu().long(), oi)) and bool(torch.equal(od.cpu().long(), oorder))
                    and _close(dl, ref, rel=1e-4))

        w.check = check
        w.graph_steps = [step] * 8
        w.step = step
        w.dominant_launch = bwd
        w.dominant = "route_bwd_kernel<f32,8>"
        w.dominant_bytes = n * e * 4 * 2
        w.bytes = n * (e * 4 + k * 4 * 4) + w.dominant_bytes
        w.desc = (f"router with statistics and auxiliary losses + its gradient, logits fp32 [{n},{e}], top-{k}")
        w.unit = "rows/s"
        w.rows = n
        return w

    if name == "moe_dispatch":
        n, e, k, d = 16384, 64, 2, 4096
        g.manual_seed(1008)
        lg = (torch.round(torch.randn(n, e, generator=g) * 4096) / 4096).to(dev)
        x = rn(n, d)
        idx, wt, cnt, sl, od = _hip.route(lg, k)
        xs = torch.empty(n * k, d, device=dev, dtype=torch.bfloat16)
        out = torch.empty_like(x)

        def gather():     # from the token's side (fm_route hands out slot as well as order)
            _check(L.fm_moe_scatter(x.data_ptr(), sl.data_ptr(), None, xs.data_ptr(), n, d, k, BF, st),
                   "fm_moe_scatter")

        def combine():
            _check(L.fm_moe_combine(xs.data_ptr(), wt.data_ptr(), sl.data_ptr(), out.data_ptr(), n, d, k,
                                    BF, st), "fm_moe_combine")

        def step():
            gather()
            combine()

        def check(r=256):
            from oracle import oracle as O
            step()
            torch.cuda.synchronize()
            # gathered rows against x[order // k]; the combine against its definition on the first tokens
            ok = bool(torch.equal(xs[:r].cpu(), x.cpu()[(od[:r].cpu().long() // k)]))
            t0 = 64
            ref = sum(wt[:t0, j, None].cpu() * xs.cpu()[sl.cpu().long().view(n, k)[:t0, j]].float() for j in range(k))
            return ok and _close(out[:t0], ref)

        w.check = check
        w.step = step
        w.dominant_launch = combine
        xs_a, xs_b = xs[:n], xs[n:]
        w.floor = [lambda i: ((x,), (xs_a, xs_b)), lambda i: ((xs_a, xs_b), (out,))]
        w.dominant = "combine_kernel<bf16>"
        w.dominant_bytes = n * d * 2 * (k + 1)
        w.bytes = 2 * n * d * 2 * (k + 1)
        w.desc = (f"token gather into expert order + weighted combine back, x bf16 [{n},{d}], "
                  f"top-{k} over {e} experts")
        w.rows = n
        return w

    raise ValueError(name)


def _close(a, b, rel=1e-2):
    a, b = a.detach().float().cpu(), b.detach().float().cpu()
    return bool(((a - b).abs().max() <= rel * b.abs().max().clamp_min(1e-30)).item())


def time_steps(torch, fn, steps, warmup):
    # at least `warmup` untimed steps, and at least 20 ms of them: the self-check that runs before
    # is CPU work, the GPU idles meanwhile and its first launches afterwards run below full clocks
    t_warm = time.perf_counter()
    done = 0
    while done < warmup or time.perf_counter() - t_warm < 0.02:
        fn()
        done += 1
        if done % 16 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps     # ms per step


def time_kernel_events(torch, fn, steps, before=None):
    """Average duration of the launches `fn` enqueues, HIP events on the launch stream (the
    benchmark's own stream is torch's current stream, so these events are recorded on it).
    `before` (untimed) is what precedes those launches in every step of the workload: a backward
    is timed behind its forward, as it runs in the timed region and in a profile of this run."""
    pairs = []
    for _ in range(steps):
        if before is not None:
            before()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        pairs.append((a, b))
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) for a, b in pairs)
    return sum(times) / len(times), times[0], times[len(times) // 2]


def time_back_to_back(torch, fn, reps, batches=2):
    """ms per launch of `reps` launches enqueued back to back between one pair of events (no event,
    hence no cache write-back, between the launches): best of `batches`."""
    best = float("inf")
    for _ in range(batches):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b) / reps)
    return best


def time_graph(torch, step_fns, steps):
    """The same launches replayed from one HIP graph that holds len(step_fns) steps: what the step
    costs when the host enqueues nothing. ms per step."""
    stream = torch.cuda.current_stream()
    for fn in step_fns:
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for fn in step_fns:
            fn()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    reps = max(2, steps // len(step_fns))
    t0 = time.perf_counter()
    for _ in range(reps):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / (reps * len(step_fns))


def time_cpu(fn, budget_s=8.0, tries=3):
    """min of up to `tries` passes of a CPU callable, stopping once `budget_s` is spent. seconds."""
    best = float("inf")
    t_all = time.perf_counter()
    for _ in range(tries):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
        if time.perf_counter() - t_all > budget_s:
            break
    return best


def time_eager(torch, fn):
    """min of 5 event-timed passes of a torch expression on the GPU, after 2 warm-up passes. ms."""
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b))
    return best


def measure(torch, w, steps, warmup, L, cpu=True):
    # gate first: one step's output against the CPU oracle on a bounded row sample (the idea of the
    # reference's kbench gate, forgemind/cli/kbench.py:197-213, 264-278); outside every timed region
    checked = bool(w.check()) if hasattr(w, "check") else None
    ms = time_steps(torch, w.step, steps, warmup)
    avg, best, med = time_kernel_events(torch, w.dominant_launch, steps, getattr(w, "dominant_before", None))
    kernel = L.fm_last_kernel().decode()
    out = {
        "desc": w.desc,
        "checked": checked,
        "ms_per_step": round(ms, 5),
        "algorithmic_bytes": w.bytes,
        "gbps": round(w.bytes / ms / 1e6, 1),
        "frac_of_hbm_peak": round(w.bytes / ms / 1e6 / HBM_PEAK_GBPS, 4),
        "rows_per_s": round(w.rows / ms * 1e3, 1),
        "dominant_kernel": kernel,
        "dominant_launches": w.dominant,
        "dominant_ms_avg": round(avg, 5), "dominant_ms_min": round(best, 5),
        "dominant_ms_median": round(med, 5),
        "dominant_gbps": round(w.dominant_bytes / avg / 1e6, 1),
        "dominant_traffic_bytes": measured_traffic(kernel),
        "unit": w.unit,
    }
    if hasattr(w, "required_bytes"):
        # bytes the dataflow must move (rows with an ignored label are never read), next to the
        # per-logit accounting above
        out["required_bytes"] = w.required_bytes
        out["required_gbps"] = round(w.required_bytes / ms / 1e6, 1)
        out["required_frac_of_hbm_peak"] = round(w.required_bytes / ms / 1e6 / HBM_PEAK_GBPS, 4)
    if hasattr(w, "l2_bytes"):       # bytes that cross the L2 boundary (both sweeps of a row), as counted
        out["l2_boundary_bytes"] = w.l2_bytes
        out["l2_boundary_gbps"] = round(w.l2_bytes / ms / 1e6, 1)
        out["l2_boundary_frac_of_hbm_peak"] = round(w.l2_bytes / ms / 1e6 / HBM_PEAK_GBPS, 4)
    if hasattr(w, "warm_step"):      # same buffers every step: served by the memory-side cache
        out["cache"] = "cold (buffer sets rotate through more than the 256 MB memory-side cache)"
        wm = time_steps(torch, w.warm_step, steps, warmup)
        out["warm_cache_ms_per_step"] = round(wm, 5)
        out["warm_cache_gbps"] = round(w.bytes / wm / 1e6, 1)
        out["warm_cache_rows_per_s"] = round(w.rows / wm * 1e3, 1)
    if hasattr(w, "graph_steps"):    # launch-sized workloads: is the eager loop bound by the host?
        gm = time_graph(torch, w.graph_steps, max(steps, 4 * len(w.graph_steps)))
        out["graph_replay_ms_per_step"] = round(gm, 5)
        out["graph_replay_rows_per_s"] = round(w.rows / gm * 1e3, 1)
    if hasattr(w, "eager"):          # the reference's torch expression on this GPU (its no-kernel path)
        out["torch_eager_gpu_ms"] = round(time_eager(torch, w.eager), 4)
    if cpu and hasattr(w, "cpu"):    # the CPU oracle on this box's host cores, bounded sample
        fn, scale, sample = w.cpu()
        sec = time_cpu(fn) * scale
        out["cpu_ms"] = round(sec * 1e3, 1)
        out["cpu_gbps"] = round(w.bytes / sec / 1e9, 3)
        out["cpu_sample"] = sample
    if hasattr(w, "floor"):          # last: the sweeps overwrite the workload's outputs
        out.update(measure_floor(torch, w, steps, warmup, L, ms))
    return out


# ---------------------------------------------------------------------------- floors
# (threads, vectors per thread) of fm_stream_probe_mix and the persistent grids tried with each
FLOOR_SHAPES = ((256, 2), (256, 4), (512, 2), (1024, 4))
FLOOR_GRIDS = (0, 2048, 1024)       # 0: one workgroup per tile


def measure_floor(torch, w, steps, warmup, L, ms):
    """The workload's step as bare data movement: for each of its launches the best
    fm_stream_probe_mix variant over tile shapes, grids and store kinds, on the workload's own
    buffers with that launch's reads and writes; then those best sweeps timed back to back with
    the protocol the real step was timed with."""
    st = torch.cuda.current_stream().cuda_stream
    dev = torch.device("cuda:0")
    sink = torch.zeros(1, device=dev, dtype=torch.int32)
    sets = getattr(w, "sets", 1)

    def launcher(spec, kind, thr, vec, grid):
        def go(i):
            rd, wr = spec(i)
            nbytes = rd[0].numel() * rd[0].element_size()
            ptr = [t.data_ptr() for t in rd] + [None] * (3 - len(rd))
            out = [t.data_ptr() for t in wr] + [None] * (2 - len(wr))
            _check(L.fm_stream_probe_mix(ptr[0], ptr[1], ptr[2], out[0], out[1], sink.data_ptr(), nbytes,
                                         len(rd), len(wr), kind, thr, vec, grid, st), "fm_stream_probe_mix")
        return go

    per_launch = []      # for every launch: {store kind: (ms, launcher, label)}, the best shape and grid of that kind
    for spec in w.floor:
        rd, wr = spec(0)
        nbytes = rd[0].numel() * rd[0].element_size()
        kinds = (0,) if not wr else ((0, 1) if len(wr) == 1 else (0, 1, 2))
        best = {}
        for thr, vec in FLOOR_SHAPES:
            if nbytes % (thr * vec * 16):
                continue
            tiles = nbytes // (thr * vec * 16)
            for grid in FLOOR_GRIDS:
                if grid >= tiles and grid != 0:
                    continue
                for kind in kinds:
                    go = launcher(spec, kind, thr, vec, grid)
                    state = {"i": 0}

                    def one():
                        state["i"] = (state["i"] + 1) % sets
                        go(state["i"])
                    for _ in range(3):
                        one()
                    avg = time_back_to_back(torch, one, 10)
                    if kind not in best or avg < best[kind][0]:
                        best[kind] = (avg, go, f"{len(rd)}r{len(wr)}w {thr}x{vec} grid {grid or tiles} store {kind}")
        if not best:
            return {"floor_ms": None}
        per_launch.append(best)
    # the store kinds are chosen for the step as a whole (what one launch leaves in the caches is
    # what the next one finds): every combination of kinds, each launch in its best shape for that kind
    import itertools
    fms, names = None, None
    for combo in itertools.product(*[sorted(b) for b in per_launch]):
        chosen = [per_launch[j][kind][1] for j, kind in enumerate(combo)]
        state = {"i": 0}

        def floor_step():
            i = state["i"] = (state["i"] + 1) % sets
            for go in chosen:
                go(i)
        t = time_steps(torch, floor_step, steps, warmup)
        if fms is None or t < fms:
            fms = t
            names = [f"{per_launch[j][kind][2]}: {per_launch[j][kind][0] * 1e3:.1f} us" for j, kind in enumerate(combo)]
    return {"floor_ms": round(fms, 5), "of_floor": round(fms / ms, 4), "floor_sweeps": names}


def stream_ceiling(torch, L, dev):
    """What a plain read sweep and a plain copy reach on this GPU (1 GiB, ten launches back to back,
    best of two such batches; the copy over both store kinds, two tile shapes and two grids)."""
    n = 1 << 30
    src = torch.empty(n, device=dev, dtype=torch.uint8).fill_(1)
    dst = torch.empty_like(src)
    sink = torch.zeros(1, device=dev, dtype=torch.int32)
    st = torch.cuda.current_stream().cuda_stream
    out = {}
    fn = lambda: _check(L.fm_stream_probe(src.data_ptr(), dst.data_ptr(), sink.data_ptr(), n, 0, st),
                        "fm_stream_probe")
    fn()
    best = time_back_to_back(torch, fn, 10)
    out["read_gbps"] = round(n / best / 1e6, 1)
    best_copy = None
    for thr, vec in ((512, 2), (1024, 4)):
        for grid in (0, 2048):
            for kind in (0, 1):
                fn = lambda: _check(L.fm_stream_probe_mix(src.data_ptr(), None, None, dst.data_ptr(), None,
                                                          sink.data_ptr(), n, 1, 1, kind, thr, vec, grid, st),
                                    "fm_stream_probe_mix")
                fn()
                b = time_back_to_back(torch, fn, 10)
                if best_copy is None or b < best_copy[0]:
                    best_copy = (b, f"{thr}x{vec} grid {grid or 'tiles'} store {'nt' if kind else 'plain'}")
    out["copy_gbps"] = round(2 * n / best_copy[0] / 1e6, 1)
    out["copy_form"] = best_copy[1]
    return out


def kbench_style(torch):
    """The reference's own protocol (forgemind/cli/kbench.py:122-158): public API, fresh
    detach().clone().requires_grad_() inputs and autograd inside the timed region, warm-up 5,
    min of 20; shapes and forward-only cases as forgemind/cli/kbench.py:55-116 builds them.
    Reported next to the kernel-only numbers, never instead of them. ms per call."""
    import forgeminds_amd as fm
    dev = "cuda:0"
    out = {}

    def run(make, fn, backward=True):
        tensors = make()
        def step():
            ins = [t.detach().clone().requires_grad_(t.is_floating_point() and backward) for t in tensors]
            o = fn(ins)
            if backward:
                o.float().sum().backward()
        for _ in range(5):
            step()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(20):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            step()
            b.record()
            torch.cuda.synchronize()
            best = min(best, a.elapsed_time(b))
        return round(best, 4)

    rnd = lambda *sh: torch.randn(*sh, device=dev).bfloat16()
    out["rms_norm [8192,4096]"] = run(lambda: [rnd(8192, 4096), torch.ones(4096, device=dev).bfloat16()],
                                      lambda t: fm.kernels.rms_norm(t[0], t[1], 1e-6))
    out["add_rms_norm [8192,4096]"] = run(
        lambda: [rnd(8192, 4096), rnd(8192, 4096), torch.ones(4096, device=dev).bfloat16()],
        lambda t: sum(fm.kernels.add_rms_norm(t[0], t[1], t[2], 1e-6)))
    out["swiglu [8192,11008]"] = run(lambda: [rnd(8192, 11008), rnd(8192, 11008)],
                                     lambda t: fm.kernels.swiglu(t[0], t[1]))
    out["swiglu_split [8192,22016]"] = run(lambda: [rnd(8192, 22016)], lambda t: fm.kernels.swiglu_split(t[0]))
    ang = torch.randn(2048, 64, device=dev)
    out["qk_norm_rope [8,2048,32,128]"] = run(
        lambda: [rnd(8, 2048, 32, 128), torch.ones(128, device=dev), ang.cos(), ang.sin()],
        lambda t: fm.kernels.qk_norm_rope(t[0], t[1], t[2].detach(), t[3].detach(), 1e-6))
    out["kl_div_logits [512,32000] fwd"] = run(lambda: [rnd(512, 32000), rnd(512, 32000)],
                                               lambda t: fm.kernels.kl_div_logits(t[0], t[1]), backward=False)
    out["topk [512,32000] k=64"] = run(lambda: [rnd(512, 32000)], lambda t: fm.kernels.topk(t[0], 64)[0])
    out["softmax [8192,128]"] = run(lambda: [rnd(8192, 128)], lambda t: fm.kernels.softmax(t[0], -1))
    out["softmax [8192,4096]"] = run(lambda: [rnd(8192, 4096)], lambda t: fm.kernels.softmax(t[0], -1))
    return out


KBENCH_NOTE = ("reference PERF.md:775-782 lists 0.591 / 1.239 / 2.466 / 2.436 / 1.394 ms for its Triton kernels and "
               "0.276 / 0.436 / 1.314 / 1.563 / - ms for inductor at the first five shapes on an unrecorded NVIDIA "
               "GPU, PERF.md:761-766 85 ms (topk) and 2.6 ms (softmax [8192,128]) on a CPU; the timed region holds "
               "the input clones and autograd as there")


# ---------------------------------------------------------------------------- CPU baseline
def cpu_baseline(torch, w):
    """The CPU oracle on the headline workload's own shape (a bounded sample where the whole shape
    would take more than seconds), on this box's host cores: a reported baseline, never a target."""
    fn, scale, sample = w.cpu()
    fn()                                         # warm-up
    sec = time_cpu(fn, budget_s=25.0) * scale
    unit_rows = w.unit == "rows/s"
    return {
        "value": round(w.rows / sec, 1) if unit_rows else round(w.bytes / sec / 1e9, 3),
        "unit": w.unit, "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"oracle (CPU restatement of the reference's torch expression) on {sample}, "
                  f"min of up to 3 passes, {sec * 1e3:.1f} ms for the whole workload, same byte accounting",
    }


# BASELINE.json's configurations, in its order, and the workload that measures each
CONFIGS = (("cfg1", "rmsnorm"), ("cfg2", "ce"), ("cfg3", "route"), ("cfg4", "add_rmsnorm"), ("cfg5", "kl"),
           ("cfg5b", "topk"))


def config_row(r, rows_unit):
    """One BASELINE configuration as numbers only."""
    row = {
        "ms": r["ms_per_step"],
        "frac": None if rows_unit else r.get("required_frac_of_hbm_peak", r["frac_of_hbm_peak"]),
        "frac_per_element_accounting": None if rows_unit else r["frac_of_hbm_peak"],
        "rows_per_s": r["rows_per_s"], "checked": r["checked"],
        "dom_kernel": r["dominant_kernel"].split("<")[0],
        "dom_us": round(r["dominant_ms_avg"] * 1e3, 2), "dom_us_min": round(r["dominant_ms_min"] * 1e3, 2),
        "floor_ms": r.get("floor_ms"), "of_floor": r.get("of_floor"),
    }
    if "warm_cache_ms_per_step" in r:
        row["warm_ms"] = r["warm_cache_ms_per_step"]
    if "graph_replay_ms_per_step" in r:
        row["graph_ms"] = r["graph_replay_ms_per_step"]
    return row


def short_row(r):
    row = {"ms": r["ms_per_step"], "gbps": r["gbps"], "frac": r["frac_of_hbm_peak"], "checked": r["checked"]}
    if r.get("unit") == "rows/s":
        row["rows_per_s"] = r["rows_per_s"]
    if "l2_boundary_frac_of_hbm_peak" in r:
        row["frac_l2_boundary"] = r["l2_boundary_frac_of_hbm_peak"]
    if "floor_ms" in r and r["floor_ms"] is not None:
        row["floor_ms"], row["of_floor"] = r["floor_ms"], r["of_floor"]
    return row


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py: this path is measured on ONE MI355X (no sharding, no collectives); "
              f"--gpus {a.gpus} is not a supported configuration", file=sys.stderr)
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    from forgeminds_amd.kernels import _hip
    L = _hip.lib()          # raises if libfmhip.so is not built: never a silent fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if a.copy_probe:
        # one plain copy of known size per step: what FETCH_SIZE / WRITE_SIZE are calibrated on
        n = a.copy_probe << 20
        src = torch.empty(n, device=dev, dtype=torch.uint8).fill_(1)
        dst = torch.empty_like(src)
        st = torch.cuda.current_stream().cuda_stream
        for _ in range(max(a.steps, 1)):
            _check(L.fm_stream_probe(src.data_ptr(), dst.data_ptr(), None, n, 1, st), "fm_stream_probe")
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_bytes_read": n, "copy_probe_bytes_written": n,
                          "launches": max(a.steps, 1)}))
        return 0

    # everything runs on a stream of the benchmark's own (torch's current stream from here on):
    # the library calls get its raw handle, the events are recorded on it, and it can be captured
    side = torch.cuda.Stream(device=dev)
    torch.cuda.set_stream(side)

    head = make_workload(a.workload, torch, L, dev)
    res = measure(torch, head, a.steps, a.warmup, L, cpu=False)
    avg_ms = res["dominant_ms_avg"]
    kernel = res["dominant_kernel"]
    # the dominant kernel against the roofline, on the bytes it has to move (for the cross entropy:
    # rows with an ignored label are written but never read)
    dom_bytes = getattr(head, "dominant_required_bytes", head.dominant_bytes)
    achieved = dom_bytes / avg_ms / 1e6
    line = {
        "metric": METRIC,
        "value": res["rows_per_s"] if head.unit == "rows/s" else res["gbps"],
        "unit": head.unit,
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if a.workload not in ("route", "route_256x8", "route_train") else "f32", "data": "synthetic",
        "config": {"workload": head.desc, "name": a.workload,
                   "timing": "K steps between two device synchronisations, inputs resident in HBM",
                   "inputs": "torch.Generator(cpu).manual_seed(1000 + config number), drawn in row chunks"},
        "checked": res["checked"],
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic(kernel),
            "traffic_source": TRAFFIC_SOURCE if measured_traffic(kernel) is not None else None,
            "kernel": kernel, "algorithmic_bytes_per_launch": dom_bytes,
            "per_element_accounting_bytes": head.dominant_bytes,
            "avg_launch_ms": avg_ms,
        },
        "frac_of_hbm_peak": res["frac_of_hbm_peak"],
    }
    line["cpu_baseline"] = None if (a.no_cpu or not hasattr(head, "cpu")) else cpu_baseline(torch, head)
    head_unit_rows = head.unit == "rows/s"
    del head
    torch.cuda.empty_cache()
    detail = {a.workload: res}
    units = {a.workload: head_unit_rows}
    if not a.no_extras:
        chosen = [n for n in a.only.split(",") if n] or WORKLOADS
        for name in chosen:
            if name == a.workload:
                continue
            wl = make_workload(name, torch, L, dev)
            detail[name] = measure(torch, wl, a.steps, a.warmup, L, cpu=not a.no_cpu)
            units[name] = wl.unit == "rows/s"
            del wl
            torch.cuda.empty_cache()
        if line["cpu_baseline"] is not None:     # the headline's CPU column, in the table's units
            cb = line["cpu_baseline"]
            if cb["unit"] == "GB/s":
                detail[a.workload]["cpu_gbps"] = cb["value"]
                detail[a.workload]["cpu_ms"] = round(detail[a.workload]["algorithmic_bytes"] / cb["value"] / 1e6, 1)
    _SHARED.clear()
    torch.cuda.empty_cache()
    by_workload = dict(CONFIGS)
    line["roofline"]["configs"] = {c: config_row(detail[wn], units[wn]) for c, wn in CONFIGS if wn in detail}
    named = set(by_workload.values())
    line["workloads"] = {n: short_row(r) for n, r in detail.items() if n not in named}
    if not a.no_extras and not a.only:
        line["kbench"] = kbench_style(torch)
    line["hbm_ceiling_measured"] = stream_ceiling(torch, L, dev)
    if a.detail:
        os.makedirs(os.path.dirname(os.path.abspath(a.detail)), exist_ok=True)
        with open(a.detail, "w") as f:
            json.dump({"line": line, "workloads": detail, "kbench_note": KBENCH_NOTE}, f, indent=1)
    print(json.dumps(line, separators=(",", ":")))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""The public ``fm.kernels`` surface on a GPU: the HIP path is the one that runs (``stats()``
counts it as fast), autograd / custom-op / torch.compile plumbing gives the same numbers as the
direct launches, and the module-level callers (nn.RMSNorm, loss, moe.Router) sit on top of it.
"""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import forgeminds_amd as fm
from forgeminds_amd import kernels
from forgeminds_amd.kernels import _hip, _ops
from forgeminds_amd.loss import chunked_cross_entropy, logits_cross_entropy
from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_gpu_and_library():
    assert torch.cuda.is_available() and _hip.loaded(), _hip.load_error()
    assert kernels.available()


def close(a, b, rel=1e-2):
    a, b = a.detach().float().cpu(), b.detach().float().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item() <= rel


def test_gpu_calls_take_the_hip_path():
    kernels.reset_stats()
    x = torch.randn(64, 256, device=DEV, dtype=torch.bfloat16)
    w = torch.ones(256, device=DEV)
    kernels.rms_norm(x, w)
    kernels.add_rms_norm(x, x, w)
    kernels.cross_entropy(torch.randn(8, 100, device=DEV), torch.randint(0, 100, (8,), device=DEV))
    kernels.kl_div_logits(torch.randn(8, 100, device=DEV), torch.randn(8, 100, device=DEV))
    kernels.topk(torch.randn(8, 100, device=DEV), 5)
    kernels.softmax(torch.randn(8, 100, device=DEV))
    kernels.moe_route(torch.randn(8, 16, device=DEV), 2)
    st = kernels.stats()
    assert st["fast"] == 7 and st["fallback"] == 0, st
    kernels.set_backend("fallback")
    kernels.rms_norm(x, w)
    assert kernels.stats()["reasons"] == {"backend=fallback": 1}
    kernels.set_backend("triton")              # the reference's name for "force the kernels"
    kernels.rms_norm(x, w)
    assert kernels.stats()["fast"] == 8
    kernels.set_backend("auto")
    kernels.rms_norm(x.double(), w.double())   # float64 stays with torch, and says why
    assert "dtype torch.float64" in kernels.stats()["reasons"]


def test_inference_calls_record_no_graph_and_give_the_same_bits():
    x = torch.randn(64, 256, device=DEV, dtype=torch.bfloat16)
    w = (1 + 0.1 * torch.randn(256, device=DEV)).bfloat16()
    b = torch.zeros_like(w)
    xg, wg = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    cos, sin = torch.randn(8, 32, device=DEV), torch.randn(8, 32, device=DEV)
    calls = [
        (lambda a, ww: kernels.rms_norm(a, ww), (x, w), (xg, wg)),
        (lambda a, ww: kernels.add_rms_norm(a, a, ww)[1], (x, w), (xg, wg)),
        (lambda a, ww: kernels.layer_norm(a, ww, b), (x, w), (xg, wg)),
        (lambda a, ww: kernels.add_layer_norm(a, a, ww, b)[1], (x, w), (xg, wg)),
        (lambda a, ww: kernels.softmax(a), (x, w), (xg, wg)),
        (lambda a, ww: kernels.swiglu(a, a), (x, w), (xg, wg)),
        (lambda a, ww: kernels.swiglu_split(a), (x, w), (xg, wg)),
        (lambda a, ww: kernels.topk(a, 5)[0], (x, w), (xg, wg)),
        (lambda a, ww: kernels.qk_norm_rope(a.view(1, 8, 8, 256)[..., :64].contiguous(), ww[:64].contiguous(), cos, sin),
         (x, w), (xg, wg)),
    ]
    for fn, plain, tracked in calls:
        y0 = fn(*plain)
        assert y0.grad_fn is None and not y0.requires_grad
        y1 = fn(*tracked)
        assert y1.grad_fn is not None
        assert torch.equal(y0, y1.detach())
        with torch.no_grad():
            y2 = fn(*tracked)
        assert y2.grad_fn is None and torch.equal(y2, y0)


@pytest.mark.parametrize("dt,wdt", [(torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                    (torch.float32, torch.float32), (torch.float16, torch.float16)])
def test_rms_norm_autograd_matches_oracle(dt, wdt):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 50, 512, generator=g).to(dt)
    w = (1 + 0.1 * torch.randn(512, generator=g)).to(wdt)
    dy = torch.randn(3, 50, 512, generator=g).to(dt)
    xd = x.to(DEV).requires_grad_(True)
    wd = w.to(DEV).requires_grad_(True)
    y = kernels.rms_norm(xd, wd, 1e-6)
    y.backward(dy.to(DEV))
    oy, _ = O.rms_norm(x, w)
    odx, odw = O.rms_norm_bwd(x, w, dy)
    assert y.shape == x.shape and y.dtype == dt
    assert close(y, oy) and close(xd.grad, odx) and close(wd.grad, odw)
    assert wd.grad.dtype == wdt
    # non-contiguous input (reference tests/test_edge_cases.py:106-111)
    xt = torch.randn(512, 40, device=DEV).t()
    assert not xt.is_contiguous()
    assert close(kernels.rms_norm(xt, torch.ones(512, device=DEV)), F.rms_norm(xt, (512,), None, 1e-6), 1e-5)


def test_add_rms_norm_autograd_and_partial_use():
    g = torch.Generator().manual_seed(1)
    x, dl = torch.randn(40, 768, generator=g).bfloat16(), torch.randn(40, 768, generator=g).bfloat16()
    w = 1 + 0.1 * torch.randn(768, generator=g)
    gy, gxn = torch.randn(40, 768, generator=g).bfloat16(), torch.randn(40, 768, generator=g).bfloat16()
    xd, dd, wd = (t.to(DEV).requires_grad_(True) for t in (x, dl, w))
    xn, y = kernels.add_rms_norm(xd, dd, wd, 1e-5)
    torch.autograd.backward([xn, y], [gxn.to(DEV), gy.to(DEV)])
    oxn, oy, _ = O.add_rms_norm(x, dl, w, 1e-5)
    odx, odw = O.add_rms_norm_bwd(oxn, w, gy, gxn, 1e-5)
    assert torch.equal(xn.cpu(), oxn) and close(y, oy)
    assert close(xd.grad, odx) and torch.equal(xd.grad, dd.grad) and close(wd.grad, odw)
    assert xd.grad.data_ptr() != dd.grad.data_ptr()          # leaves do not share storage
    # only the normalised output used / only the residual used
    xd2, dd2 = (t.to(DEV).requires_grad_(True) for t in (x, dl))
    _, y2 = kernels.add_rms_norm(xd2, dd2, w.to(DEV), 1e-5)
    y2.backward(gy.to(DEV))
    assert close(xd2.grad, O.add_rms_norm_bwd(oxn, w, gy, None, 1e-5)[0])
    xd3, dd3 = (t.to(DEV).requires_grad_(True) for t in (x, dl))
    xn3, _ = kernels.add_rms_norm(xd3, dd3, w.to(DEV), 1e-5)
    xn3.backward(gxn.to(DEV))
    assert torch.equal(xd3.grad.cpu(), gxn)


def test_op_path_equals_eager_path_bit_for_bit():
    # reference tests/test_kernel_ops.py:94-109
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 64, generator=g).to(DEV)
    w = torch.randn(64, generator=g).to(DEV)

    def run(mode, fn):
        _ops.use_custom_ops(mode)
        ins = [t.clone().requires_grad_(True) for t in (x, x * 0.5, w)]
        out = fn(ins)
        out.square().sum().backward()
        return out.detach().clone(), [t.grad.clone() for t in ins if t.grad is not None]

    for fn in (lambda t: kernels.rms_norm(t[0], t[2], 1e-6),
               lambda t: sum(kernels.add_rms_norm(t[0], t[1], t[2], 1e-6)),
               lambda t: kernels.swiglu(t[0], t[1]) * t[2],
               lambda t: kernels.swiglu_split(t[0]) * t[2][:32] + t[1][:, :32]):
        ye, ge = run(False, fn)
        yo, go = run(True, fn)
        assert torch.equal(ye, yo) and len(ge) == len(go)
        assert all(torch.equal(a, b) for a, b in zip(ge, go))
    _ops.use_custom_ops(True)
    with torch.no_grad():
        assert not kernels.rms_norm(x, w).requires_grad


def test_compile_fullgraph_and_export_keep_the_kernel():
    # reference tests/test_kernel_ops.py:120-153
    x = torch.randn(6, 64, device=DEV)
    w = torch.randn(64, device=DEV)

    def fn(t, ww):
        a, b = kernels.add_rms_norm(t, t * 2, ww, 1e-6)
        return kernels.rms_norm(a + b, ww, 1e-6)

    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    fn(xr, wr).square().sum().backward()
    xc, wc = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    out = torch.compile(fn, backend="aot_eager", fullgraph=True)(xc, wc)
    out.square().sum().backward()
    assert torch.allclose(out, fn(x, w), atol=2e-6, rtol=1e-5)
    assert torch.allclose(xc.grad, xr.grad, atol=1e-4, rtol=1e-4)
    assert torch.allclose(wc.grad, wr.grad, atol=1e-4, rtol=1e-4)

    class M(nn.Module):
        def forward(self, t):
            return kernels.rms_norm(t, w, 1e-6)

    ep = torch.export.export(M(), (x,))
    targets = [str(n.target) for n in ep.graph.nodes if n.op == "call_function"]
    assert "forgemind.rms_norm.default" in targets, targets


def test_cross_entropy_autograd_and_callers():
    g = torch.Generator().manual_seed(3)
    lg = (2 * torch.randn(300, 4000, generator=g)).bfloat16()
    y = torch.randint(0, 4000, (300,), generator=g)
    y[::7] = -100
    ol, og = O.cross_entropy(lg, y)
    lgd = lg.to(DEV).requires_grad_(True)
    loss = kernels.cross_entropy(lgd, y.to(DEV))
    (loss * 3.0).backward()
    assert loss.dtype == torch.float32 and loss.item() == pytest.approx(ol.item(), rel=1e-4)
    assert close(lgd.grad, og.float() * 3.0)
    # the gradient written over an owned logits tensor; one backward per forward
    owned = lg.to(DEV)
    leaf = owned.clone().requires_grad_(True)
    tmp = leaf * 1.0                                   # a temporary that only the loss reads
    l_in = kernels.cross_entropy(tmp, y.to(DEV), inplace=True)
    l_in.backward(retain_graph=True)
    assert l_in.item() == loss.item() and close(leaf.grad, og.float())
    with pytest.raises(RuntimeError, match="already consumed"):
        l_in.backward()
    with torch.no_grad():                              # no gradient wanted: plain forward
        assert kernels.cross_entropy(owned, y.to(DEV)).item() == pytest.approx(ol.item(), rel=1e-4)
    # logits_cross_entropy on [B, T, V] (reference tests/test_edge_cases.py:50-56)
    l3 = logits_cross_entropy(lg.to(DEV).view(3, 100, 4000), y.to(DEV).view(3, 100))
    assert l3.item() == pytest.approx(ol.item(), rel=1e-4)
    # chunked CE over h @ W^T equals the unchunked one, and trains both operands
    h = torch.randn(70, 64, generator=g).to(DEV).requires_grad_(True)
    wt = torch.randn(500, 64, generator=g).to(DEV).requires_grad_(True)
    yy = torch.randint(0, 500, (70,), generator=g).to(DEV)
    yy[3] = -100
    a = chunked_cross_entropy(h, wt, yy, chunk=32)
    a.backward()
    ref = F.cross_entropy(h.detach() @ wt.detach().t(), yy, ignore_index=-100)
    assert a.item() == pytest.approx(ref.item(), rel=1e-4)
    assert h.grad is not None and wt.grad is not None
    # all ignored: 0.0 and a usable backward (reference tests/test_edge_cases.py:21-28)
    h2 = torch.randn(6, 64, device=DEV, requires_grad=True)
    z = chunked_cross_entropy(h2, wt, torch.full((6,), -100, device=DEV), chunk=4)
    z.backward()
    assert z.item() == 0.0 and h2.grad is not None and not h2.grad.any()


def test_kl_gradient_in_forward_reuse_and_second_backward():
    g = torch.Generator().manual_seed(41)
    s = (3 * torch.randn(12, 3000, generator=g)).bfloat16()
    t = (s.float() + 0.5 * torch.randn(12, 3000, generator=g)).bfloat16()
    _, og = O.kl_div(s, t, "mean", 1.0)
    leaf = s.to(DEV).requires_grad_(True)
    tmp = leaf * 1.0                                   # a temporary that only the loss reads
    loss = kernels.kl_div_logits(tmp, t.to(DEV), reuse=True)
    (loss * 2.0).backward(retain_graph=True)
    assert close(leaf.grad, og.float() * 2.0)
    with pytest.raises(RuntimeError, match="already consumed"):
        loss.backward()
    # distillation loop: chunk logits overwritten by their gradient, both operands train
    hs = torch.randn(40, 32, generator=g).to(DEV).requires_grad_(True)
    w = torch.randn(700, 32, generator=g).to(DEV).requires_grad_(True)
    ht = torch.randn(40, 32, generator=g).to(DEV)
    head = nn.Linear(32, 700, bias=False).to(DEV)
    out = kernels.kl_distill_loss(hs, ht, w, head, chunk=16)
    out.backward()
    ref = F.kl_div(torch.log_softmax(hs.detach() @ w.detach().t(), -1), torch.softmax(head(ht).detach(), -1),
                   reduction="sum") / 40
    assert out.item() == pytest.approx(ref.item(), rel=1e-4)
    assert hs.grad is not None and w.grad is not None and hs.grad.abs().sum() > 0


def test_last_kernel_names_what_ran():
    x = torch.randn(64, 1024, device=DEV).bfloat16()
    w = torch.ones(1024, device=DEV)
    _hip.rmsnorm_fwd(x, w, 1e-6)
    # a plain norm's forward keeps x cached for its backward, the fused add streams it
    assert _hip.last_kernel() == "norm_fwd_kernel<bf16_t, float, 64, 2, false, false, true>"
    _hip.add_rmsnorm_fwd(x, x, w, 1e-6)
    assert _hip.last_kernel() == "norm_fwd_kernel<bf16_t, float, 64, 2, true, false, false>"
    _hip.topk(torch.randn(8, 128256, device=DEV).bfloat16(), 64, torch.int32)
    assert _hip.last_kernel().startswith("topk_lds_kernel<bf16_t, ")


def test_row_width_picks_the_form_that_was_measured_faster():
    """The one-launch KL and the norm backward choose a kernel form by row width and dtype; the
    names say which ran (what each choice rests on is written next to the dispatch in the source)."""
    def kl_kernel(v, dt):
        s = torch.randn(4, v, device=DEV).to(dt)
        _hip.kl_loss_grad(s, s.flip(0).contiguous(), 1.0, "mean", dt)
        return _hip.last_kernel()

    bf, f32 = torch.bfloat16, torch.float32
    assert kl_kernel(16384, bf).startswith("kl_loss_grad_kernel<bf16_t, bf16_t")          # registers
    assert kl_kernel(20000, bf) == "kl_loss_grad_held_kernel<bf16_t, bf16_t, 256, 13, 3>"  # 3 workgroups a unit
    assert kl_kernel(50304, bf) == "kl_loss_grad_held_kernel<bf16_t, bf16_t, 256, 22, 9>"  # 2
    assert kl_kernel(128256, bf) == "kl_loss_grad_held_kernel<bf16_t, bf16_t, 512, 22, 9>"  # 1
    assert kl_kernel(32000, f32) == "kl_loss_grad_held_kernel<float, float, 512, 22, 9>"
    assert kl_kernel(300000, bf).startswith("kl_loss_grad_wide_kernel<bf16_t, bf16_t")    # two sweeps

    def norm_kernel(d, dt, ln):
        x = torch.randn(3, d, device=DEV).to(dt)
        w = torch.ones(d, device=DEV, dtype=dt)
        if ln:
            _, _, mean, rstd = _hip.layernorm_fwd(x, w, w, 1e-5)
            _hip.layernorm_bwd(x, w, mean, rstd, x)
        else:
            _, rstd = _hip.rmsnorm_fwd(x, w, 1e-6)
            _hip.rmsnorm_bwd(x, w, rstd, x)
        return _hip.last_kernel()

    # <T, WT, LayerNorm, vectors a thread, dy in LDS, next row under the output sweep>
    assert norm_kernel(32768, bf, False) == "norm_bwd_wide_acc<bf16_t, bf16_t, false, 4, false, false>"
    assert norm_kernel(32768, bf, True) == "norm_bwd_wide_acc<bf16_t, bf16_t, true, 4, true, false>"
    assert norm_kernel(20480, f32, False) == "norm_bwd_wide_acc<float, float, false, 6, true, false>"
    assert norm_kernel(32768, f32, False) == "norm_bwd_wide_acc<float, float, false, 8, true, true>"


def test_norm_reads_x_cached_only_when_it_fits_the_memory_side_cache():
    """Forward and backward of a plain norm read x with cached loads up to 256 MiB of x and with
    streaming loads beyond; both forms give the same numbers (the load kind is the only difference)."""
    w = torch.ones(2048, device=DEV)
    names, outs = [], []
    for n in (65536, 65544):             # 256 MiB of bf16 x exactly, and eight rows more
        x = torch.randn(n, 2048, device=DEV).bfloat16()
        y, rstd = _hip.rmsnorm_fwd(x, w, 1e-6)
        names.append(_hip.last_kernel())
        dx, dw = _hip.rmsnorm_bwd(x, w, rstd, y)[:2]
        torch.cuda.synchronize()
        outs.append((x, y, rstd, dx, dw))
    assert names[0].startswith("norm_fwd_kernel<bf16_t, float, ") and names[0].endswith(", false, false, true>")
    assert names[1].startswith("norm_fwd_kernel<bf16_t, float, ") and names[1].endswith(", false, false, false>")
    # the larger call on the first call's rows: bit-identical y and dx for those rows
    x0, y0, r0, dx0, _ = outs[0]
    xb = torch.cat([x0, outs[1][0][-8:]])
    yb, rb = _hip.rmsnorm_fwd(xb, w, 1e-6)
    dxb = _hip.rmsnorm_bwd(xb, w, rb, yb)[0]
    assert torch.equal(yb[:65536], y0) and torch.equal(rb[:65536], r0) and torch.equal(dxb[:65536], dx0)


def test_fp16_losses_apply_the_upstream_gradient_before_rounding():
    # a loss scaler multiplies the loss by 65536; (softmax - onehot) / 8192 rounded to fp16 FIRST
    # would lose most entries (p / 8192 < 6e-5 is subnormal or zero in fp16)
    g = torch.Generator().manual_seed(77)
    n, v, scale = 8192, 512, 65536.0
    lg = (2 * torch.randn(n, v, generator=g)).half()
    y = torch.randint(0, v, (n,), generator=g)
    y[::9] = -100
    ref = lg.double().requires_grad_(True)           # fp64 autograd of the library routine, unrounded
    (F.cross_entropy(ref, y, ignore_index=-100) * scale).backward()
    want = ref.grad
    lgd = lg.to(DEV).requires_grad_(True)
    (kernels.cross_entropy(lgd, y.to(DEV)) * scale).backward()
    got = lgd.grad.double().cpu()
    assert lgd.grad.dtype == torch.float16
    # one fp16 rounding of the scaled value: half an ulp relative, nothing flushed
    err = (got - want).abs()
    assert (err <= want.abs() * 2.0 ** -10 + 2.0 ** -24).all()
    assert torch.count_nonzero(got) >= 0.99 * torch.count_nonzero(want)
    # KL with an fp16 gradient: same rule
    s = (3 * torch.randn(4096, 256, generator=g)).half()
    t = (s.float() + 0.5 * torch.randn(4096, 256, generator=g)).half()
    sref = s.double().requires_grad_(True)
    (F.kl_div(torch.log_softmax(sref, -1), torch.softmax(t.double(), -1), reduction="sum") / 4096 * scale).backward()
    wantk = sref.grad
    sd = s.to(DEV).requires_grad_(True)
    (kernels.kl_div_logits(sd, t.to(DEV)) * scale).backward()
    errk = (sd.grad.double().cpu() - wantk).abs()
    # one fp16 rounding, plus the fp32 rounding of the two probabilities (up to 1) whose difference
    # the gradient is, times the factor scale / rows = 16 they are multiplied by
    assert (errk <= wantk.abs() * 2.0 ** -10 + (scale / 4096) * 2.0 ** -20).all()
    assert torch.count_nonzero(sd.grad) >= 0.99 * torch.count_nonzero(wantk)


def test_fp16_chunked_cross_entropy_under_checkpointing():
    # fp16 takes the two-pass form, here inside the checkpoint-per-chunk loop of loss.py:23-51
    g = torch.Generator().manual_seed(79)
    h = torch.randn(90, 64, generator=g).half().to(DEV).requires_grad_(True)
    wt = (0.2 * torch.randn(700, 64, generator=g)).half().to(DEV).requires_grad_(True)
    yy = torch.randint(0, 700, (90,), generator=g).to(DEV)
    yy[::11] = -100
    loss = chunked_cross_entropy(h, wt, yy, chunk=32)
    (loss * 1024.0).backward()
    hr = h.detach().float().requires_grad_(True)
    wr = wt.detach().float().requires_grad_(True)
    ref = F.cross_entropy((hr.half().float() @ wr.t()).half().float(), yy, ignore_index=-100)
    (ref * 1024.0).backward()
    assert loss.item() == pytest.approx(ref.item(), rel=2e-3)
    assert close(h.grad, hr.grad, rel=2e-2) and close(wt.grad, wr.grad, rel=2e-2)


def test_losses_allow_a_second_backward_when_asked_to_retain():
    # the reference's KL multiplies its stored gradient out of place (kernels/kl.py:183-191), so
    # retain_graph=True works there; here the first backward scales in place, and with retain=True
    # (which keeps the inputs alive) later ones redo the pass. Without it only the gradient buffer
    # is saved and a second backward says so.
    g = torch.Generator().manual_seed(78)
    lg = (2 * torch.randn(64, 4000, generator=g)).bfloat16()
    y = torch.randint(0, 4000, (64,), generator=g)
    _, og = O.cross_entropy(lg, y)
    lgd = lg.to(DEV).requires_grad_(True)
    once = kernels.cross_entropy(lgd, y.to(DEV))
    saved = [t for t in (once.grad_fn.saved_tensors if hasattr(once.grad_fn, "saved_tensors") else ())]
    assert len(saved) == 1 and saved[0].shape == (64, 4000)      # the gradient buffer only: the logits are not pinned
    once.backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="already consumed"):
        once.backward()
    lgd.grad = None
    loss = kernels.cross_entropy(lgd, y.to(DEV), retain=True)
    (loss * 3.0).backward(retain_graph=True)
    first = lgd.grad.clone()
    lgd.grad = None
    (loss * 5.0).backward()
    assert close(first, og.float() * 3.0) and close(lgd.grad, og.float() * 5.0)
    s = (3 * torch.randn(12, 3000, generator=g)).bfloat16()
    t = (s.float() + 0.5 * torch.randn(12, 3000, generator=g)).bfloat16()
    _, kg = O.kl_div(s, t, "mean", 1.0)
    sd = s.to(DEV).requires_grad_(True)
    kl1 = kernels.kl_div_logits(sd, t.to(DEV))
    kl1.backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="already consumed"):
        kl1.backward()
    sd.grad = None
    kl = kernels.kl_div_logits(sd, t.to(DEV), retain=True)
    (kl * 2.0).backward(retain_graph=True)
    a = sd.grad.clone()
    sd.grad = None
    kl.backward()
    assert close(a, kg.float() * 2.0) and close(sd.grad, kg.float())


def test_compiled_losses_write_the_gradient_in_the_forward():
    # under torch.compile the bf16 / fp32 losses are ONE op whose extra output is the gradient for an
    # upstream gradient of 1 (aux outputs as in the reference's forgemind/kernels/_ops.py:44-48), and the
    # backward is an op that scales that buffer in place: same kernels, same bits as the eager path
    g = torch.Generator().manual_seed(91)
    lg = (2 * torch.randn(96, 4000, generator=g)).bfloat16().to(DEV)
    y = torch.randint(0, 4000, (96,), generator=g)
    y[::9] = -100
    y = y.to(DEV)
    s = (3 * torch.randn(24, 3000, generator=g)).bfloat16().to(DEV)
    t = (s.float() + 0.5 * torch.randn(24, 3000, generator=g).to(DEV)).bfloat16()

    def ce(x):
        return kernels.cross_entropy(x * 1.0, y) * 3.0

    def kl(x):
        return kernels.kl_div_logits(x * 1.0, t, temperature=2.0) * 0.5

    for fn, x0, kernel in ((ce, lg, "ce_loss_grad"), (kl, s, "kl_loss_grad")):
        xe = x0.clone().requires_grad_(True)
        le = fn(xe)
        le.backward()
        xc = x0.clone().requires_grad_(True)
        compiled = torch.compile(fn, backend="aot_eager", fullgraph=True)
        lc = compiled(xc)
        assert kernel in _hip.last_kernel(), _hip.last_kernel()      # the one-pass kernel ran in the compiled forward
        lc.backward()
        assert torch.equal(le, lc) and torch.equal(xe.grad, xc.grad)
        # a second compiled step (the graph is cached; the buffer of the first step was consumed, not reused)
        xc2 = x0.clone().requires_grad_(True)
        lc2 = compiled(xc2)
        lc2.backward()
        assert torch.equal(lc2, le) and torch.equal(xc2.grad, xe.grad)
    # one node per loss in the traced graph
    class M(nn.Module):
        def forward(self, x):
            return kernels.cross_entropy(x, y)
    ep = torch.export.export(M(), (lg.clone().requires_grad_(True),))
    targets = [str(n.target) for n in ep.graph.nodes if n.op == "call_function"]
    assert sum("forgemind.cross_entropy" in t_ for t_ in targets) == 1, targets
    # fp16 keeps the two-pass ops (the upstream gradient is applied in fp32 before the one rounding)
    lh = lg.half().clone().requires_grad_(True)
    out = torch.compile(lambda x: kernels.cross_entropy(x, y) * 1024.0, backend="aot_eager", fullgraph=True)(lh)
    fwd_kernel = _hip.last_kernel()          # (the backward runs on autograd's thread; this is the forward's)
    out.backward()
    assert "loss_grad" not in fwd_kernel and fwd_kernel.endswith("true, false>"), fwd_kernel   # loss only, no gradient
    lr = lg.half().clone().requires_grad_(True)
    (kernels.cross_entropy(lr, y) * 1024.0).backward()
    assert torch.equal(lr.grad, lh.grad)


def test_kl_autograd_reductions_and_temperature():
    g = torch.Generator().manual_seed(4)
    s = (3 * torch.randn(20, 3000, generator=g)).bfloat16()
    t = (s.float() + 0.5 * torch.randn(20, 3000, generator=g)).bfloat16()
    for red in ("mean", "sum", "none"):
        sd = s.to(DEV).requires_grad_(True)
        out = kernels.kl_div_logits(sd, t.to(DEV), red, temperature=2.0)
        ol, og = O.kl_div(s, t, red, 2.0)
        assert torch.allclose(out.cpu(), ol, rtol=1e-4, atol=1e-6)
        (out.sum() * 2.0).backward()
        assert close(sd.grad, og.float() * 2.0) and sd.grad.dtype == torch.bfloat16
    sd = s.to(DEV).requires_grad_(True)
    keep = sd.detach().clone()
    kernels.kl_div_logits(sd, t.to(DEV), grad_dtype=torch.float32).backward()
    assert torch.equal(sd.detach(), keep)                    # inputs are never written
    # distillation loop (reference tests/test_kernels.py:143-166)
    hs = torch.randn(16, 32, generator=g).to(DEV).requires_grad_(True)
    ht = torch.randn(16, 32, generator=g).to(DEV)
    w = torch.randn(200, 32, generator=g).to(DEV)
    wt = torch.randn(200, 32, generator=g).to(DEV).requires_grad_(True)
    loss = kernels.kl_distill_loss(hs, ht, w, lambda zz: zz @ wt.t(), chunk=5)
    loss.backward()
    ref, _ = O.kl_div((hs.detach() @ w.t()).cpu(), (ht @ wt.detach().t()).cpu(), "mean")
    assert loss.item() == pytest.approx(ref.item(), rel=1e-4) and wt.grad is None


def test_topk_softmax_surface_on_gpu():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 30, 5000, generator=g)
    xd = x.to(DEV).requires_grad_(True)
    v, idx = kernels.topk(xd, 12)
    ov, oi = O.topk(x, 12)
    assert idx.dtype == torch.int64 and torch.equal(idx.cpu(), oi) and torch.equal(v.detach().cpu(), ov)
    (v * 2).sum().backward()
    assert int((xd.grad != 0).sum()) == 2 * 30 * 12
    with pytest.raises(RuntimeError, match="selected index k out of range"):
        kernels.topk(xd, 5001)
    tv, ti = torch.topk(xd.detach(), 2, dim=0)
    v0, i0 = kernels.topk(xd.detach(), 2, dim=0)
    assert torch.equal(v0, tv) and torch.equal(i0, ti)
    kernels.reset_stats()
    kernels.topk(torch.randn(2, 2048, device=DEV), 600)       # k > 512: torch path, counted
    assert kernels.stats()["fallback"] == 1
    xs = torch.randn(4, 256, device=DEV, requires_grad=True)
    y = kernels.softmax(xs)
    gr = torch.randn(4, 256, device=DEV)
    y.backward(gr)
    xr = xs.detach().clone().requires_grad_(True)
    torch.softmax(xr, -1).backward(gr)
    assert torch.allclose(y, torch.softmax(xr, -1), rtol=1e-5, atol=1e-6)
    assert torch.allclose(xs.grad, xr.grad, rtol=1e-4, atol=1e-6)
    # bf16 attention-shaped input; an fp32 gradient arriving on a bf16 output takes tensor ops
    xb = torch.randn(2, 4, 128, 128, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    gb = torch.randn(2, 4, 128, 128, device=DEV, dtype=torch.bfloat16)
    kernels.softmax(xb).backward(gb)
    x32 = xb.detach().float().requires_grad_(True)
    torch.softmax(x32, -1).backward(gb.float())
    assert ((xb.grad.float() - x32.grad).abs().max() / x32.grad.abs().max()).item() < 1e-2
    xb.grad = None
    (kernels.softmax(xb).float() * gb.float()).sum().backward()
    assert ((xb.grad.float() - x32.grad).abs().max() / x32.grad.abs().max()).item() < 1e-2
    fn = torch.compile(lambda t: kernels.topk(kernels.softmax(t), 8)[0].sum(), fullgraph=True, backend="eager")
    fn(xs)                                                   # traces to aten, no graph break


def test_router_module_and_route_backward():
    g = torch.Generator().manual_seed(6)
    router = fm.moe.Router(64, 16, 2).to(DEV)
    x = torch.randn(300, 64, generator=g).to(DEV)
    w, idx, aux, z = router(x)
    logits = router.gate(x).float()
    oi, ow, oc, oslot, oorder = O.router(logits.detach().cpu(), 2)
    assert torch.equal(idx.cpu(), oi) and torch.allclose(w.cpu(), ow, rtol=1e-5)
    plan = router.last_plan
    assert torch.equal(plan.order.cpu(), oorder) and torch.equal(plan.counts.cpu(), oc)
    assert torch.equal(plan.offsets.cpu().long(), oc.cumsum(0))
    # gradient of the renormalised weights wrt the logits == autograd through the torch expression
    lg = logits.detach().clone().requires_grad_(True)
    r = kernels.moe_route(lg, 2)
    gw = torch.randn(300, 2, generator=g).to(DEV)
    r.weights.backward(gw)
    lr = logits.detach().clone().requires_grad_(True)
    p = lr.softmax(-1)
    pk = p.gather(1, r.idx.long())
    (pk / pk.sum(-1, keepdim=True)).backward(gw)
    assert torch.allclose(lg.grad, lr.grad, rtol=1e-4, atol=1e-7)
    (w.sum() + aux + z).backward()
    assert router.gate.weight.grad is not None
    # auxiliary losses and their gradients against the reference expression (moe.py:92-95)
    la = logits.detach().clone().requires_grad_(True)
    ra = kernels.moe_route(la, 2, with_aux=True)
    (3.0 * ra.aux + 0.5 * ra.z + (ra.weights * gw).sum()).backward()
    lb = logits.detach().clone().requires_grad_(True)
    pb = lb.softmax(-1)
    pkb = pb.gather(1, ra.idx.long())
    wb = pkb / pkb.sum(-1, keepdim=True)
    frac = ra.counts.float() / ra.idx.numel()
    aux_b = 16 * (frac * pb.mean(0)).sum()
    z_b = lb.logsumexp(-1).pow(2).mean()
    (3.0 * aux_b + 0.5 * z_b + (wb * gw).sum()).backward()
    assert ra.aux.item() == pytest.approx(aux_b.item(), rel=1e-5) and ra.z.item() == pytest.approx(z_b.item(), rel=1e-5)
    assert torch.allclose(la.grad, lb.grad, rtol=1e-4, atol=1e-7)


def test_modules_on_gpu():
    m = fm.nn.RMSNorm(256, eps=1e-5).to(DEV)
    ref = nn.RMSNorm(256, eps=1e-5).to(DEV)
    x = torch.randn(4, 9, 256, device=DEV, dtype=torch.bfloat16)
    kernels.reset_stats()
    y = m(x)                                  # fp32 parameter, bf16 activations: still the kernel
    assert kernels.stats()["fast"] == 1
    assert close(y, ref(x.float()).bfloat16())
    normed, res = m.forward_with_residual(x, x)
    assert torch.equal(res, x + x) and close(normed, ref((x + x).float()))
    net = nn.Sequential(nn.Linear(256, 256), nn.RMSNorm(256)).to(DEV)
    exp = net(x.float())
    kernels.enable(net)
    assert net._fm_fused["norm"] == 1 and torch.allclose(net(x.float()), exp, atol=1e-5, rtol=1e-5)
    kernels.revert(net)


def test_swiglu_module_on_gpu():
    """fm.nn.SwiGLU (reference nn.py:150-217): both parameter layouts run the packed kernels and
    agree with the eager expression, forward and backward."""
    torch.manual_seed(3)
    mlp = fm.nn.SwiGLU(256, hidden=640, dtype=torch.bfloat16, device=DEV)
    x = torch.randn(6, 11, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    kernels.reset_stats()
    y = mlp(x)
    assert kernels.stats()["fast"] == 1 and kernels.stats()["fallback"] == 0
    xr = x.detach().clone().requires_grad_(True)
    ref = mlp.w2(F.silu(mlp.w1(xr)) * mlp.w3(xr))
    assert close(y, ref)
    g = torch.randn_like(y)
    y.backward(g)
    gw1 = mlp.w1.weight.grad.clone()
    mlp.zero_grad()
    ref.backward(g)
    assert close(x.grad, xr.grad) and close(gw1, mlp.w1.weight.grad)
    stacked = mlp.to_split(inplace=False)
    assert not hasattr(stacked, "w1") and hasattr(mlp, "w1") and stacked.gate_up.weight.shape == (1280, 256)
    kernels.reset_stats()
    ys = stacked(x.detach())
    assert kernels.stats()["fast"] == 1 and close(ys, y)


def test_launches_are_graph_capturable():
    """No allocation, no sync, no memset node inside the library: a captured fwd+bwd replays
    to the same bits as the eager launches, replay after replay."""
    n, d = 512, 1024
    x = torch.randn(n, d, device=DEV).bfloat16()
    w = torch.randn(d, device=DEV)
    dy = torch.randn(n, d, device=DEV).bfloat16()
    y, rstd = torch.empty_like(x), torch.empty(n, device=DEV)
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    L = _hip.lib()
    nb = L.fm_rmsnorm_bwd_workspace(n, d, _hip.BF16)
    ws = torch.empty(nb, device=DEV, dtype=torch.uint8)

    def launch(stream):
        assert L.fm_rmsnorm_fwd(x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), n, d,
                                _hip.BF16, _hip.F32, 1e-6, stream) == 0
        assert L.fm_rmsnorm_bwd(x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dy.data_ptr(),
                                dx.data_ptr(), dw.data_ptr(), ws.data_ptr(), nb, n, d, _hip.BF16,
                                _hip.F32, stream) == 0

    launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    ref = [t.clone() for t in (y, dx, dw)]
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(side.cuda_stream)                         # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            launch(side.cuda_stream)
    for _ in range(3):
        for t in (y, dx, dw):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip((y, dx, dw), ref))


def test_loss_selection_and_routing_launches_replay_in_a_graph():
    """The rest of the library under capture (outputs come from the graph's own pool): every
    replay gives the bits of the eager call, with eager work and synchronisations in between."""
    g = torch.Generator().manual_seed(77)
    lg = (2 * torch.randn(300, 4096, generator=g)).bfloat16().to(DEV)
    narrow = torch.randn(700, 100, generator=g).to(DEV)
    y = torch.randint(0, 4096, (300,), generator=g).to(DEV)
    y[::7] = -100
    yn = torch.randint(0, 100, (700,), generator=g).to(DEV)
    s_, t_ = lg, (lg.float() + 0.5 * torch.randn(300, 4096, generator=g).to(DEV)).bfloat16()
    wide = (3 * torch.randn(8, 128256, generator=g)).bfloat16().to(DEV)
    wide2 = (wide.float() + 0.5 * torch.randn(8, 128256, generator=g).to(DEV)).bfloat16()
    mid = (3 * torch.randn(900, 20000, generator=g)).bfloat16().to(DEV)
    mid2 = (mid.float() + 0.5 * torch.randn(900, 20000, generator=g).to(DEV)).bfloat16()
    short = torch.randn(500, 1000, generator=g).to(DEV)
    logits = torch.randn(2048, 64, generator=g).to(DEV)
    xs = torch.randn(2048, 512, generator=g).bfloat16().to(DEV)
    aligned = torch.randn(700, 512, generator=g).bfloat16().to(DEV)
    aligned2 = torch.randn(700, 512, generator=g).bfloat16().to(DEV)
    ya = torch.randint(0, 512, (700,), generator=g).to(DEV)
    huge = (3 * torch.randn(2, 262144, generator=g)).bfloat16().to(DEV)      # prefixes past 64 KB of LDS
    logits256 = torch.randn(600, 256, generator=g).to(DEV)
    xw = torch.randn(300, 18432, generator=g).bfloat16().to(DEV)             # backward just past the register path
    ww = torch.randn(18432, generator=g).to(DEV)

    def step():
        out = []
        out += list(_hip.topk(huge, 64, torch.int32))
        out += list(_hip.route(logits256, 8, True, True))                    # picks from lane-sorted keys
        yw, rw = _hip.rmsnorm_fwd(xw, ww, 1e-6)
        out += [yw, rw] + list(_hip.rmsnorm_bwd(xw, ww, rw, xw))
        loss, dl, nv, rows = _hip.ce_loss_grad(lg, y, -100, "mean")
        out += [loss, dl, nv, rows]
        loss2, lse, nv2, rows2 = _hip.ce_fwd(narrow, yn, -100, "mean")
        out += [loss2, lse, _hip.ce_bwd(narrow, yn, lse, nv2, None, -100)]
        kl, rkl, ls, lt = _hip.kl_fwd(s_, t_, 0.5, "mean")
        out += [kl, rkl, _hip.kl_bwd(s_, t_, ls, lt, None, False, torch.bfloat16, 0.5, 1.0 / 300)]
        out += [t for t in _hip.kl_fwd_topk(wide, wide, 64, 1.0, "mean", torch.int32) if t is not None]
        out += list(_hip.topk(wide, 64, torch.int32)) + list(_hip.topk(short, 8, torch.int64))
        out += list(_hip.topk(short, 300, torch.int32))
        sm = _hip.softmax_fwd(short)
        out += [sm, _hip.softmax_bwd(sm, short)]
        idx, wts, counts, slot, order, stats = _hip.route(logits, 2, True, True)
        gathered = _hip.moe_gather(xs, order, 2)
        out += [idx, wts, counts, slot, order, stats, gathered, _hip.moe_combine(gathered, wts, slot, 2048, 2)]
        out += [_hip.route_bwd(logits, idx, wts, counts, stats[65], stats[66])]
        # the lane-group forms: narrow top-k, rows of whole vectors in the loss kernels, and the
        # two-wave top-k of rows of a few thousand elements
        out += list(_hip.topk(logits, 2, torch.int32)) + list(_hip.topk(lg, 8, torch.int32))
        l3, d3, _, r3 = _hip.ce_loss_grad(aligned, ya, -100, "mean")
        k3, g3, rk3 = _hip.kl_loss_grad(aligned, aligned2, 1.0, "mean", torch.bfloat16)
        out += [l3, d3, r3, k3, g3, rk3]
        # rows kept on the chip by workgroups that walk several rows (one and three per compute unit)
        out += list(_hip.kl_loss_grad(wide, wide2, 0.5, "mean", torch.bfloat16))
        out += list(_hip.kl_loss_grad(mid, mid2, 1.0, "sum", torch.bfloat16))
        out += [_hip.swiglu_split_fwd(xs), _hip.swiglu_split_bwd(xs, xs[:, :256].contiguous())]
        return out

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                           # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = step()
    for _ in range(3):
        for t in outs:
            t.zero_()
        _hip.softmax_fwd(short)                          # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, eager):
            assert torch.equal(a, b)


@pytest.mark.parametrize("e,k", [(8, 2), (32, 10)])
def test_moe_layer_matches_the_reference_expression(e, k):
    """MoE.forward of forgemind/moe.py:227-251 written with aten ops vs the fused pipeline (also
    with more than eight experts a token: no step of the layer leaves the library)."""
    g = torch.Generator().manual_seed(7)
    n, d, h = 300, 64, 128
    layer = fm.moe.MoE(d, h, e, k).to(DEV)
    x = torch.randn(n, d, generator=g).to(DEV).requires_grad_(True)
    kernels.reset_stats()
    out = layer(x)
    assert kernels.stats()["fallback"] == 0
    out.square().sum().backward()
    gx = x.grad.clone()
    gate_g = layer.router.gate.weight.grad.clone()

    # reference expression, same parameters
    xr = x.detach().clone().requires_grad_(True)
    layer.zero_grad()
    logits = layer.router.gate(xr).float()
    probs = logits.softmax(-1)
    w, idx = probs.topk(k, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    flat = idx.reshape(-1)
    order = torch.sort(flat, stable=True).indices
    tok = order // k
    xs = xr[tok]
    counts = torch.bincount(flat, minlength=e).tolist()
    ys = layer.experts(xs, counts)
    ys = ys * w.reshape(-1)[order].unsqueeze(-1)
    ref = torch.zeros_like(xr).index_add_(0, tok, ys.to(xr.dtype))
    ref.square().sum().backward()
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5)
    # the reference side sums with atomics (index_add_), so its own last bits move from run to run:
    # tolerances are relative to each tensor's scale
    assert torch.allclose(gx, xr.grad, rtol=1e-3, atol=1e-4 * float(xr.grad.abs().max()))
    gw = layer.router.gate.weight.grad
    assert torch.allclose(gate_g, gw, rtol=1e-3, atol=1e-4 * float(gw.abs().max()))


def test_qk_norm_rope_surface_and_op_path():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 9, 4, 64, generator=g).to(DEV)
    w = torch.randn(64, generator=g).to(DEV)
    cos, sin = torch.randn(9, 32, generator=g).to(DEV), torch.randn(9, 32, generator=g).to(DEV)

    def run(mode):
        _ops.use_custom_ops(mode)
        xi, wi = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        out = kernels.qk_norm_rope(xi, wi, cos, sin, 1e-6)
        out.square().sum().backward()
        return out.detach(), xi.grad, wi.grad

    eager, op = run(False), run(True)
    assert all(torch.equal(a, b) for a, b in zip(eager, op))
    kernels.set_backend("fallback")
    ref = run(False)
    kernels.set_backend("auto")
    assert all(torch.allclose(a, b, rtol=1e-4, atol=1e-4) for a, b in zip(eager, ref))
    with pytest.raises(ValueError):
        kernels.qk_norm_rope(x[0], w, cos, sin)
    # a broadcast-shaped table and a longer one give the bits of the [T, D/2] call
    base = kernels.qk_norm_rope(x, w, cos, sin)
    assert torch.equal(kernels.qk_norm_rope(x, w, cos.view(1, 9, 1, 32), sin.view(1, 9, 1, 32)), base)
    pad = torch.randn(7, 32, device=DEV)
    assert torch.equal(kernels.qk_norm_rope(x, w, torch.cat((cos, pad)), torch.cat((sin, pad))), base)


def test_kl_div_logits_topk_autograd_and_wide_rows():
    g = torch.Generator().manual_seed(77)
    s = (3 * torch.randn(6, 5000, generator=g)).bfloat16()
    t = (s.float() + 0.5 * torch.randn(6, 5000, generator=g)).bfloat16()
    sd = s.to("cuda").requires_grad_(True)
    loss, probs, idx = kernels.kl_div_logits_topk(sd, t.to("cuda"), 16, temperature=2.0, index_dtype=torch.int32)
    loss.backward()
    sr = s.to("cuda").requires_grad_(True)
    ref = kernels.kl_div_logits(sr, t.to("cuda"), temperature=2.0)
    ref.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=1e-4)     # two kernels, two summation orders
    assert torch.allclose(sd.grad.float(), sr.grad.float(), rtol=1e-2, atol=1e-9)
    assert not probs.requires_grad and idx.dtype == torch.int32
    assert torch.equal(idx.cpu().long(), O.topk(t, 16)[1])
    # a row wider than the fused kernel takes goes through the two kernels, same results
    s = torch.randn(1, 66561 * 4 + 40, generator=g)
    t = torch.randn(1, 66561 * 4 + 40, generator=g)
    loss, probs, idx = kernels.kl_div_logits_topk(s.to("cuda"), t.to("cuda"), 8, reduction="sum")
    assert torch.equal(idx.cpu(), O.topk(t, 8)[1])
    want = torch.gather(torch.softmax(t.double(), -1), -1, idx.cpu())
    assert torch.allclose(probs.cpu().double(), want, rtol=1e-4)
    assert loss.item() == pytest.approx(O.kl_div(s, t, "sum", 1.0, acc=torch.float64)[0].item(), rel=1e-4)
    with pytest.raises(RuntimeError):
        kernels.kl_div_logits_topk(s.to("cuda"), t.to("cuda"), 0)


def test_layer_norm_autograd_module_and_op_path():
    g = torch.Generator().manual_seed(51)
    x = (0.5 + torch.randn(4, 50, 768, generator=g)).bfloat16()
    w, b = 1 + 0.02 * torch.randn(768, generator=g), 0.1 * torch.randn(768, generator=g)
    dy = torch.randn(4, 50, 768, generator=g).bfloat16()
    odx, odw, odb = O.layer_norm_bwd(x, w, dy, 1e-5)
    xd = x.to(DEV).requires_grad_(True)
    wd, bd = w.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True)
    kernels.reset_stats()
    y = kernels.layer_norm(xd, wd, bd, 1e-5)
    y.backward(dy.to(DEV))
    assert kernels.stats()["fast"] == 1 and kernels.stats()["fallback"] == 0
    assert close(y, O.layer_norm(x, w, b, 1e-5)[0]) and close(xd.grad, odx)
    assert close(wd.grad, odw, 1e-3) and close(bd.grad, odb, 1e-3)
    # the op path gives the same bits as the eager path
    x2 = x.to(DEV).requires_grad_(True)
    _ops.use_custom_ops(True)
    y2 = kernels.layer_norm(x2, wd.detach(), bd.detach(), 1e-5)
    y2.backward(dy.to(DEV))
    _ops.use_custom_ops(None)
    assert torch.equal(y2, y) and torch.equal(x2.grad, xd.grad)
    # residual form through the module, against torch.nn.LayerNorm
    m = fm.nn.LayerNorm(768).to(DEV)
    ref = nn.LayerNorm(768).to(DEV)
    with torch.no_grad():
        m.weight.copy_(w); m.bias.copy_(b); ref.weight.copy_(w); ref.bias.copy_(b)
    h = torch.randn(6, 768, device=DEV, requires_grad=True)
    r = torch.randn(6, 768, device=DEV)
    normed, res = m.forward_with_residual(h, r)
    (normed.sum() + res.sum()).backward()
    h2 = h.detach().clone().requires_grad_(True)
    s2 = h2 + r
    (ref(s2).sum() + s2.sum()).backward()
    assert torch.equal(res, h.detach() + r) and torch.allclose(normed, ref(h.detach() + r), atol=1e-5)
    assert torch.allclose(h.grad, h2.grad, atol=1e-4) and torch.allclose(m.bias.grad, ref.bias.grad, atol=1e-5)
    assert torch.allclose(m.weight.grad, ref.weight.grad, atol=1e-4)
    fn = torch.compile(lambda t: kernels.layer_norm(t, wd.detach(), bd.detach()).float().sum(), fullgraph=True,
                       backend="eager")
    assert torch.isfinite(fn(x.to(DEV)))


def test_losses_and_moe_pieces_trace_in_one_graph():
    g = torch.Generator().manual_seed(61)
    lg = (2 * torch.randn(40, 700, generator=g)).bfloat16().to(DEV)
    lab = torch.randint(0, 700, (40,), generator=g).to(DEV)
    lab[::9] = -100
    t = (lg.float() + 0.5 * torch.randn(40, 700, generator=g).to(DEV)).bfloat16()
    for name in ("cross_entropy", "cross_entropy_backward", "kl_div", "kl_div_backward"):
        assert hasattr(torch.ops.forgemind, name), name

    def both(fn):
        a = lg.clone().requires_grad_(True)
        out = fn(a)
        out.sum().backward()
        b = lg.clone().requires_grad_(True)
        cout = torch.compile(fn, fullgraph=True, backend="eager")(b)
        cout.sum().backward()
        assert torch.allclose(out, cout, rtol=1e-5, atol=1e-7)
        assert close(b.grad, a.grad)
    both(lambda a: kernels.cross_entropy(a, lab))
    both(lambda a: kernels.cross_entropy(a, lab, reduction="sum"))
    both(lambda a: kernels.kl_div_logits(a, t, temperature=2.0))
    both(lambda a: kernels.kl_div_logits(a, t, "none"))
    both(lambda a: kernels.kl_div_logits_topk(a, t, 8)[0])
    # the exported graph keeps the loss as one node
    class M(nn.Module):
        def forward(self, a):
            return kernels.cross_entropy(a, lab)
    ep = torch.export.export(M(), (lg,))
    targets = [str(n.target) for n in ep.graph.nodes if n.op == "call_function"]
    assert "forgemind.cross_entropy.default" in targets, targets
    # router and token moves: the traced graph gets the tensor expression, same results
    rl = torch.round(torch.randn(200, 16, generator=g) * 64).to(DEV) / 64
    x = torch.randn(200, 64, generator=g).to(DEV)

    def moe(a):
        r = kernels.moe_route(rl, 2)
        xs = kernels.moe_gather(a, r.order, 2, r.slot)
        return kernels.moe_combine(xs, r.weights, r.slot, r.order)
    eager = moe(x)
    traced = torch.compile(moe, fullgraph=True, backend="eager")(x)
    assert torch.allclose(eager, traced, rtol=1e-5, atol=1e-6)

"""fm_rmsnorm_bwd_static, the entry point that allocates nothing, through the C ABI: its dx and
dw must equal fm_rmsnorm_bwd's bit for bit (same kernels, the partial weight gradients in the
library's built-in buffer instead of a caller's workspace), on two calls in a row that share the
buffer, the second on a smaller input, and both must agree with the CPU oracle.
"""

import pytest
import torch

from forgeminds_amd.kernels import _hip
from oracle import oracle as O

pytestmark = pytest.mark.gpu

CASES = [
    # (first call, second call): (rows, width); the second is smaller in rows, width or both
    ((8192, 1024), (1000, 1024)),
    ((2048, 8192), (300, 4096)),
    ((4096, 1000), (64, 96)),        # widths off the 16-byte grid take the any-width kernels
]


def _inputs(n, d, dtype, wdtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, d, generator=g).to(dtype)
    w = (1 + 0.02 * torch.randn(d, generator=g)).to(wdtype)
    dy = torch.randn(n, d, generator=g).to(dtype)
    return x, w, dy


def _both(lib, x, w, dy, eps=1e-6):
    dev = "cuda:0"
    xd, wd, dyd = x.to(dev), w.to(dev), dy.to(dev)
    n, d = xd.shape
    xdt, wdt = _hip.dtype_code(xd.dtype), _hip.dtype_code(wd.dtype)
    y = torch.empty_like(xd)
    rstd = torch.empty(n, device=dev, dtype=torch.float32)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.fm_rmsnorm_fwd(xd.data_ptr(), wd.data_ptr(), y.data_ptr(), rstd.data_ptr(), n, d, xdt, wdt,
                              eps, st) == 0
    nbytes = int(lib.fm_rmsnorm_bwd_workspace(n, d, xdt))
    ws = torch.empty(max(nbytes, 16), device=dev, dtype=torch.uint8)
    dx_a, dw_a = torch.empty_like(xd), torch.empty_like(wd)
    rc = lib.fm_rmsnorm_bwd(xd.data_ptr(), wd.data_ptr(), rstd.data_ptr(), dyd.data_ptr(), dx_a.data_ptr(),
                            dw_a.data_ptr(), ws.data_ptr(), nbytes, n, d, xdt, wdt, st)
    assert rc == 0, lib.fm_last_error()
    # poisoned outputs: whatever the call does not write shows up in the comparison
    dx_b = torch.full_like(xd, float("nan"))
    dw_b = torch.full_like(wd, float("nan"))
    rc = lib.fm_rmsnorm_bwd_static(xd.data_ptr(), wd.data_ptr(), rstd.data_ptr(), dyd.data_ptr(),
                                   dx_b.data_ptr(), dw_b.data_ptr(), n, d, xdt, wdt, st)
    assert rc == 0, lib.fm_last_error()
    torch.cuda.synchronize()
    return (dx_a, dw_a), (dx_b, dw_b)


@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.float32), (torch.float32, torch.float32),
                                          (torch.float16, torch.float16)])
@pytest.mark.parametrize("first,second", CASES)
def test_static_scratch_backward_matches_the_workspace_form(first, second, dtype, wdtype):
    lib = _hip.lib()
    for i, (n, d) in enumerate((first, second)):      # the second call re-uses the buffer the first left
        x, w, dy = _inputs(n, d, dtype, wdtype, seed=7 + i)
        (dx_a, dw_a), (dx_b, dw_b) = _both(lib, x, w, dy)
        assert torch.equal(dx_a, dx_b), (n, d)
        assert torch.equal(dw_a, dw_b), (n, d)
        odx, odw = O.rms_norm_bwd(x, w, dy)
        tol = 1e-2 if dtype != torch.float32 else 1e-4
        assert (dx_b.float().cpu() - odx.float()).abs().max() <= tol * odx.float().abs().max()
        assert (dw_b.float().cpu() - odw.float()).abs().max() <= tol * odw.float().abs().max()


def test_static_scratch_backward_without_weight_gradient_and_empty_batch():
    lib = _hip.lib()
    x, w, dy = _inputs(512, 2048, torch.bfloat16, torch.float32, seed=3)
    dev = "cuda:0"
    xd, wd, dyd = x.to(dev), w.to(dev), dy.to(dev)
    rstd = torch.rsqrt(xd.float().pow(2).mean(-1) + 1e-6)
    st = torch.cuda.current_stream().cuda_stream
    dx = torch.full_like(xd, float("nan"))
    assert lib.fm_rmsnorm_bwd_static(xd.data_ptr(), wd.data_ptr(), rstd.data_ptr(), dyd.data_ptr(),
                                     dx.data_ptr(), None, 512, 2048, _hip.BF16, _hip.F32, st) == 0
    ref = torch.empty_like(xd)
    assert lib.fm_rmsnorm_bwd(xd.data_ptr(), wd.data_ptr(), rstd.data_ptr(), dyd.data_ptr(), ref.data_ptr(),
                              None, None, 0, 512, 2048, _hip.BF16, _hip.F32, st) == 0
    dw = torch.full_like(wd, float("nan"))
    assert lib.fm_rmsnorm_bwd_static(None, wd.data_ptr(), None, None, None, dw.data_ptr(), 0, 2048, _hip.BF16,
                                     _hip.F32, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(dx, ref)
    assert torch.count_nonzero(dw).item() == 0


def test_static_scratch_backward_rejects_shapes_past_its_buffer():
    lib = _hip.lib()
    # 256 partial rows of 16384 floats = 16 MiB > the 8 MiB the library holds: refused before any launch
    assert lib.fm_rmsnorm_bwd_static(None, None, None, None, None, 1, 4096, 16384, _hip.BF16, _hip.F32, None) == 2
    assert b"built-in buffer" in lib.fm_last_error()


def test_static_scratch_limit_follows_the_backward_grid():
    # the buffer holds (partial rows) x d x 4 bytes and there is one partial row per workgroup of the
    # persistent grid: with two workgroups per compute unit a [4096, 8192] problem needs twice the
    # bytes and is refused, where the default grid fits exactly
    lib = _hip.lib()
    n, d = 4096, 8192
    limit = 8 << 20
    try:
        need1 = int(lib.fm_rmsnorm_bwd_workspace(n, d, _hip.BF16))
        _hip.set_param("norm_bwd_blocks_per_cu", 2)
        need2 = int(lib.fm_rmsnorm_bwd_workspace(n, d, _hip.BF16))
        assert need2 == 2 * need1
        rc = lib.fm_rmsnorm_bwd_static(None, None, None, None, None, 1, n, d, _hip.BF16, _hip.F32, None)
        assert (rc == 2) == (need2 > limit), (need1, need2)
        if need2 > limit:
            assert b"built-in buffer" in lib.fm_last_error()
    finally:
        _hip.set_param("norm_bwd_blocks_per_cu", 0)
    assert need1 <= limit

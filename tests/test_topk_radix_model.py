"""CPU model of the radix selection the top-k kernels fall back to when a row has long runs of
equal values at its k-th place (forgeminds_amd/csrc/fm_topk.hip.h, exact path of wide rows):
order-preserving 32-bit keys, eight key bits per sweep from the top, per sweep a 256-bin count
of the elements that match the prefix so far, the bin of the k-th largest from suffix sums; then
everything above the k-th key plus the first ties in ascending column order. Checked against
the oracle's lexicographic sort (canonical order of forgemind/kernels/topk.py:13-19) on the
rows that drive the kernel into that path: all-equal, two-valued, fifty-valued, NaN and zero runs.
"""

import numpy as np
import pytest
import torch

from oracle import oracle as O

MASK = {torch.bfloat16: (0xFFFF0000, 16), torch.float16: (0xFFFFE000, 13), torch.float32: (0xFFFFFFFF, 0)}


def keys_of(row: torch.Tensor) -> np.ndarray:
    f = row.float().numpy().copy()
    f = f + np.float32(0.0)                               # -0.0 -> +0.0
    b = f.view(np.uint32).astype(np.uint64)
    neg = (b >> 31) & 1
    key = np.where(neg == 1, b ^ 0xFFFFFFFF, b ^ 0x80000000)
    key = np.where(np.isnan(f), 0xFFFFFFFF, key)
    return key.astype(np.uint64)


def radix_topk(row: torch.Tensor, k: int):
    mask, low = MASK[row.dtype]
    key = keys_of(row) & mask
    prefix, pmask, kk = 0, 0, k
    shift = 24
    while shift + 8 > low:
        ok = (key & pmask) == prefix
        hist = np.bincount(((key[ok] >> shift) & 255).astype(np.int64), minlength=256)
        above = 0
        for b in range(255, -1, -1):
            if above < kk <= above + hist[b]:
                break
            above += hist[b]
        else:  # pragma: no cover
            raise AssertionError("no bin holds the k-th element")
        prefix |= b << shift
        pmask |= 255 << shift
        kk -= above
        shift -= 8
    kth, c_gt, need = prefix, k - kk, kk
    cols = np.arange(key.size)
    taken = np.concatenate([cols[key > kth], cols[key == kth][:need]])
    assert (key > kth).sum() == c_gt and taken.size == k
    full = keys_of(row)                                    # final order on the whole key, then column
    order = np.lexsort((taken, -full[taken].astype(np.float64)))
    # lexsort on float64 of a uint32 key is exact (32 bits fit the mantissa)
    return taken[order]


CASES = []
for dt in (torch.bfloat16, torch.float16, torch.float32):
    CASES += [(dt, "all_equal"), (dt, "two_valued"), (dt, "fifty_valued"), (dt, "nan_and_zero_runs"), (dt, "random")]


@pytest.mark.parametrize("dtype,kind", CASES)
def test_radix_selection_matches_the_lexicographic_sort(dtype, kind):
    g = torch.Generator().manual_seed(hash((str(dtype), kind)) % 10000)
    n = 5000
    if kind == "all_equal":
        x = torch.full((n,), 1.25)
    elif kind == "two_valued":
        x = torch.where(torch.rand(n, generator=g) < 0.5, torch.tensor(-0.75), torch.tensor(3.5))
    elif kind == "fifty_valued":
        x = torch.randn(50, generator=g)[torch.randint(0, 50, (n,), generator=g)]
    elif kind == "nan_and_zero_runs":
        x = torch.randn(n, generator=g)
        x[torch.rand(n, generator=g) < 0.3] = 0.0
        x[torch.rand(n, generator=g) < 0.2] = -0.0
        x[torch.rand(n, generator=g) < 0.01] = float("nan")
        x[torch.rand(n, generator=g) < 0.01] = float("inf")
        x[torch.rand(n, generator=g) < 0.01] = float("-inf")
    else:
        x = torch.randn(n, generator=g) * 3
    x = x.to(dtype)
    for k in (1, 7, 64, 512, n):
        got = radix_topk(x, k)
        want = O.topk(x.view(1, -1), k)[1][0].numpy()
        assert np.array_equal(got, want), (dtype, kind, k)

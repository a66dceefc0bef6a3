"""The entry point that allocates nothing, nq_hinv_upper_f64_dev, through the C ABI against the entry point it is a
variant of (nq_hinv_upper_f64: same kernels, so the same bits), twice in a row with the second matrix smaller:
the library's fixed scratch keeps the first call's contents, and nothing of them may leak into the second."""
import numpy as np
import pytest
import torch

from noeira_amd import _lib as L
from noeira_amd.gptq import hinv_upper_f64, hinv_upper_f64_dev

pytestmark = pytest.mark.gpu

INT32_MAX = 0x7FFFFFFF


def spd(rng, n):
    a = rng.standard_normal((n, 2 * n))
    return a @ a.T / (2 * n) + 0.05 * np.eye(n)


def test_no_alloc_matches_the_allocating_entry_point_twice():
    rng = np.random.default_rng(5)
    for n in (200, 72):  # the second call is smaller: the scratch still holds the first one's factor
        h = spd(rng, n)
        want = hinv_upper_f64(h)
        hd = torch.from_numpy(h).cuda()
        u = torch.full((n, n), float("nan"), dtype=torch.float64, device="cuda")
        pivot = torch.full((1,), -7, dtype=torch.int32, device="cuda")
        hinv_upper_f64_dev(hd, u, pivot)
        torch.cuda.synchronize()
        assert int(pivot.item()) == INT32_MAX
        assert np.array_equal(u.cpu().numpy().view(np.uint64), want.view(np.uint64)), n
        assert torch.equal(hd.cpu(), torch.from_numpy(h)), "h was modified"


def test_no_alloc_reports_the_pivot_and_the_limit():
    bad = torch.tensor([[1.0, 2.0], [2.0, 1.0]], dtype=torch.float64, device="cuda")
    _, pivot = hinv_upper_f64_dev(bad)
    torch.cuda.synchronize()
    assert 0 <= int(pivot.item()) < 2
    with pytest.raises(L.NQError, match="exceeds the 1024"):
        hinv_upper_f64_dev(torch.eye(1025, dtype=torch.float64, device="cuda"))
    # the largest size the scratch holds
    rng = np.random.default_rng(6)
    h = spd(rng, 1024)
    u, pivot = hinv_upper_f64_dev(torch.from_numpy(h).cuda())
    torch.cuda.synchronize()
    assert int(pivot.item()) == INT32_MAX
    assert np.array_equal(u.cpu().numpy().view(np.uint64), hinv_upper_f64(h).view(np.uint64))

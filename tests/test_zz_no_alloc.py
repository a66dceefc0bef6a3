"""The entry point that allocates nothing, nq_hinv_upper_f64_dev, through the C ABI against the entry point it is a
variant of (nq_hinv_upper_f64: same kernels, so the same bits), twice in a row with the second matrix smaller:
the library's fixed scratch keeps the first call's contents, and nothing of them may leak into the second.  Also
what the entry point is for: the device's free memory is the same before and after a call, and a call recorded
into a device graph replays over changed inputs with the eager call's bits.  The limit case n = 1024 is held
against the CPU oracle's factorization, not only against the sibling entry point."""
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


def test_no_alloc_allocates_nothing_and_can_be_captured():
    """What the entry point exists for.  (1) hipMemGetInfo reads the same free bytes before and after calls (torch's
    caching allocator is out of the picture: inputs and outputs exist before the first reading).  (2) A call is
    recorded into a device graph once and replayed over changed matrices, with eager calls and synchronisations in
    between; every replay returns the eager call's bits."""
    rng = np.random.default_rng(9)
    n = 160
    hs = [torch.from_numpy(spd(rng, n)).cuda() for _ in range(4)]
    hd = hs[0].clone()
    u = torch.empty((n, n), dtype=torch.float64, device="cuda")
    pivot = torch.empty((1,), dtype=torch.int32, device="cuda")
    hinv_upper_f64_dev(hd, u, pivot)  # (first call on this device: any one-time set-up is behind us)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        hinv_upper_f64_dev(hd, u, pivot)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    # ---- capture once, replay over changed h
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        hinv_upper_f64_dev(hd, u, pivot)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        hinv_upper_f64_dev(hd, u, pivot)
    for h in hs:
        want_u, want_p = hinv_upper_f64_dev(h.clone())  # eager, its own output
        torch.cuda.synchronize()
        hd.copy_(h)
        u.fill_(float("nan"))
        pivot.fill_(-3)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(u.view(torch.int64), want_u.view(torch.int64))
        assert int(pivot.item()) == int(want_p.item()) == INT32_MAX


def test_no_alloc_limit_case_against_the_oracle():
    """n = 1024, the largest matrix the scratch holds, against the CPU oracle's `hinv_upper_f64` (dense.mojo:1-30
    restated: Cholesky of the index-reversed matrix, triangular inverse, reversed back), within fp64 round-off of
    the factor's largest entry (the device blocks the factorization by 64, so sums meet in another order than the
    oracle's at this size); U^T U = H^-1 is checked on top."""
    from oracle import oracle as O

    rng = np.random.default_rng(6)
    h = spd(rng, 1024)
    u, pivot = hinv_upper_f64_dev(torch.from_numpy(h).cuda())
    torch.cuda.synchronize()
    assert int(pivot.item()) == INT32_MAX
    got = u.cpu().numpy()
    want = O.hinv_upper_f64(h)
    assert np.abs(got - want).max() <= 1e-10 * np.abs(want).max()
    assert np.abs(np.tril(got, -1)).max() == 0.0
    assert np.abs(got.T @ got @ h - np.eye(1024)).max() < 1e-8

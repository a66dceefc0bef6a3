"""GPTQ onto the Q4_0 grid on the GPU, through the C ABI, against the CPU oracle
and the reference's fixture.

Gates as the reference's tests/nn/quant/test_gptq.mojo [1]-[5] and
test_cholesky.mojo.  The device code runs every sum in the order the oracle
states, so beyond the reference's own gates (objective within 1 %, >= 90 % of
rows identical) the codes, scales and the factor U are compared bit for bit.
"""
import os

import numpy as np
import pytest
import torch

from noeira_amd import _lib as L
from noeira_amd.gptq import HessianAccumulator, gptq_q4_0, hinv_upper_f64, q4_0_objective, set_weight_gptq
from noeira_amd.qlinear import QLinear
from noeira_amd.safetensors_io import SafeTensors
from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fix(golden_dir):
    f = SafeTensors(os.path.join(golden_dir, "gptq_q4_0.safetensors"))
    return {c: dict(w=f.read_f32(c + ".w"), h=f.read_f32(c + ".h"), q=f.read(c + ".q"), d=f.read_f32(c + ".d"),
                    obj=f.read_f32(c + ".obj")) for c in "ab"}


def spd(rng, n, cond=1e4):
    x = rng.standard_normal((3 * n, n)) * np.geomspace(1.0, np.sqrt(cond), n)[rng.permutation(n)]
    return x.T @ x + 1e-3 * np.eye(n)


def f16bits(d):
    return np.asarray(d, np.float32).astype(np.float16).view(np.uint16)


# ── the factor of H^-1 (test_cholesky.mojo; dense.mojo:355-363) ────────────
@pytest.mark.parametrize("n", [1, 2, 7, 63, 64, 65, 160, 300, 384])
def test_hinv_upper_matches_oracle_and_numpy(n):
    rng = np.random.default_rng(n)
    a = spd(rng, n)
    u = hinv_upper_f64(a)
    assert np.array_equal(np.tril(u, -1), np.zeros_like(u)) and (np.diag(u) > 0).all()
    assert np.abs(u.T @ u @ a - np.eye(n)).max() < 1e-7
    want = np.linalg.cholesky(np.linalg.inv(a)).T
    assert np.abs(u - want).max() <= 1e-8 * np.abs(want).max()
    assert np.array_equal(u.view(np.uint64), O.hinv_upper_f64(a).view(np.uint64)), "differs from the oracle's bits"


def test_hinv_upper_rejects_indefinite():
    with pytest.raises(L.NQError, match="not positive definite"):
        hinv_upper_f64(np.array([[1.0, 2.0], [2.0, 1.0]]))


# ── the calibration Hessian (hessian.mojo:41-77) ───────────────────────────
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hessian_accumulator(dtype):
    rng = np.random.default_rng(4)
    n = 200
    x = torch.from_numpy(rng.standard_normal((333, n)).astype(np.float32)).to(dtype)
    x[:, 17] = 0
    acc = HessianAccumulator(n)
    acc.add(x[:100].contiguous().cuda())
    acc.add(x[100:].contiguous().cuda(), rows=200)   # the first 200 rows of the slab only
    assert acc.rows == 300
    want = np.zeros((n, n))
    xf = x.float().numpy()
    O.hessian_add(want, xf[:100])
    O.hessian_add(want, xf[100:300])
    got = acc.h
    assert np.array_equal(got.view(np.uint64), want.view(np.uint64))
    assert got[17, 17] == 0
    ref = xf[:300].astype(np.float64).T @ xf[:300].astype(np.float64)
    assert np.abs(got - ref).max() <= 1e-12 * np.abs(ref).max()
    with pytest.raises(L.NQError, match="the slab holds"):
        acc.add(x[:10].contiguous().cuda(), rows=11)


# ── [1] parity with the reference's fixture (test_gptq.mojo:47-82) ─────────
@pytest.mark.parametrize("case", ["a", "b"])
def test_gptq_parity_with_reference_fixture(fix, case):
    c = fix[case]
    w, h = c["w"], c["h"].astype(np.float64)
    n, k = w.shape
    q, d, st = gptq_q4_0(w, n, k, h)
    assert st.dead == {"a": 3, "b": 2}[case]
    rows_same = (q == c["q"]).all(axis=1)
    scale_bad = (f16bits(d) != f16bits(c["d"]))[rows_same].sum()
    layer = QLinear(k, n)
    acc = HessianAccumulator(k).set(h)
    set_weight_gptq(layer, w, acc)
    obj = q4_0_objective(layer, w, acc)
    rel = abs(obj - float(c["obj"][0])) / float(c["obj"][0])
    assert rel < 0.01 and rows_same.sum() * 10 >= n * 9 and scale_bad == 0, (rel, int(rows_same.sum()), scale_bad)
    # and the oracle bit for bit (which itself reproduces the fixture code for code)
    qo, do, dead_o, damp_o = O.gptq_q4_0(w, h)
    assert st.dead == dead_o and st.damp == damp_o
    assert np.array_equal(q, qo), f"{(q != qo).sum()} codes differ from the oracle"
    assert np.array_equal(f16bits(d), f16bits(do))
    assert obj == pytest.approx(O.q4_0_objective(w, qo, do, h), rel=1e-12)


# ── [2] a diagonal Hessian: GPTQ is RTN bit for bit (test_gptq.mojo:90-113)
def test_gptq_with_diagonal_hessian_is_rtn():
    rng = np.random.default_rng(5)
    n, k = 70, 288
    w = ((rng.random((n, k)) - 0.5) * 0.3).astype(np.float32)
    h = np.diag(0.1 + 10.0 * rng.random(k))
    g = QLinear(k, n)
    st = set_weight_gptq(g, w, HessianAccumulator(k).set(h))
    r = QLinear(k, n)
    r.set_weight(w)
    assert st.dead == 0
    assert np.array_equal(g.blocks(), r.blocks())


# ── [3] objectives (test_gptq.mojo:115-135) ────────────────────────────────
@pytest.mark.parametrize("case", ["a", "b"])
def test_objectives(fix, case):
    c = fix[case]
    w, h = c["w"], c["h"].astype(np.float64)
    n, k = w.shape
    acc = HessianAccumulator(k).set(h)
    r = QLinear(k, n)
    r.set_weight(w)
    o_rtn = q4_0_objective(r, w, acc)
    assert abs(o_rtn - float(c["obj"][1])) / float(c["obj"][1]) < 1e-6
    g = QLinear(k, n)
    set_weight_gptq(g, w, acc)
    assert q4_0_objective(g, w, acc) < 0.85 * o_rtn


# ── [4] rows are independent; runs repeat (test_gptq.mojo:137-163) ─────────
def test_rows_independent_and_repeatable(fix):
    w, h = fix["b"]["w"], fix["b"]["h"].astype(np.float64)
    n, k = w.shape
    qa, da, _ = gptq_q4_0(w, n, k, h)
    qb, db, _ = gptq_q4_0(w, n, k, h)
    qs, ds, _ = gptq_q4_0(w[:40], 40, k, h)
    assert np.array_equal(qa, qb) and np.array_equal(f16bits(da), f16bits(db))
    assert np.array_equal(qa[:40], qs) and np.array_equal(f16bits(da[:40]), f16bits(ds))


# ── [5] errors (test_gptq.mojo:165-173; gptq.mojo:78-83) ───────────────────
def test_errors():
    with pytest.raises(L.NQError, match="not a multiple of 32"):
        gptq_q4_0(np.zeros((1, 40), np.float32), 1, 40, np.ones((40, 40)))
    with pytest.raises(L.NQError, match="smaller than"):
        gptq_q4_0(np.zeros((2, 64), np.float32), 2, 64, np.ones((32, 32)))
    layer = QLinear(64, 2)
    with pytest.raises(L.NQError, match="smaller than"):
        set_weight_gptq(layer, np.zeros((2, 64), np.float32), HessianAccumulator(32))
    # a Hessian that stays indefinite after damping
    bad = -np.eye(64)
    with pytest.raises(L.NQError, match="not positive definite"):
        set_weight_gptq(layer, np.zeros((2, 64), np.float32), HessianAccumulator(64).set(bad))
    with pytest.raises(L.NQError, match="no weights"):
        layer.forward(torch.zeros((1, 64), device="cuda"))


# ── a SmolVLA-shaped projection, Hessian accumulated on the device from calibration slabs ──
def test_gptq_smolvla_kv_projection_end_to_end():
    rng = np.random.default_rng(9)
    n, k, rows = 320, 960, 2048
    x = rng.standard_normal((rows, k)).astype(np.float32) * np.geomspace(1.0, 30.0, k).astype(np.float32)[rng.permutation(k)]
    x[:, [5, 700]] = 0.0
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    acc = HessianAccumulator(k)
    xd = torch.from_numpy(x).cuda()
    for r0 in range(0, rows, 512):
        acc.add(xd[r0:r0 + 512].contiguous())
    h = acc.h
    g = QLinear(k, n)
    st = set_weight_gptq(g, w, acc)
    assert st.dead == 2
    qo, do, dead_o, damp_o = O.gptq_q4_0(w, h)
    assert (st.dead, st.damp) == (dead_o, damp_o)
    blocks = g.blocks().reshape(n, k // 32, 18)
    q = np.concatenate([blocks[:, :, 2:] & 0xF, blocks[:, :, 2:] >> 4], axis=2).reshape(n, k)
    assert np.array_equal(q, qo), f"{(q != qo).sum()} of {q.size} codes differ from the oracle"
    assert np.array_equal(np.ascontiguousarray(blocks[:, :, :2]).view(np.uint16).reshape(n, -1), f16bits(do))
    # what GPTQ is for: the layer's output error on the calibration rows is below RTN's
    r = QLinear(k, n)
    r.set_weight(w)
    exact = x.astype(np.float64) @ w.astype(np.float64).T
    err_g = np.sum((g.forward(xd).cpu().numpy() - exact) ** 2)
    err_r = np.sum((r.forward(xd).cpu().numpy() - exact) ** 2)
    assert err_g < 0.85 * err_r
    assert err_g == pytest.approx(q4_0_objective(g, w, acc), rel=1e-3)

"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each check is chosen so that a plausible mistake -- a dropped term, a wrong
divisor, an off-by-one in the prefix/suffix range, a transposed operand, a wrong
sign -- fails at least one of them:

* exact rational known-answer vectors (tests/golden/kat_exact.json),
* definition-level brute force loops,
* torch autograd in float64 on an independent torch restatement,
* central finite differences,
* algebraic identities between the two losses and special cases,
* numpy's stable argsort / bincount / cumsum for the integer pair list.
"""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import make_inputs, rel_err

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kat_exact.json")
MODES = [oracle.TOPK, oracle.HIER]


def _cases():
    with open(GOLDEN) as fh:
        return json.load(fh)["cases"]


@pytest.mark.parametrize("case", _cases(), ids=lambda c: f"{c['mode']}-{c['B']}x{c['K']}x{c['F']}x{c['D']}")
def test_exact_known_answers(case):
    mode = oracle.HIER if case["mode"] == "hier" else oracle.TOPK
    args = [np.array(case[k]) for k in ("indices", "weight", "vals", "bias", "target")]
    for fn in (oracle.loss_grads, oracle.brute_force):
        L, dW, dv, db = fn(mode, *args, grad_out=case["grad_out"])
        assert L == pytest.approx(case["loss"], rel=1e-13, abs=1e-13)
        np.testing.assert_allclose(dW, np.array(case["dW"]), rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(dv, np.array(case["dvals"]), rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(db, np.array(case["dbias"]), rtol=1e-12, atol=1e-13)
    # the torch restatement agrees on the loss and (by autograd) on the gradients
    idx = torch.tensor(case["indices"])
    W, v, b = (torch.tensor(case[k], dtype=torch.float64, requires_grad=True) for k in ("weight", "vals", "bias"))
    t = torch.tensor(case["target"], dtype=torch.float64)
    loss = oracle.torch_loss(mode, idx, W, v, b, t, compute_dtype=torch.float64)
    loss.backward(torch.tensor(case["grad_out"], dtype=torch.float64))
    assert loss.item() == pytest.approx(case["loss"], rel=1e-13, abs=1e-13)
    np.testing.assert_allclose(W.grad.numpy(), np.array(case["dW"]), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(v.grad.numpy(), np.array(case["dvals"]), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(b.grad.numpy(), np.array(case["dbias"]), rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(3, 4, 7, 5), (2, 5, 3, 17), (4, 1, 9, 33)])
def test_c_oracle_matches_brute_force(mode, shape):
    B, K, F, D = shape
    args = make_inputs(B, K, F, D, seed=7 + B + K)
    got = oracle.loss_grads(mode, *args, grad_out=-0.75)
    ref = oracle.brute_force(mode, *args, grad_out=-0.75)
    assert got[0] == pytest.approx(ref[0], rel=1e-12)
    for a, b in zip(got[1:], ref[1:]):
        np.testing.assert_allclose(a, b, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(16, 16, 64, 512), (48, 64, 224, 1280), (5, 3, 11, 70)])
@pytest.mark.parametrize("chunk", [None, 7])
def test_c_oracle_matches_torch_autograd_fp64(mode, shape, chunk):
    B, K, F, D = shape
    idx, W, v, b, t = make_inputs(B, K, F, D, seed=99)
    W64, v64, b64 = (x.double().requires_grad_() for x in (W, v, b))
    loss = oracle.torch_loss(mode, idx, W64, v64, b64, t.double(), compute_dtype=torch.float64, chunk_rows=chunk)
    loss.backward(torch.tensor(1.7, dtype=torch.float64))
    L, dW, dv, db = oracle.loss_grads(mode, idx, W, v, b, t, grad_out=1.7)
    assert L == pytest.approx(loss.item(), rel=1e-12)
    assert rel_err(dW, W64.grad) < 1e-12
    assert rel_err(dv, v64.grad) < 1e-12
    assert rel_err(db, b64.grad) < 1e-12


@pytest.mark.parametrize("mode", MODES)
def test_finite_differences(mode):
    B, K, F, D = 3, 4, 6, 8
    idx, W, v, b, t = make_inputs(B, K, F, D, seed=5)
    _, dW, dv, db = oracle.loss_grads(mode, idx, W, v, b, t)
    h = 2.0 ** -6  # exactly representable; the loss is quadratic in each single entry

    def L(W_, v_, b_):
        return oracle.loss_grads(mode, idx, W_, v_, b_, t, want_grads=False)[0]

    rng = np.random.default_rng(0)
    for _ in range(12):
        f, d = int(rng.integers(F)), int(rng.integers(D))
        Wp, Wm = W.clone(), W.clone()
        Wp[f, d] += h
        Wm[f, d] -= h
        assert (L(Wp, v, b) - L(Wm, v, b)) / (2 * h) == pytest.approx(dW[f, d], rel=1e-8, abs=1e-10)
        bi, k = int(rng.integers(B)), int(rng.integers(K))
        vp, vm = v.clone(), v.clone()
        vp[bi, k] += h
        vm[bi, k] -= h
        assert (L(W, vp, b) - L(W, vm, b)) / (2 * h) == pytest.approx(dv[bi, k], rel=1e-8, abs=1e-10)
        bp, bm = b.clone(), b.clone()
        bp[d] += h
        bm[d] -= h
        assert (L(W, v, bp) - L(W, v, bm)) / (2 * h) == pytest.approx(db[d], rel=1e-8, abs=1e-10)


def test_hier_k1_equals_topk_k1():
    args = make_inputs(9, 1, 13, 40, seed=3)
    a = oracle.loss_grads(oracle.HIER, *args, grad_out=0.3)
    b = oracle.loss_grads(oracle.TOPK, *args, grad_out=0.3)
    assert a[0] == pytest.approx(b[0], rel=1e-14)
    for x, y in zip(a[1:], b[1:]):
        np.testing.assert_allclose(x, y, rtol=1e-13, atol=1e-15)


def test_hier_is_mean_of_prefix_topk():
    B, K, F, D = 6, 8, 20, 24
    idx, W, v, b, t = make_inputs(B, K, F, D, seed=11)
    Lh, dWh, dvh, dbh = oracle.loss_grads(oracle.HIER, idx, W, v, b, t)
    L = 0.0
    dW = np.zeros((F, D))
    dv = np.zeros((B, K))
    db = np.zeros(D)
    for k in range(1, K + 1):
        Lk, dWk, dvk, dbk = oracle.loss_grads(oracle.TOPK, idx[:, :k], W, v[:, :k], b, t)
        L += Lk / K
        dW += dWk / K
        dv[:, :k] += dvk / K
        db += dbk / K
    assert Lh == pytest.approx(L, rel=1e-13)
    np.testing.assert_allclose(dWh, dW, rtol=1e-11, atol=1e-14)
    np.testing.assert_allclose(dvh, dv, rtol=1e-11, atol=1e-14)
    np.testing.assert_allclose(dbh, db, rtol=1e-11, atol=1e-14)


@pytest.mark.parametrize("mode", MODES)
def test_zero_vals_closed_form(mode):
    idx, W, v, b, t = make_inputs(5, 4, 9, 12, seed=2)
    L, dW, dv, db = oracle.loss_grads(mode, idx, W, torch.zeros_like(v), b, t)
    assert L == pytest.approx(((b.double() - t.double()) ** 2).mean().item(), rel=1e-14)
    assert np.all(dW == 0.0)
    # dbias = 2/(B*D) * sum_b (bias - t_b), whatever K is
    np.testing.assert_allclose(db, (2.0 / (5 * 12)) * (b.double() - t.double()).sum(0).numpy(), rtol=1e-13)


def test_column_permutation():
    idx, W, v, b, t = make_inputs(4, 8, 30, 16, seed=8)
    perm = torch.randperm(8, generator=torch.Generator().manual_seed(1))
    a = oracle.loss_grads(oracle.TOPK, idx, W, v, b, t)
    p = oracle.loss_grads(oracle.TOPK, idx[:, perm], W, v[:, perm], b, t)
    assert a[0] == pytest.approx(p[0], rel=1e-13)
    np.testing.assert_allclose(a[1], p[1], rtol=1e-11, atol=1e-14)
    np.testing.assert_allclose(a[2][:, perm], p[2], rtol=1e-11, atol=1e-14)
    # the hierarchical loss does depend on the column order
    h = oracle.loss_grads(oracle.HIER, idx, W, v, b, t)
    hp = oracle.loss_grads(oracle.HIER, idx[:, perm], W, v[:, perm], b, t)
    assert abs(h[0] - hp[0]) > 1e-6 * abs(h[0])


def test_duplicate_index_merges_for_topk():
    idx, W, v, b, t = make_inputs(3, 4, 10, 8, seed=4)
    idx[:, 1] = idx[:, 0]
    merged_idx = idx[:, [0, 2, 3]]
    merged_v = torch.stack([v[:, 0] + v[:, 1], v[:, 2], v[:, 3]], dim=1)
    a = oracle.loss_grads(oracle.TOPK, idx, W, v, b, t)
    m = oracle.loss_grads(oracle.TOPK, merged_idx, W, merged_v, b, t)
    assert a[0] == pytest.approx(m[0], rel=1e-6)  # vals sum rounds in fp32
    np.testing.assert_allclose(a[1], m[1], rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("mode", MODES)
def test_grad_out_linearity_and_mass_conservation(mode):
    B, K, F, D = 7, 8, 40, 16
    idx, W, v, b, t = make_inputs(B, K, F, D, seed=6)
    _, dW1, dv1, db1 = oracle.loss_grads(mode, idx, W, v, b, t, grad_out=1.0)
    _, dW3, dv3, db3 = oracle.loss_grads(mode, idx, W, v, b, t, grad_out=-3.0)
    np.testing.assert_allclose(dW3, -3.0 * dW1, rtol=1e-13)
    np.testing.assert_allclose(dv3, -3.0 * dv1, rtol=1e-13)
    np.testing.assert_allclose(db3, -3.0 * db1, rtol=1e-13)
    # rows of untouched latents stay exactly zero
    untouched = np.setdiff1d(np.arange(F), idx.numpy().ravel())
    assert untouched.size > 0 and np.all(dW1[untouched] == 0.0)
    # sum_f <W[f], dW[f]> = sum_{b,k} v dvals  (both equal sum <v w, S>)
    lhs = (W.double().numpy() * dW1).sum()
    rhs = (v.double().numpy() * dv1).sum()
    assert lhs == pytest.approx(rhs, rel=1e-11)


@pytest.mark.parametrize("shape", [(1, 1, 1), (4, 8, 16), (37, 16, 5), (64, 32, 4096)])
def test_csr_matches_numpy_stable_sort(shape):
    B, K, F = shape
    idx = torch.randint(0, F, (B, K), generator=torch.Generator().manual_seed(B * K + F))
    begin, mp = oracle.csr(idx, F)
    flat = idx.numpy().ravel()
    counts = np.bincount(flat, minlength=F)
    np.testing.assert_array_equal(begin, np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32))
    np.testing.assert_array_equal(mp, np.argsort(flat, kind="stable").astype(np.uint32))


def test_oracle_rejects_out_of_range_index():
    idx, W, v, b, t = make_inputs(2, 2, 4, 4)
    idx[0, 0] = 4
    with pytest.raises(ValueError):
        oracle.loss_grads(oracle.HIER, idx, W, v, b, t)
    with pytest.raises(ValueError):
        oracle.csr(idx, 4)


def test_float32_dw_option_matches_double():
    args = make_inputs(8, 4, 12, 20, seed=10)
    _, dW, _, _ = oracle.loss_grads(oracle.HIER, *args)
    _, dW32, _, _ = oracle.loss_grads(oracle.HIER, *args, dw_float32=True)
    assert dW32.dtype == np.float32
    np.testing.assert_allclose(dW32, dW.astype(np.float32), rtol=0, atol=0)

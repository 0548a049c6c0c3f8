"""Pins the router oracle (softmax / sigmoid + top-k) before anything is compared with it."""
import numpy as np
import pytest
import scipy.special

import oracle


def _rows(seed, rows, experts, scale=3.0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((rows, experts)) * scale).astype(np.float32)


@pytest.mark.parametrize("rows,experts,topk", [(7, 8, 2), (33, 64, 6), (16, 128, 8), (5, 256, 8), (3, 1000, 17)])
def test_against_scipy_softmax_and_argsort(rows, experts, topk):
    x = _rows(rows * experts + topk, rows, experts)
    w, idx = oracle.topk_softmax(x, topk)
    p = scipy.special.softmax(x.astype(np.float64), axis=1)
    order = np.argsort(-p, axis=1, kind="stable")[:, :topk]
    assert np.array_equal(idx, order.astype(np.int32))
    np.testing.assert_allclose(w, np.take_along_axis(p, order, axis=1), rtol=2e-6, atol=0)


def test_closed_forms():
    # equal logits: every weight 1/E, ties go to the lowest expert ids in order
    w, idx = oracle.topk_softmax(np.full((2, 16), 1.25, np.float32), 4)
    assert np.array_equal(idx, np.tile(np.arange(4, dtype=np.int32), (2, 1)))
    np.testing.assert_allclose(w, 1.0 / 16, rtol=1e-6)
    # shift invariance of the softmax and weights of all experts summing to one
    x = _rows(1, 9, 32)
    w0, i0 = oracle.topk_softmax(x, 32)
    w1, i1 = oracle.topk_softmax(x + np.float32(8.0), 32)
    assert np.array_equal(i0, i1)
    np.testing.assert_allclose(w0, w1, rtol=2e-5)
    np.testing.assert_allclose(w0.sum(axis=1), 1.0, rtol=1e-6)
    assert np.all(np.diff(w0, axis=1) <= 0)  # descending
    # one dominant logit: its weight tends to one
    x = np.zeros((1, 8), np.float32)
    x[0, 5] = 40.0
    w, idx = oracle.topk_softmax(x, 1)
    assert idx[0, 0] == 5 and abs(w[0, 0] - 1.0) < 1e-6


def test_sigmoid_and_renormalise():
    x = _rows(3, 11, 64)
    w, idx = oracle.topk_softmax(x, 8, sigmoid=True)
    s = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    order = np.argsort(-s, axis=1, kind="stable")[:, :8]
    assert np.array_equal(idx, order.astype(np.int32))
    np.testing.assert_allclose(w, np.take_along_axis(s, order, axis=1), rtol=2e-6)
    wn, idn = oracle.topk_softmax(x, 8, sigmoid=True, renorm=True)
    assert np.array_equal(idn, idx)
    np.testing.assert_allclose(wn, w / w.sum(axis=1, keepdims=True), rtol=2e-6)
    np.testing.assert_allclose(wn.sum(axis=1), 1.0, rtol=1e-6)


@pytest.mark.skipif(oracle.ck_ref() is None, reason="oracle/_ref not built")
@pytest.mark.parametrize("seed", range(4))
def test_matches_ck_tile_reference(seed):
    rng = np.random.default_rng(seed)
    rows, experts = int(rng.integers(1, 200)), int(rng.choice([8, 32, 64, 128, 256]))
    topk = int(rng.integers(1, min(experts, 9)))
    x = _rows(seed + 100, rows, experts)
    w, idx = oracle.topk_softmax(x, topk)
    cw, cidx = oracle.ck_topk_softmax(x, topk)
    assert np.array_equal(idx, cidx)  # random fp32 logits: no ties
    assert np.array_equal(w, cw)      # same operation order as the reference: bit-exact


def test_golden_fixture():
    import os
    f = np.load(os.path.join(os.path.dirname(__file__), "golden", "router_ck_reference.npz"))
    w, idx = oracle.topk_softmax(f["logits"], int(f["topk"]))
    assert np.array_equal(idx, f["ids"]) and np.array_equal(w, f["weights"])

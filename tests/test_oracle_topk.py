"""Pins of the routing-producer oracle (softmax -> top-k -> renormalise) that do
not retype its formula: closed forms, an identity in float64, brute force."""
import itertools

import numpy as np
import pytest

from oracle import routing


def test_closed_form_log_integers():
    # logits ln(1), ln(2), .., ln(E): probabilities are i / (E (E+1) / 2)
    E = 4
    logits = np.log(np.arange(1, E + 1, dtype=np.float64)).astype(np.float32)[None, :]
    w, ids = routing.fused_topk(logits, 2, renormalize=False)
    assert ids.tolist() == [[3, 2]]
    np.testing.assert_allclose(w, [[0.4, 0.3]], rtol=1e-6)
    w, ids = routing.fused_topk(logits, 2, renormalize=True)
    np.testing.assert_allclose(w, [[4 / 7, 3 / 7]], rtol=1e-6)
    w, ids = routing.fused_topk(logits, 4, renormalize=True)
    assert ids.tolist() == [[3, 2, 1, 0]]
    np.testing.assert_allclose(w, [[0.4, 0.3, 0.2, 0.1]], rtol=1e-6)


def test_uniform_logits_and_ties_take_lower_ids():
    w, ids = routing.fused_topk(np.zeros((3, 8), np.float32), 3, renormalize=False)
    assert ids.tolist() == [[0, 1, 2]] * 3
    np.testing.assert_allclose(w, np.full((3, 3), 1 / 8), rtol=1e-6)
    w, ids = routing.fused_topk(np.array([[1, 5, 5, 0, 5]], np.float32), 2)
    assert ids.tolist() == [[1, 2]]
    np.testing.assert_allclose(w, [[0.5, 0.5]], rtol=1e-6)


@pytest.mark.parametrize("n,E,k,seed", [(64, 8, 2, 0), (33, 64, 6, 1), (17, 5, 5, 2), (9, 130, 8, 3)])
def test_renormalised_weights_are_softmax_over_kept_logits(n, E, k, seed):
    # identity: (p_j / s) / sum_kept (p_i / s) = softmax restricted to the kept experts; checked in float64
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, E)).astype(np.float32)
    w, ids = routing.fused_topk(x, k, renormalize=True)
    kept = np.take_along_axis(x.astype(np.float64), ids.astype(np.int64), axis=1)
    ref = np.exp(kept - kept.max(axis=1, keepdims=True))
    ref /= ref.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(w, ref, rtol=2e-6)
    # kept logits descend, and nothing left out beats the smallest kept one
    assert (np.diff(kept, axis=1) <= 0).all()
    for i in range(n):
        rest = np.delete(x[i], ids[i])
        assert rest.size == 0 or rest.max() <= kept[i, -1]


def test_brute_force_selection_small():
    rng = np.random.default_rng(5)
    x = rng.integers(-2, 3, size=(40, 6)).astype(np.float32)   # many ties
    w, ids = routing.fused_topk(x, 3, renormalize=False)
    for i in range(x.shape[0]):
        p = np.exp(x[i].astype(np.float64))
        p /= p.sum()
        # best subset in (value desc, id asc) order by exhaustive search over ordered triples
        best = max(itertools.permutations(range(6), 3), key=lambda c: [(x[i][e], -e) for e in c])
        assert ids[i].tolist() == list(best)
        np.testing.assert_allclose(w[i], p[list(best)], rtol=2e-6)

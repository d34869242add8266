"""The oracle's sigmoid router (cuda/moe/gate_topk.cu:140-200, 329-364) pinned by what the
definition fixes: float64 probabilities, an independent numpy selection, the tie rule, the floor
of the renormalization."""
import numpy as np

import oracle
from loken_amd import synth


def test_sigmoid_router_matches_an_independent_selection():
    tokens, experts, k = 40, 128, 8
    logits = synth.normal(7, 1, tokens * experts).reshape(tokens, experts) * 2.0
    bias = 0.3 * synth.normal(7, 2, experts)
    ids, w = oracle.topk_sigmoid(logits, k, bias=bias, renorm=True, scale=2.5)
    p = 1.0 / (1.0 + np.exp(-logits.astype(np.float64)))
    want_ids = np.argsort(-(p + bias), axis=1, kind="stable")[:, :k]
    assert np.array_equal(ids, want_ids)
    chosen = np.take_along_axis(p, want_ids, axis=1)
    want_w = chosen / chosen.sum(axis=1, keepdims=True) * 2.5
    assert np.abs(w - want_w).max() < 1e-6
    # the bias steers the choice only: without renorm the weights are the plain probabilities
    ids2, w2 = oracle.topk_sigmoid(logits, k, bias=bias, renorm=False)
    assert np.array_equal(ids2, want_ids) and np.abs(w2 - chosen).max() < 1e-6


def test_ties_go_to_the_lower_expert_and_tiny_sums_hit_the_floor():
    logits = np.zeros((1, 32), np.float32)
    ids, w = oracle.topk_sigmoid(logits, 4, renorm=True)
    assert ids.tolist() == [[0, 1, 2, 3]] and np.allclose(w, 0.25)
    deep = np.full((1, 32), -30.0, np.float32)          # p ~ 9e-14: the sum of four is below 2^-14
    ids, w = oracle.topk_sigmoid(deep, 4, renorm=True)
    p = 1.0 / (1.0 + np.exp(30.0))
    assert np.allclose(w, p / 6.103515625e-5, rtol=1e-5)

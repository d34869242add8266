"""Router-side launchers on the card: the fused gate mat-vec + softmax + top-k, the sigmoid
router and the stable sorts, against the oracle and numpy."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import moe, synth

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("tokens,hidden,experts,k,renorm", [(1, 2048, 128, 8, True), (16, 2048, 128, 8, True),
                                                            (256, 2048, 128, 8, False), (3, 4096, 64, 4, True),
                                                            (2, 1030, 32, 2, True), (5, 8192, 256, 8, True),
                                                            (2, 514, 40, 3, False)])
def test_gate_topk_softmax_matches_the_two_step_path(tokens, hidden, experts, k, renorm):
    x = synth.normal(20, 1, tokens * hidden).reshape(tokens, hidden)
    gate = (synth.normal(20, 2, experts * hidden) * (1.5 / np.sqrt(hidden))).reshape(experts, hidden).astype(np.float32)
    logits = x.astype(np.float64) @ gate.astype(np.float64).T
    want_ids, want_w = oracle.topk_softmax(logits.astype(np.float32), k, renorm)
    w, ids = moe.gate_topk_softmax(dev(x), dev(gate), k, renorm)
    w, ids = w.cpu().numpy(), ids.cpu().numpy()
    # a logit here is a 64-lane f32 sum: where two probabilities at the cut lie closer than that
    # rounding, either order is right; everywhere else the experts must be the oracle's
    p = np.exp(logits - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    ranked = -np.sort(-p, axis=1)
    clear = (ranked[:, :k] - ranked[:, 1:k + 1]).min(axis=1) > 1e-5 * ranked[:, :1].ravel()
    assert clear.mean() > 0.9
    assert np.array_equal(ids[clear], want_ids[clear])
    assert np.abs(w[clear] - want_w[clear]).max() < 2e-5
    # the launch agrees with itself split in two: logits through the unfused router
    w2, ids2 = moe.topk_softmax(dev(logits.astype(np.float32)), k, renorm)
    assert np.array_equal(ids2.cpu().numpy()[clear], ids[clear])


@pytest.mark.parametrize("tokens,experts,k,renorm,scale,with_bias", [(1, 256, 8, True, 2.5, True), (33, 128, 8, True, 1.0, False),
                                                                     (7, 64, 6, False, 1.0, True), (4, 40, 3, True, 0.5, True),
                                                                     (2, 512, 10, True, 1.0, True)])
def test_topk_sigmoid_post(tokens, experts, k, renorm, scale, with_bias):
    logits = synth.normal(21, 1, tokens * experts).reshape(tokens, experts) * 2.0
    bias = (0.2 * synth.normal(21, 2, experts)).astype(np.float32) if with_bias else None
    want_ids, want_w = oracle.topk_sigmoid(logits, k, bias=bias, renorm=renorm, scale=scale)
    w, ids = moe.topk_sigmoid_post(dev(logits), k, dev(bias) if with_bias else None, renorm, scale)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.abs(w.cpu().numpy() - want_w).max() <= 1e-6 * scale


def test_sigmoid_ties_and_floor():
    w, ids = moe.topk_sigmoid_post(dev(np.zeros((2, 64), np.float32)), 5)
    assert ids.cpu().numpy().tolist() == [[0, 1, 2, 3, 4]] * 2 and np.allclose(w.cpu().numpy(), 0.2)
    deep = np.full((1, 64), -30.0, np.float32)
    w, _ = moe.topk_sigmoid_post(dev(deep), 4)
    want_ids, want_w = oracle.topk_sigmoid(deep, 4)
    assert np.allclose(w.cpu().numpy(), want_w, rtol=1e-5)


@pytest.mark.parametrize("n,experts,small", [(1, 128, True), (8, 128, True), (32, 128, True), (200, 8, True), (257, 128, False),
                                              (2048, 128, False), (5000, 3, False), (4096, 100000, False)])
def test_stable_sorts_match_numpy(n, experts, small):
    keys = synth.rand_ints(22, n, n, experts).astype(np.uint32)
    got, order = moe.stable_sort_u32(dev(keys.view(np.int32)), small=small)
    want_order = np.argsort(keys, kind="stable")
    assert np.array_equal(order.cpu().numpy().view(np.uint32), want_order.astype(np.uint32))
    assert np.array_equal(got.cpu().numpy().view(np.uint32), keys[want_order])

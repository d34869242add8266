"""Pins the oracle's router and MoE block by decomposition into single-matrix calls.

out[t] = sum_k w[t,k] * down_e( silu(gate_e x_t) * up_e x_t ), each projection an independent
oracle matmul; the reference's own host path is built the same way
(src/inference/moe_cuda_cpu/mod.rs:459-605, 1478-1660).
"""
import numpy as np
import pytest

import oracle
from loken_amd import synth


def test_router_is_softmax_topk_renormalized():
    rng = np.random.default_rng(20)
    logits = rng.standard_normal((7, 32)).astype(np.float32)
    logits[3, 5] = logits[3, 9]  # a tie: the lower index wins
    ids, w = oracle.topk_softmax(logits, 4, renorm=True)
    p = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    for t in range(7):
        order = sorted(range(32), key=lambda e: (-p[t, e], e))[:4]
        assert ids[t].tolist() == order
        np.testing.assert_allclose(w[t], p[t, order] / p[t, order].sum(), rtol=2e-6)
    ids2, w2 = oracle.topk_softmax(logits, 4, renorm=False)
    assert ids2.tolist() == ids.tolist()
    np.testing.assert_allclose(w2, np.take_along_axis(p, ids.astype(np.int64), 1), rtol=2e-6)


def test_grouping_is_a_stable_sort_by_expert():
    rng = np.random.default_rng(21)
    ids = rng.integers(0, 6, 40).astype(np.int32)
    slots, experts = oracle.group_by_expert(ids)
    want = np.argsort(ids, kind="stable")
    assert slots.tolist() == want.tolist()
    assert experts.tolist() == ids[want].tolist()


@pytest.mark.parametrize("family", [0, 1])
@pytest.mark.parametrize("dt_down", [oracle.Q4_K, oracle.Q6_K])
def test_moe_block_decomposes_into_single_matrix_calls(family, dt_down):
    tokens, hidden, ffn, n_experts, topk = 5, 512, 256, 6, 2
    dt = oracle.Q4_K
    gate = synth.weight(dt, n_experts * ffn, hidden, seed=22, stream=1)
    up = synth.weight(dt, n_experts * ffn, hidden, seed=22, stream=2)
    down = synth.weight(dt_down, n_experts * hidden, ffn, seed=22, stream=3)
    # larger block scales so the GLU output is O(1) and quantizes meaningfully
    x = synth.activation(tokens, hidden, seed=22) * np.float32(30.0)
    logits = synth.activation(tokens, n_experts, seed=22, stream=7)
    ids, w = oracle.topk_softmax(logits, topk)
    out, h = oracle.moe_forward(family, dt, dt_down, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)

    mm = (lambda d, a, b, n: oracle.ob_matmul(d, a, b, n)) if family else (lambda d, a, b, n: oracle.oa_matmul(d, a, b, n))
    gate_e = gate.reshape(n_experts, ffn, -1, 144)
    up_e = up.reshape(n_experts, ffn, -1, 144)
    down_e = down.reshape(n_experts, hidden, -1, oracle.BLOCK_BYTES[dt_down])
    slots, experts = oracle.group_by_expert(ids)
    want = np.zeros((tokens, hidden), np.float32)
    for j, (slot, e) in enumerate(zip(slots, experts)):
        t = slot // topk
        g = mm(dt, x[t:t + 1], gate_e[e], ffn)[0]
        u = mm(dt, x[t:t + 1], up_e[e], ffn)[0]
        with np.errstate(over="ignore"):
            hj = (u * (g / (np.float32(1.0) + np.exp(-g, dtype=np.float32)))).astype(np.float32)
        # expf of libm vs numpy may differ in the last place
        np.testing.assert_allclose(h[j], hj, rtol=1e-6, atol=1e-30)
        dn = mm(dt_down, h[j:j + 1], down_e[e], hidden)[0]
        want[t] += w.reshape(-1)[slot] * dn
    assert np.abs(out).max() > 0
    np.testing.assert_allclose(out, want, rtol=1e-6, atol=1e-12)


def test_moe_result_does_not_depend_on_order_within_a_token_beyond_rounding():
    # permuting a token's choices permutes its slots; only the f32 fold order changes
    tokens, hidden, ffn, n_experts, topk = 3, 256, 256, 5, 3
    dt = oracle.Q4_K
    gate = synth.weight(dt, n_experts * ffn, hidden, seed=23, stream=1)
    up = synth.weight(dt, n_experts * ffn, hidden, seed=23, stream=2)
    down = synth.weight(dt, n_experts * hidden, ffn, seed=23, stream=3)
    x = synth.activation(tokens, hidden, seed=23) * np.float32(30.0)
    ids, w = oracle.topk_softmax(synth.activation(tokens, n_experts, seed=23, stream=7), topk)
    a = oracle.moe_forward(1, dt, dt, x, gate, up, down, ids, w, n_experts, ffn)
    b = oracle.moe_forward(1, dt, dt, x, gate, up, down, ids[:, ::-1], w[:, ::-1], n_experts, ffn)
    np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-9)

"""Pins the three activation quantizers of the oracle.

Q8_0 against ggml's own bytes (same recipe: d = amax/127, id = 1/d, roundf); Q8_K against ggml's
bytes away from exact ties; all three against closed forms where the codes are known exactly,
the construction the reference's imma_reference test uses
(src/inference/moe_cuda/imma_reference.rs:17-29).
"""
import numpy as np

import oracle


def _q81(x):
    b = oracle.quantize_q8_1(x).reshape(-1, 36)
    d = b[:, 0:2].copy().view(np.float16).reshape(-1)
    s = b[:, 2:4].copy().view(np.float16).reshape(-1)
    q = b[:, 4:].copy().view(np.int8)
    return d, s, q


def test_q8_0_quantizer_reproduces_ggml_bytes(ggml_vectors):
    got = oracle.quantize_q8_0(ggml_vectors["input"])
    assert got.tolist() == ggml_vectors["q8_0"]["quant"].tolist()


def test_q8_k_quantizer_reproduces_ggml_bytes_away_from_ties(ggml_vectors):
    x = ggml_vectors["input"]
    got = oracle.quantize_q8_k(x).reshape(-1, 292)
    want = ggml_vectors["q8_K"]["quant"].reshape(-1, 292)
    # ggml rounds to nearest even, loken half away from zero; they can differ only on exact ties.
    d = got[:, :4].copy().view(np.float32).reshape(-1)
    assert d.view(np.uint32).tolist() == want[:, :4].copy().view(np.float32).reshape(-1).view(np.uint32).tolist()
    gq = got[:, 4:260].copy().view(np.int8).astype(np.int32)
    wq = want[:, 4:260].copy().view(np.int8).astype(np.int32)
    diff = np.argwhere(gq != wq)
    for b, l in diff:
        inv = np.float32(-127.0) / np.float32(x[b * 256:(b + 1) * 256][np.argmax(np.abs(x[b * 256:(b + 1) * 256]))])
        v = np.float32(inv * x[b * 256 + l])
        assert abs(v - np.trunc(v)) == 0.5, "codes may differ from ggml only on a tie"
    assert len(diff) <= 2
    if len(diff) == 0:
        assert got[:, 260:].tolist() == want[:, 260:].tolist()


def test_q8_1_exact_grid_codes():
    # values n * 2^-6 with one |n| = 127 per block: d = 2^-6 exactly and the codes are n
    rng = np.random.default_rng(5)
    n = rng.integers(-127, 128, (16, 32))
    n[:, 0] = np.where(rng.integers(0, 2, 16) == 0, 127, -127)
    x = (n * 2.0 ** -6).astype(np.float32)
    d, s, q = _q81(x)
    assert (d == np.float16(2.0 ** -6)).all()
    assert q.tolist() == n.tolist()
    assert s.tolist() == (n.sum(axis=1).astype(np.float32) * np.float32(2.0 ** -6)).astype(np.float16).tolist()
    b0 = oracle.quantize_q8_0(x).reshape(-1, 34)
    assert b0[:, 2:].copy().view(np.int8).tolist() == n.tolist()


def test_q8_1_zero_block_and_range_invariants():
    d, s, q = _q81(np.zeros(64, np.float32))
    assert (d == 0).all() and (s == 0).all() and (q == 0).all()
    rng = np.random.default_rng(6)
    x = rng.standard_normal((200, 32)).astype(np.float32) * np.float32(3.0)
    d, s, q = _q81(x)
    assert np.abs(q.astype(np.int32)).max() <= 127
    assert (np.abs(q.astype(np.int32)).max(axis=1) == 127).all()
    amax = np.abs(x).max(axis=1)
    dd = (amax / np.float32(127.0)).astype(np.float32)
    assert d.tolist() == dd.astype(np.float16).tolist()
    # s is f16(sum(q) * d) with d before its f16 rounding
    assert s.tolist() == (q.astype(np.int32).sum(axis=1).astype(np.float32) * dd).astype(np.float16).tolist()
    # codes are round-half-away of x * (1/d)
    inv = (np.float32(1.0) / dd).astype(np.float32)
    v = (x * inv[:, None]).astype(np.float32)
    want = np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))
    assert q.astype(np.float32).tolist() == want.tolist()


def test_q8_1_ties_round_away_from_zero():
    # d = 1 exactly (amax = 127), values n + 0.5 are exact ties
    x = np.zeros(32, np.float32)
    x[0] = 127.0
    x[1:9] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5]
    _, _, q = _q81(x)
    assert q[0, :9].tolist() == [127, 1, 2, 3, -1, -2, -3, 64, -64]


def test_q8_k_extreme_maps_to_minus_127_and_bsums():
    rng = np.random.default_rng(7)
    x = rng.standard_normal(256 * 6).astype(np.float32)
    x[256 + 3] = 500.0  # a lopsided positive extreme
    x[512:768] = 0.0    # a zero block
    blocks = oracle.quantize_q8_k(x).reshape(-1, 292)
    d = blocks[:, :4].copy().view(np.float32).reshape(-1)
    q = blocks[:, 4:260].copy().view(np.int8).astype(np.int32)
    bs = blocks[:, 260:].copy().view(np.int16).astype(np.int32)
    for b in range(6):
        xb = x[256 * b:256 * (b + 1)]
        if not xb.any():
            assert d[b] == 0 and not q[b].any() and not bs[b].any()
            continue
        e = np.argmax(np.abs(xb))
        assert q[b, e] == -127
        inv = np.float32(-127.0) / xb[e]
        assert d[b] == np.float32(1.0) / inv
        assert q[b].max() <= 127
        assert bs[b].tolist() == q[b].reshape(16, 16).sum(axis=1).tolist()
    # opposite-sign overshoot clamps to +127
    y = np.zeros(256, np.float32)
    y[0] = -1.0
    y[1] = np.nextafter(np.float32(1.0), np.float32(2.0))
    y[0] = -np.float32(1.0)
    yb = oracle.quantize_q8_k(np.concatenate([y])).reshape(-1, 292)
    assert yb[0, 4:260].copy().view(np.int8).max() <= 127

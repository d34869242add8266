"""The oracle's RMSNorm family and split activation (the decode-step producers that end in a
Q8_1 row, src/inference/cuda/mmvq_gguf.cu:805-999), pinned by what the mathematics fixes: float64
evaluations of the textbook formulas, the stated accumulation order rebuilt independently in numpy,
and special cases with closed forms."""
import numpy as np
import pytest

import oracle
from loken_amd import synth


def rms_f64(x, w, eps):
    x = x.astype(np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w.astype(np.float64)


@pytest.mark.parametrize("cols", [512, 2048, 4096])
def test_norm_modes_agree_with_float64(cols):
    rows = 3
    x = synth.normal(1, 1, rows * cols).reshape(rows, cols) * 3.0
    res = synth.normal(1, 2, rows * cols).reshape(rows, cols)
    w = 1.0 + 0.1 * synth.normal(1, 3, cols)
    w2 = 1.0 + 0.1 * synth.normal(1, 4, cols)
    close = lambda got, want: np.abs(got - want).max() <= 2e-6 * np.abs(want).max()
    assert close(oracle.norm_rows(0, x, w, eps=1e-5), rms_f64(x, w, 1e-5))
    mid, out = oracle.norm_rows(1, x, w, residual=res, eps=1e-6)
    assert np.array_equal(mid, x + res)
    assert close(out, rms_f64(x + res, w, 1e-6))
    mid, out = oracle.norm_rows(2, x, w2, w_first=w, residual=res, eps=1e-6, eps_first=1e-5)
    want_mid = rms_f64(x, w, 1e-5) + res
    assert close(mid, want_mid) and close(out, rms_f64(want_mid, w2, 1e-6))


def test_the_sum_of_squares_folds_in_the_stated_order():
    cols = 1024
    row = synth.normal(2, 1, cols)
    # lane t over t, t + 256, ... (one rounding per step: float64 holds a float32 product exactly,
    # so rounding the float64 sum once is the fused multiply-add), then the stride-halving tree
    part = np.zeros(256, np.float32)
    for j in range(cols // 256):
        v = row[256 * j:256 * (j + 1)].astype(np.float64)
        part = (v * v + part.astype(np.float64)).astype(np.float32)
    s = 128
    while s:
        part[:s] = part[:s] + part[s:2 * s]
        s //= 2
    want = np.float32(1.0) / np.sqrt(part[0] / np.float32(cols) + np.float32(1e-5), dtype=np.float32)
    assert np.float32(oracle.inv_rms_wide(row, 1e-5)) == want
    # another order gives other bits somewhere: the order is part of the statement
    seeds = [np.float32(1.0) / np.sqrt(np.float32((synth.normal(s_, 1, cols).astype(np.float32) ** 2).sum(dtype=np.float32)) /
                                       np.float32(cols) + np.float32(1e-5), dtype=np.float32) !=
             np.float32(oracle.inv_rms_wide(synth.normal(s_, 1, cols), 1e-5)) for s_ in range(20)]
    assert any(seeds)


def test_closed_forms():
    cols = 512
    ones = np.ones((1, cols), np.float32)
    # a constant row c has rms |c|: out = sign(c) * w up to the eps term
    out = oracle.norm_rows(0, -4.0 * ones, 2.0 * ones, eps=0.0)
    assert np.array_equal(out, -2.0 * ones)
    # a zero row stays zero (rms = 1 / sqrt(eps), finite)
    assert np.array_equal(oracle.norm_rows(0, 0.0 * ones, ones, eps=1e-6), 0.0 * ones)
    # scale invariance without eps: rmsnorm(2^k x) == rmsnorm(x) exactly (powers of two commute with rounding)
    x = synth.normal(3, 1, cols).reshape(1, cols)
    w = synth.normal(3, 2, cols)
    assert np.array_equal(oracle.norm_rows(0, x, w, eps=0.0), oracle.norm_rows(0, 8.0 * x, w, eps=0.0))


@pytest.mark.parametrize("act", [0, 1])
def test_split_activation_agrees_with_float64(act):
    n = 96
    gu = synth.normal(4, act, 2 * 2 * n).reshape(2, 2 * n) * 4.0
    g, u = gu[:, :n].astype(np.float64), gu[:, n:].astype(np.float64)
    if act == 0:
        want = g / (1.0 + np.exp(-g)) * u
    else:
        want = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3))) * u
    got = oracle.split_act_mul(gu, act)
    assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())
    # zeros in, zeros out; a zero gate silences the pair whatever `up` holds
    z = gu.copy()
    z[:, :n] = 0.0
    assert np.array_equal(oracle.split_act_mul(z, act), np.zeros((2, n), np.float32))

"""Pins the oracle's integer sums and f32 combines without retyping its formulas.

  * integer sub-block dots: numpy int64 brute force over nibbles/codes decoded by an
    independent numpy decoder (itself checked against ggml's DEQUANT in this file);
  * f32 outputs: an f64 sum over dequantized weights x dequantized activations (the bound the
    reference uses, src/tensor/quantized/tests.rs:576-632) and the special case sc=1, m=0, d=1
    where the Q4_K product is a plain int8 GEMV;
  * the threaded AVX2 baseline against the scalar path at the reference's vector-vs-scalar bound
    (src/tensor/quant_cpu/avx/parity.rs:50-56).
"""
import numpy as np
import pytest

import oracle
from loken_amd import synth

LEGACY = {"q4_0": oracle.Q4_0, "q4_1": oracle.Q4_1, "q5_0": oracle.Q5_0, "q5_1": oracle.Q5_1, "iq4_nl": oracle.IQ4_NL,
          "mxfp4": oracle.MXFP4}
LEVELS = {oracle.IQ4_NL: np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int64),
          oracle.MXFP4: np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.int64)}
LOWBIT = {"q2_k": oracle.Q2_K, "q3_k": oracle.Q3_K}
DT = {"q4_k": oracle.Q4_K, "q5_k": oracle.Q5_K, "q6_k": oracle.Q6_K, "q8_0": oracle.Q8_0, "iq4_xs": oracle.IQ4_XS, **LEGACY,
      **LOWBIT}
FAST = sorted(set(DT) - {"q5_k", "iq4_xs"} - set(LEGACY) - set(LOWBIT))   # formats the timed AVX2 baseline serves


# ---- independent numpy decoders: integer codes and float scales per value ----
def np_codes_q4k(w):
    """w [n, nb, 144] -> codes [n, nb*256] (0..15), sc [n, nb*8], mn [n, nb*8], d, dmin [n, nb]."""
    n, nb, _ = w.shape
    qs = w[:, :, 16:].reshape(n, nb, 4, 32)
    codes = np.stack([qs & 0xF, qs >> 4], axis=3).reshape(n, nb * 256).astype(np.int64)
    p = w[:, :, 4:16].astype(np.int64)
    sc = np.empty((n, nb, 8), np.int64)
    mn = np.empty((n, nb, 8), np.int64)
    sc[..., :4] = p[..., 0:4] & 63
    mn[..., :4] = p[..., 4:8] & 63
    sc[..., 4:] = (p[..., 8:12] & 0xF) | ((p[..., 0:4] >> 6) << 4)
    mn[..., 4:] = (p[..., 8:12] >> 4) | ((p[..., 4:8] >> 6) << 4)
    d = w[:, :, 0:2].copy().view(np.float16).reshape(n, nb).astype(np.float64)
    dmin = w[:, :, 2:4].copy().view(np.float16).reshape(n, nb).astype(np.float64)
    return codes, sc.reshape(n, nb * 8), mn.reshape(n, nb * 8), d, dmin


def np_codes_q5k(w):
    """w [n, nb, 176]: the Q4_K decoding of the same fields, plus bit s of qh[l] worth sixteen."""
    n, nb, _ = w.shape
    as_q4k = np.concatenate([w[:, :, :16], w[:, :, 48:]], axis=2)
    codes, sc, mn, d, dmin = np_codes_q4k(as_q4k)
    qh = w[:, :, 16:48].astype(np.int64)                                  # [n, nb, l]
    fifth = (qh[:, :, None, :] >> np.arange(8)[None, None, :, None]) & 1  # [n, nb, s, l]
    return codes + 16 * fifth.reshape(n, nb * 256), sc, mn, d, dmin


def np_codes_q6k(w):
    n, nb, _ = w.shape
    ql = w[:, :, 0:128].reshape(n, nb, 2, 2, 32).astype(np.int64)      # [half][span][l]
    qh = w[:, :, 128:192].reshape(n, nb, 2, 32).astype(np.int64)       # [half][l]
    codes = np.empty((n, nb, 2, 4, 32), np.int64)
    for g in range(4):
        low = (ql[:, :, :, g % 2, :] >> (0 if g < 2 else 4)) & 0xF
        high = (qh >> (2 * g)) & 3
        codes[:, :, :, g, :] = (low | (high << 4)) - 32
    sc = w[:, :, 192:208].copy().view(np.int8).reshape(n, nb * 16).astype(np.int64)
    d = w[:, :, 208:210].copy().view(np.float16).reshape(n, nb).astype(np.float64)
    return codes.reshape(n, nb * 256), sc, d


def np_codes_q80(w):
    n, nb, _ = w.shape
    codes = w[:, :, 2:].copy().view(np.int8).reshape(n, nb * 32).astype(np.int64)
    d = w[:, :, 0:2].copy().view(np.float16).reshape(n, nb).astype(np.float64)
    return codes, d


def np_codes_legacy(dtype, w):
    """w [n, nb, bytes] of a 32-value nibble format -> codes less their bias [n, nb*32], d, m [n, nb]."""
    n, nb, _ = w.shape
    qs_at = {oracle.Q4_0: 2, oracle.Q4_1: 4, oracle.Q5_0: 6, oracle.Q5_1: 8, oracle.IQ4_NL: 2, oracle.MXFP4: 1}[dtype]
    qs = w[:, :, qs_at:qs_at + 16].astype(np.int64)
    codes = np.concatenate([qs & 0xF, qs >> 4], axis=2)                       # value v at [..., v]
    if dtype in (oracle.Q5_0, oracle.Q5_1):
        qh = w[:, :, qs_at - 4:qs_at].copy().view(np.uint32).reshape(n, nb, 1).astype(np.int64)
        codes = codes | (((qh >> np.arange(32)[None, None, :]) & 1) << 4)
    codes = codes - {oracle.Q4_0: 8, oracle.Q5_0: 16}.get(dtype, 0)
    if dtype in LEVELS:
        codes = LEVELS[dtype][codes]
    if dtype == oracle.MXFP4:   # E8M0 scale, halved: 2^(e - 128) (the generator keeps e well above 1)
        d = np.exp2(w[:, :, 0].astype(np.float64) - 128.0)
    else:
        d = w[:, :, 0:2].copy().view(np.float16).reshape(n, nb).astype(np.float64)
    m = (w[:, :, 2:4].copy().view(np.float16).reshape(n, nb).astype(np.float64)
         if dtype in (oracle.Q4_1, oracle.Q5_1) else np.zeros((n, nb)))
    return codes.reshape(n, nb * 32), d, m


def np_codes_lowbit(dtype, w):
    """Q2_K [n, nb, 84] / Q3_K [n, nb, 110] -> values [n, nb*256], scales, mins [n, nb*16], d, dmin [n, nb]."""
    n, nb, _ = w.shape
    q2 = dtype == oracle.Q2_K
    qs = w[:, :, 16:80] if q2 else w[:, :, 32:96]
    qs = qs.reshape(n, nb, 2, 2, 16).astype(np.int64)                          # [half of block][byte half][l]
    vals = np.empty((n, nb, 16, 16), np.int64)
    for sb in range(16):
        half, t = sb // 8, sb % 8
        vals[:, :, sb, :] = (qs[:, :, half, t % 2, :] >> (2 * (t // 2))) & 3
        if not q2:
            hm = w[:, :, 16 * (t % 2):16 * (t % 2) + 16].astype(np.int64)
            vals[:, :, sb, :] -= 4 * (1 - ((hm >> (4 * half + t // 2)) & 1))
    if q2:
        sc = (w[:, :, 0:16] & 0xF).astype(np.int64)
        mn = (w[:, :, 0:16] >> 4).astype(np.int64)
        d = w[:, :, 80:82].copy().view(np.float16).reshape(n, nb).astype(np.float64)
        dmin = w[:, :, 82:84].copy().view(np.float16).reshape(n, nb).astype(np.float64)
    else:
        p = w[:, :, 96:108].astype(np.int64)
        sc = np.empty((n, nb, 16), np.int64)
        for i in range(16):
            group, j = i // 4, i % 4
            byte = p[:, :, j + 4 * (group % 2)]
            low = (byte & 0xF) if group < 2 else (byte >> 4)
            sc[:, :, i] = (low | (((p[:, :, 8 + j] >> (2 * group)) & 3) << 4)) - 32
        mn = np.zeros((n, nb, 16), np.int64)
        d = w[:, :, 108:110].copy().view(np.float16).reshape(n, nb).astype(np.float64)
        dmin = np.zeros((n, nb))
    return vals.reshape(n, nb * 256), sc.reshape(n, nb * 16), mn.reshape(n, nb * 16), d, dmin


def np_codes_iq4xs(w):
    """w [n, nb, 136] -> levels [n, nb*256], run scales (six bits less 32) [n, nb*8], d [n, nb]."""
    n, nb, _ = w.shape
    q = w[:, :, 8:136].reshape(n, nb, 8, 16).astype(np.int64)
    lv = LEVELS[oracle.IQ4_NL]
    vals = np.concatenate([lv[q & 0xF], lv[q >> 4]], axis=3)                         # [n, nb, run, 32]
    sl = w[:, :, 4:8].astype(np.int64)
    sh = w[:, :, 2:4].copy().view(np.uint16).reshape(n, nb).astype(np.int64)
    ls = np.stack([((sl[:, :, ib // 2] >> (4 * (ib % 2))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4) for ib in range(8)], axis=2) - 32
    d = w[:, :, 0:2].copy().view(np.float16).reshape(n, nb).astype(np.float64)
    return vals.reshape(n, nb * 256), ls.reshape(n, nb * 8), d


def np_q81(act_bytes):
    b = act_bytes.reshape(-1, 36)
    d = b[:, 0:2].copy().view(np.float16).reshape(-1).astype(np.float64)
    q = b[:, 4:].copy().view(np.int8).astype(np.int64)
    return d, q


def np_dequant(dtype, w):
    n = w.shape[0]
    if dtype in (oracle.Q4_K, oracle.Q5_K):
        codes, sc, mn, d, dmin = (np_codes_q4k if dtype == oracle.Q4_K else np_codes_q5k)(w)
        scale = np.repeat(sc * np.repeat(d, 8, axis=1), 32, axis=1)
        off = np.repeat(mn * np.repeat(dmin, 8, axis=1), 32, axis=1)
        return scale * codes - off
    if dtype == oracle.Q6_K:
        codes, sc, d = np_codes_q6k(w)
        return np.repeat(sc * np.repeat(d, 16, axis=1), 16, axis=1) * codes
    if dtype in LEGACY.values():
        codes, d, m = np_codes_legacy(dtype, w)
        return np.repeat(d, 32, axis=1) * codes + np.repeat(m, 32, axis=1)
    if dtype == oracle.IQ4_XS:
        vals, ls, d = np_codes_iq4xs(w)
        return np.repeat(ls * np.repeat(d, 8, axis=1), 32, axis=1) * vals
    if dtype in LOWBIT.values():
        vals, sc, mn, d, dmin = np_codes_lowbit(dtype, w)
        return (np.repeat(sc * np.repeat(d, 16, axis=1), 16, axis=1) * vals
                - np.repeat(mn * np.repeat(dmin, 16, axis=1), 16, axis=1))
    codes, d = np_codes_q80(w)
    return np.repeat(d, 32, axis=1) * codes


def test_numpy_decoders_agree_with_ggml(ggml_vectors):
    for name, dtype in (("q4_K", oracle.Q4_K), ("q5_K", oracle.Q5_K), ("q6_K", oracle.Q6_K), ("q8_0", oracle.Q8_0),
                        ("q4_0", oracle.Q4_0), ("q4_1", oracle.Q4_1), ("q5_0", oracle.Q5_0), ("q5_1", oracle.Q5_1),
                        ("mxfp4", oracle.MXFP4), ("q2_K", oracle.Q2_K), ("q3_K", oracle.Q3_K)):
        rec = ggml_vectors[name]
        w = rec["quant"].reshape(1, -1, rec["block_bytes"])
        got = np_dequant(dtype, w).reshape(-1)
        np.testing.assert_allclose(got, rec["dequant"].astype(np.float64), rtol=2e-7, atol=0)


@pytest.mark.parametrize("name", sorted(DT))
def test_integer_subdots_match_numpy_brute_force(name):
    dtype = DT[name]
    n, k = 16, 1024
    w = synth.weight(dtype, n, k, seed=11, stream=1)
    x = synth.activation(1, k, seed=11)
    act = oracle.quantize_q8_1(x)
    dots, sums = oracle.ob_subdots(dtype, k, n, w, act)
    _, q = np_q81(act)
    q = q.reshape(-1)
    assert sums.tolist() == q.reshape(-1, 32).sum(axis=1).tolist()
    if dtype in (oracle.Q4_K, oracle.Q5_K):
        codes = (np_codes_q4k if dtype == oracle.Q4_K else np_codes_q5k)(w)[0]
        want = (codes * q[None, :]).reshape(n, k // 32, 32).sum(axis=2)
    elif dtype == oracle.Q6_K:
        codes = np_codes_q6k(w)[0]
        want = (codes * q[None, :]).reshape(n, k // 16, 16).sum(axis=2)
    elif dtype in LOWBIT.values():
        want = (np_codes_lowbit(dtype, w)[0] * q[None, :]).reshape(n, k // 16, 16).sum(axis=2)
    elif dtype == oracle.IQ4_XS:
        want = (np_codes_iq4xs(w)[0] * q[None, :]).reshape(n, k // 32, 32).sum(axis=2)
    else:
        codes = np_codes_legacy(dtype, w)[0] if dtype in LEGACY.values() else np_codes_q80(w)[0]
        want = (codes * q[None, :]).reshape(n, k // 32, 32).sum(axis=2)
    assert dots.astype(np.int64).tolist() == want.tolist()


def test_q4k_extreme_subdot_value():
    # all-15 nibbles against all-127 activations: 15 * 127 * 32 = 60960 per sub-block
    w = np.zeros((1, 1, 144), np.uint8)
    w[..., 16:] = 0xFF
    x = np.full((1, 256), 127.0, np.float32)
    dots, sums = oracle.ob_subdots(oracle.Q4_K, 256, 1, w, oracle.quantize_q8_1(x))
    assert dots.tolist() == [[60960] * 8] and sums.tolist() == [127 * 32] * 8


def test_q4k_reduces_to_int8_gemv_when_scales_are_one():
    # sc = 1, m = 0, d = 1, activations on the exact grid with d8 = 1: out = nibbles @ codes
    rng = np.random.default_rng(12)
    n, k = 8, 512
    w = synth.weight(oracle.Q4_K, n, k, seed=12)
    w[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w[:, :, 2:4] = 0
    w[:, :, 4:16] = oracle.pack_scales_mins([1] * 8, [0] * 8)
    a = rng.integers(-127, 128, (2, k))
    a[:, ::32] = 127
    x = a.astype(np.float32)
    want = a @ np_codes_q4k(w)[0].T
    got_b = oracle.ob_matmul(oracle.Q4_K, x, w, n)
    assert got_b.astype(np.int64).tolist() == want.tolist()


@pytest.mark.parametrize("name", sorted(DT))
@pytest.mark.parametrize("m", [1, 4])
def test_same_codes_f32_is_the_f64_product_up_to_rounding(name, m):
    dtype = DT[name]
    n, k = 24, 2048
    w = synth.weight(dtype, n, k, seed=13, stream=2)
    x = synth.activation(m, k, seed=13)
    got = oracle.ob_matmul(dtype, x, w, n)
    ref = oracle.ob_matmul_f64(dtype, x, w, n)
    # independent f64: numpy decoders on both operands
    d8, q8 = np_q81(oracle.quantize_q8_1(x))
    xa = (q8 * d8[:, None]).reshape(m, k)
    ref_np = xa @ np_dequant(dtype, w).T
    np.testing.assert_allclose(ref, ref_np, rtol=1e-12, atol=1e-15)
    # f32 accumulation over k/32 terms: error far below the 1e-3 parity tolerance
    absdot = np.abs(xa) @ np.abs(np_dequant(dtype, w)).T
    assert (np.abs(got - ref) <= 2e-6 * absdot + 1e-9).all()


@pytest.mark.parametrize("name", sorted(DT))
@pytest.mark.parametrize("m", [1, 4])
def test_served_path_matches_f64_over_dequantized_weights(name, m):
    # the reference's own matmul-level check and tolerance (quantized/tests.rs:576-632)
    dtype = DT[name]
    n, k = 16, 1024
    w = synth.weight(dtype, n, k, seed=14, stream=3)
    x = synth.activation(m, k, seed=14)
    got = oracle.oa_matmul(dtype, x, w, n)
    wd = np_dequant(dtype, w)
    ref = x.astype(np.float64) @ wd.T
    bound = 5e-3 * (np.abs(x.astype(np.float64)) @ np.abs(wd).T) + 1e-3
    assert (np.abs(got - ref) <= bound).all()
    # and it is the exact-fold variant up to f32 summation order
    if dtype in (oracle.Q4_K, oracle.Q6_K):   # the formats the reference states an exact fold for
        ex = oracle.oa_matmul(dtype, x, w, n, exact=True)
        assert (np.abs(ex - got) <= 1e-3 * np.maximum(np.abs(got), 1.0)).all()


def crafted_exact_case(dtype, n, nb, seed):
    """Weights with d = dmin = 1 and small scales, activations on the integer grid with -127 leading every
    super-block (Q8_K then has d = 1 and the codes are the values): every f32 operation of the exact fold is
    exact, so the result is the integer product of the dequantized weights with the activations."""
    rng = np.random.default_rng(seed)
    one = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    if dtype == oracle.Q4_K:
        w = np.zeros((n, nb, 144), np.uint8)
        w[:, :, 0:2] = one
        w[:, :, 2:4] = one
        sc = rng.integers(0, 8, size=(n, nb, 8), dtype=np.uint8)
        mn = rng.integers(0, 8, size=(n, nb, 8), dtype=np.uint8)
        w[:, :, 4:8] = sc[:, :, 0:4]
        w[:, :, 8:12] = mn[:, :, 0:4]
        w[:, :, 12:16] = sc[:, :, 4:8] | (mn[:, :, 4:8] << 4)   # six-bit values below 16: no high bits to place
        w[:, :, 16:] = rng.integers(0, 256, size=(n, nb, 128), dtype=np.uint8)
    else:
        w = np.zeros((n, nb, 210), np.uint8)
        w[:, :, 0:192] = rng.integers(0, 256, size=(n, nb, 192), dtype=np.uint8)
        w[:, :, 192:208] = rng.integers(-7, 8, size=(n, nb, 16)).astype(np.int8).view(np.uint8)
        w[:, :, 208:210] = one
    x = rng.integers(-126, 127, size=(3, nb * 256)).astype(np.float32)
    x.reshape(3, nb, 256)[:, :, 0] = -127.0
    return w.reshape(n, -1), x


@pytest.mark.parametrize("name", ["q4_k", "q6_k"])
def test_exact_fold_is_the_integer_product_where_every_step_is_exact(name):
    # pins oa_matmul_exact (dot_exact, q4_k.rs:117-156, q6_k.rs:121-163) without retyping its loops: a dropped
    # min term, a wrong bsum index or a sign would change the integer
    dtype = DT[name]
    n, nb = 12, 4
    w, x = crafted_exact_case(dtype, n, nb, seed=16)
    got = oracle.oa_matmul(dtype, x, w, n, exact=True)
    wd = np_dequant(dtype, w.reshape(n, nb, -1))
    want = x.astype(np.int64) @ np.rint(wd).astype(np.int64).T
    assert np.abs(want).max() < 2 ** 24
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, np.rint(got))
    # all-zero activations: the fold starts from -0.0 and every block adds +0.0 or -0.0 terms to it
    z = oracle.oa_matmul(dtype, np.zeros((1, nb * 256), np.float32), w, n, exact=True)
    assert np.array_equal(z, np.zeros_like(z))


@pytest.mark.parametrize("name", sorted(DT))
def test_served_path_integer_core_with_q8k_codes(name):
    # f64 product of dequantized weights with dequantized O-A activations: pins the Q8_K / Q8_0
    # pairing and the bsums use, independent of the oracle's loops.
    dtype = DT[name]
    n, k = 8, 768
    w = synth.weight(dtype, n, k, seed=15, stream=4)
    x = synth.activation(2, k, seed=15)
    slack = 0.0
    if dtype in (oracle.Q8_0, oracle.Q4_0, oracle.Q5_0, oracle.IQ4_NL, oracle.MXFP4):
        xa = oracle.dequantize(oracle.Q8_0, oracle.quantize_q8_0(x)).reshape(2, k)
    elif dtype == oracle.IQ4_XS:   # per-32 runs quantized as Q8_1 quantizes; no sum field is read
        d8, q = np_q81(oracle.quantize_q8_1(x))
        xa = (d8[:, None] * q).reshape(2, k)
    elif dtype in (oracle.Q4_1, oracle.Q5_1):
        # these pair with Q8_1 and take the block's sum from its f16 `s` field: the minimum's term
        # carries that field's rounding (2^-11 of |m * s| per block)
        d8, q = np_q81(oracle.quantize_q8_1(x))
        xa = (d8[:, None] * q).reshape(2, k)
        m = np.abs(np_codes_legacy(dtype, w)[2])                                   # [n, nb]
        s_abs = np.abs(xa.reshape(2, k // 32, 32).sum(axis=2))                     # [rows, nb]
        slack = 2.0 ** -11 * (s_abs @ m.T)
    else:
        xa = oracle.dequantize(oracle.Q8_K, oracle.quantize_q8_k(x)).reshape(2, k)
    wd = np_dequant(dtype, w)
    ref = xa.astype(np.float64) @ wd.T
    got = oracle.oa_matmul(dtype, x, w, n)
    absdot = np.abs(xa.astype(np.float64)) @ np.abs(wd).T
    assert (np.abs(got - ref) <= 4e-6 * absdot + 1e-9 + slack).all()


@pytest.mark.parametrize("name", FAST)
@pytest.mark.parametrize("m,threads", [(1, 1), (1, 3), (5, 4), (9, 2)])
def test_threaded_avx2_baseline_matches_scalar_path(name, m, threads):
    dtype = DT[name]
    n, k = 100, 1024
    w = synth.weight(dtype, n, k, seed=16, stream=5)
    x = synth.activation(m, k, seed=16)
    slow = oracle.oa_matmul(dtype, x, w, n)
    fast = oracle.oa_matmul(dtype, x, w, n, fast_threads=threads)
    assert (np.abs(fast - slow) <= 1e-3 * np.maximum(np.abs(slow), 1.0)).all()


def test_driver_error_conditions():
    w = synth.weight(oracle.Q4_K, 4, 512, seed=1)
    x = np.zeros((1, 500), np.float32)
    with pytest.raises(oracle.OracleError, match="multiple of the block"):
        oracle.oa_matmul(oracle.Q4_K, x, w, 4)
    with pytest.raises(oracle.OracleError, match="byte length"):
        oracle.oa_matmul(oracle.Q4_K, np.zeros((1, 512), np.float32), w, 5)
    with pytest.raises(oracle.OracleError, match="not handled"):
        oracle.oa_matmul(19, np.zeros((1, 512), np.float32), w, 4)   # IQ1_S: no statement of it here


def test_empty_rows_and_columns():
    w = synth.weight(oracle.Q4_K, 4, 256, seed=1)
    assert oracle.ob_matmul(oracle.Q4_K, np.zeros((0, 256), np.float32), w, 4).shape == (0, 4)
    assert oracle.oa_matmul(oracle.Q4_K, np.zeros((0, 256), np.float32), w, 4).shape == (0, 4)
    assert oracle.ob_matmul(oracle.Q4_K, np.zeros((2, 256), np.float32), w[:0], 0).shape == (2, 0)

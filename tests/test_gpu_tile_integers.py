"""The integer sub-block dot products of the PRODUCT kernels, bit for bit.

The parity probe (lk_mmvq_subdots) shows the integers of the mat-vec cores. The tiled kernels
(int8 MFMA tiles, the f16-operand Q4_K tiles, the rows-on-matrix-unit kernel) and the mat-vec
launches themselves are pinned here without a probe: the inputs are built so that the f32 output
of the shipped kernel IS one sub-block integer per weight block, summed over the row's blocks:

  * activations are integers in [-127, 127] with one 127 per 32-block, so every Q8_1 scale is
    exactly 1.0 and the codes are the values (the construction of
    src/inference/moe_cuda/imma_reference.rs:17-29 with the scale 2^-6 left out);
  * every weight block keeps its random quants but gets d = 1, dmin = 0 and a scale of 1 on ONE
    sub-block and 0 on the others (Q8_0: d = 1 on one block in eight), so
    out[token, row] = sum over blocks of D_s(block, row, token), an integer below 2^24 that f32
    holds exactly whatever the order of the additions;
  * for Q4_K / Q5_K the min term is isolated the same way (d = 0, dmin = 1, one min of 1):
    out = -sum over blocks of S_s(block, token), the integer sum of the activation codes.

Expected values are the oracle's integers (oracle.ob_subdots: the inner sums of
BlockQ4K::dot_scalar, format/q4_k.rs:62-88; q6_k.rs:51-82; q8_0.rs:83-97), summed over blocks in
int64. Equality is exact.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, ops, synth

pytestmark = pytest.mark.gpu

Q4K, Q5K, Q6K, Q80 = lib.TYPE_Q4_K, lib.TYPE_Q5_K, lib.TYPE_Q6_K, lib.TYPE_Q8_0
ONE = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
NIBBLE32 = {lib.TYPE_Q4_0: (18, None), lib.TYPE_Q4_1: (20, 2), lib.TYPE_Q5_0: (22, None), lib.TYPE_Q5_1: (24, 2)}
Q3K, Q2K = lib.TYPE_Q3_K, lib.TYPE_Q2_K
SUBS = {Q4K: 8, Q5K: 8, Q6K: 16, Q80: 8, Q3K: 16, Q2K: 16, **{t: 8 for t in NIBBLE32}}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def grid_activation(m, k, seed):
    rng = np.random.default_rng(seed)
    a = rng.integers(-127, 128, (m, k))
    a[:, ::32] = 127
    # a few blocks of extremes: every code +-127
    a[0, :32] = 127
    a[m - 1, 32:64] = -127
    a[m - 1, 32] = 127
    return a.astype(np.float32)


def isolate(wtype, w, s, min_term=False):
    """A copy of the blocks `w` [n, nb, bytes] in which only sub-block `s` of every block counts, with scale 1."""
    w = w.copy()
    if wtype in (Q4K, Q5K):
        sc = np.zeros(w.shape[:2] + (8,), np.uint8)
        mn = np.zeros_like(sc)
        (mn if min_term else sc)[..., s] = 1
        w[..., 4:16] = synth.pack_scales_mins(sc, mn)
        w[..., 0:2] = 0 if min_term else ONE
        w[..., 2:4] = ONE if min_term else 0
    elif wtype == Q6K:
        w[..., 192:208] = 0
        w[..., 192 + s] = 1
        w[..., 208:210] = ONE
    elif wtype == Q3K:
        # six-bit scales less 32: 33 for sub-block s, 32 for the rest (low nibble i / 8 of byte i % 8,
        # top two bits in field i / 4 of byte 8 + i % 4)
        w[..., 96:104] = 0
        w[..., 104:108] = 0xAA
        w[..., 96 + s % 8] = 1 << (4 * (s // 8))
        w[..., 108:110] = ONE
    elif wtype == Q2K:
        # byte g of the header: scale | minimum << 4 of group g
        w[..., 0:16] = 0
        w[..., s] = 16 if min_term else 1
        w[..., 80:82] = 0 if min_term else ONE
        w[..., 82:84] = ONE if min_term else 0
    elif wtype in NIBBLE32:
        # [n, blocks of 32, bytes]: scale 1 on every eighth block, no minimum (or the reverse)
        m_at = NIBBLE32[wtype][1]
        w[..., 0:2] = 0
        if m_at is not None:
            w[..., m_at:m_at + 2] = 0
        at = m_at if min_term else 0
        w[:, s::8, at:at + 2] = ONE
    else:
        w[..., 0:2] = 0
        w[:, s::8, 0:2] = ONE
    return w


def expected(wtype, w, x, s, min_term=False):
    """[m, n] f64: sum over blocks of the oracle's integer of sub-block `s` (or minus the code sums)."""
    n, k = w.shape[0], x.shape[1]
    per = SUBS[wtype] if wtype != Q80 else 8
    out = np.empty((x.shape[0], n), np.float64)
    for t in range(x.shape[0]):
        q = oracle.quantize_q8_1(x[t])
        dots, sums = oracle.ob_subdots(wtype, k, n, w, q)
        if min_term and wtype == Q2K:
            # the sums per 16 codes, which the Q8_1 row does not carry: from its codes
            codes = q.reshape(-1, 36)[:, 4:].view(np.int8).astype(np.int64).reshape(-1, 16, 16)
            out[t, :] = -float(codes[:, s, :].sum())
        elif min_term:
            # K-quants subtract dmin * m * sum, the 32-value formats add m * sum
            sign = 1.0 if wtype in NIBBLE32 else -1.0
            out[t, :] = sign * float(sums.reshape(-1, 8)[:, s].astype(np.int64).sum())
        else:
            out[t] = dots.reshape(n, -1, per)[:, :, s].astype(np.int64).sum(axis=1)
    return out


def check(run, wtype, n, k, m, seed, subs=None):
    w = synth.weight(wtype, n, k, seed=seed, stream=wtype)
    x = grid_activation(m, k, seed)
    # the activation really is its own code grid
    q = oracle.quantize_q8_1(x[0]).reshape(-1, 36)
    assert (q[:, 0:2].copy().view(np.float16) == 1.0).all() and np.array_equal(q[:, 4:].view(np.int8).reshape(-1), x[0].astype(np.int8))
    xd = dev(x)
    for s in (range(SUBS[wtype]) if subs is None else subs):
        got = run(dev(isolate(wtype, w, s)), xd).cpu().numpy().astype(np.float64)
        assert np.array_equal(got, expected(wtype, w, x, s)), f"sub-block {s}"
    if wtype in (Q4K, Q5K, Q2K) or NIBBLE32.get(wtype, (0, None))[1] is not None:
        for s in (((0, 3, 4, 7, 9, 15) if wtype == Q2K else (0, 3, 4, 7)) if subs is None else subs[:1]):
            got = run(dev(isolate(wtype, w, s, min_term=True)), xd).cpu().numpy().astype(np.float64)
            assert np.array_equal(got, expected(wtype, w, x, s, min_term=True)), f"min term of sub-block {s}"


# m <= 64: the int8 tiles (TM 32 / 64); above: TM 128, and for Q4_K the f16-operand tiles
@pytest.mark.parametrize("wtype", [Q4K, Q5K, Q6K, Q80, Q3K, Q2K] + sorted(NIBBLE32))
@pytest.mark.parametrize("m", [5, 40, 64, 65, 130])
def test_tiled_matmul_emits_the_exact_subblock_integers(wtype, m):
    n, k = 96, 1024
    check(lambda w, x: ops.mmq_forward(wtype, w, x, n), wtype, n, k, m, seed=80 + m)


def test_q4k_int8_tiles_above_64_rows_emit_the_exact_integers(knobs):
    knobs.set("LK_MMQ_I8")
    n, k, m = 96, 1024, 130
    check(lambda w, x: ops.mmq_forward(Q4K, w, x, n), Q4K, n, k, m, seed=91)


# up to 8 rows: registers only; up to 16: the staged form; up to 32: weights straight into the operand
@pytest.mark.parametrize("m", [3, 8, 12, 16, 24, 32])
def test_rows_on_matrix_unit_emit_the_exact_subblock_integers(m):
    n, k = 160, 1024
    check(lambda w, x: ops.dense_q4k_rows(w, x, n), Q4K, n, k, m, seed=100 + m)


# the mat-vec launches themselves: one row = the register-resident Q4_K engine, more = the staged engines
@pytest.mark.parametrize("wtype", [Q4K, Q5K, Q6K, Q80])
@pytest.mark.parametrize("m,k", [(1, 1024), (1, 4096), (4, 1024), (8, 2048)])
def test_matvec_launches_emit_the_exact_subblock_integers(wtype, m, k):
    n = 70
    check(lambda w, x: ops.mmvq(wtype, w, ops.quantize_q8_1_rows(x), k, n), wtype, n, k, m, seed=120 + m,
          subs=None if k == 1024 else [0, 5])


@pytest.mark.parametrize("k", [768, 2048, 4096])
def test_fused_and_pair_launches_ride_the_same_integers(k):
    # the in-kernel quantizing launch at one row: same integers as the two-launch path
    n = 64
    w = synth.weight(Q4K, n, k, seed=130, stream=1)
    x = grid_activation(1, k, 130)
    for s in (1, 6):
        wi = dev(isolate(Q4K, w, s))
        got = ops.mmvq_fused(Q4K, [wi], dev(x), [n])[0].cpu().numpy().astype(np.float64)
        assert np.array_equal(got, expected(Q4K, w, x, s))

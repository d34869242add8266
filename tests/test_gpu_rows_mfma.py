"""GPU parity of the matrix-unit path for a handful of activation rows (Q4_K x plain Q8_1 rows,
the library's loken_dense_q4k_imma_m8_plain).

Bars: f32 outputs within 1e-3 relative + 1e-4 absolute of the same-codes oracle (the integer
sub-block dots are the ones the mat-vec family is checked on bit for bit; here they come out of
v_mfma_i32_32x32x32_i8); agreement with the mat-vec family to summation order; a row's result
does not depend on how many other rows ride in the pass.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, ops, synth

pytestmark = pytest.mark.gpu

Q4K = lib.TYPE_Q4_K
RTOL, ATOL = 1e-3, 1e-4


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    bad = np.abs(got - want) > RTOL * np.abs(want) + ATOL
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; worst {np.abs(got - want).max()}"


@pytest.mark.parametrize("m,k,n", [(1, 256, 32), (5, 256, 64), (8, 2048, 70), (16, 1024, 130), (17, 512, 64), (32, 768, 33), (33, 512, 96),
                                   (70, 2048, 257), (9, 14336, 40), (12, 4096, 1024)])
def test_rows_on_the_matrix_unit_match_same_codes_oracle(m, k, n):
    w = synth.weight(Q4K, n, k, seed=60, stream=1)
    x = synth.activation(m, k, seed=60)
    got = ops.dense_q4k_rows(dev(w), dev(x), n).cpu().numpy()
    assert_close(got, oracle.ob_matmul(Q4K, x, w, n))


def test_rows_agree_with_matvec_family():
    m, k, n = 24, 4096, 600
    w = dev(synth.weight(Q4K, n, k, seed=61, stream=2))
    x = dev(synth.activation(m, k, seed=61))
    got = ops.dense_q4k_rows(w, x, n)
    q = ops.quantize_q8_1_rows(x)
    rows = torch.cat([ops.mmvq(Q4K, w, q[i:i + 8], k, n) for i in range(0, m, 8)])
    # same integers on both sides: only f32 summation order differs
    assert (got - rows).abs().max().item() <= 2e-5 * rows.abs().max().item()


def test_a_row_does_not_depend_on_its_company():
    # A launch is compiled for at most 8, at most 16 or more activation rows. Within one of these
    # classes a row carries the same bits whatever rides with it; across classes only the f32 order
    # of the min term differs (vector arithmetic below 17 rows, the matrix unit above).
    m, k, n = 40, 1024, 200
    w = dev(synth.weight(Q4K, n, k, seed=62, stream=3))
    x = dev(synth.activation(m, k, seed=62))
    full = ops.dense_q4k_rows(w, x, n)
    scale = full.abs().max().item()
    for rows in (list(range(10, 40)), list(range(0, 17)), list(range(5, 38))):
        assert torch.equal(ops.dense_q4k_rows(w, x[rows].contiguous(), n), full[rows])
    eight = ops.dense_q4k_rows(w, x[:8].contiguous(), n)
    for rows in ([0], [3, 4, 5], [7, 0]):
        assert torch.equal(ops.dense_q4k_rows(w, x[rows].contiguous(), n), eight[rows])
    sixteen = ops.dense_q4k_rows(w, x[8:24].contiguous(), n)
    for rows in (list(range(0, 9)), list(range(3, 16))):
        assert torch.equal(ops.dense_q4k_rows(w, x[8:24][rows].contiguous(), n), sixteen[rows])
    assert (eight - full[:8]).abs().max().item() <= 2e-6 * scale
    assert (sixteen - full[8:24]).abs().max().item() <= 2e-6 * scale


def test_full_gate_shape_against_matvec_and_sampled_oracle():
    m, k, n = 16, 4096, 14336
    w = synth.weight(Q4K, n, k, seed=0, stream=30)
    x = synth.activation(m, k, seed=0, stream=31)
    wd, xd = dev(w), dev(x)
    got = ops.dense_q4k_rows(wd, xd, n)
    q = ops.quantize_q8_1_rows(xd)
    vec = torch.cat([ops.mmvq(Q4K, wd, q[i:i + 8], k, n) for i in range(0, m, 8)])
    assert (got - vec).abs().max().item() <= 2e-5 * vec.abs().max().item()
    rng = np.random.default_rng(63)
    wr = np.sort(rng.choice(n, 300, replace=False))
    assert_close(got.cpu().numpy()[:, wr], oracle.ob_matmul(Q4K, x, w[wr], len(wr)))


def gelu_tanh(g):
    return 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))


def silu(g):
    return g / (1.0 + np.exp(-g))


@pytest.mark.parametrize("m,k,n", [(1, 256, 32), (5, 512, 70), (8, 2048, 257), (13, 1024, 130), (16, 768, 33), (33, 512, 96),
                                   (70, 2048, 64), (3, 14336, 40)])
@pytest.mark.parametrize("use_gelu", [False, True])
def test_gate_and_up_in_one_launch_match_the_closed_form_over_the_oracles_products(m, k, n, use_gelu):
    """loken_dense_q4k_imma_m8_actmul: the two products are the same-codes oracle's, the activation
    on top of them the closed form the reference's epilogue states (cuda/moe/dense_q4k_imma_m8.cu:
    33-58)."""
    gate = synth.weight(Q4K, n, k, seed=61, stream=1)
    up = synth.weight(Q4K, n, k, seed=61, stream=2)
    x = synth.activation(m, k, seed=61) * np.float32(4.0)
    g = oracle.ob_matmul(Q4K, x, gate, n).astype(np.float64)
    u = oracle.ob_matmul(Q4K, x, up, n).astype(np.float64)
    want = (gelu_tanh(g) if use_gelu else silu(g)) * u
    got = ops.dense_q4k_rows_actmul(dev(gate), dev(up), dev(x), n, use_gelu).cpu().numpy()
    assert (np.abs(got - want) <= RTOL * np.abs(want) + ATOL * max(1.0, np.abs(want).max())).all()


def test_gate_and_up_in_one_launch_carry_the_plain_launches_bits():
    """The dual launch's products are the plain launch's, bit for bit: SiLU(g) * u recomputed in f32
    from the two plain outputs differs only by the device's exp."""
    m, k, n = 7, 4096, 1024
    gate, up = dev(synth.weight(Q4K, n, k, seed=62, stream=1)), dev(synth.weight(Q4K, n, k, seed=62, stream=2))
    x = dev(synth.activation(m, k, seed=62))
    g, u = ops.dense_q4k_rows(gate, x, n).double(), ops.dense_q4k_rows(up, x, n).double()
    want = g / (1.0 + torch.exp(-g)) * u
    got = ops.dense_q4k_rows_actmul(gate, up, x, n, False).double()
    assert ((got - want).abs() <= 2e-6 * want.abs() + 1e-30).all()


Q5K = lib.TYPE_Q5_K


@pytest.mark.parametrize("m,k,n", [(1, 256, 32), (6, 512, 70), (8, 2048, 257), (16, 1024, 130), (33, 768, 96), (70, 2048, 64),
                                   (4, 14336, 40)])
def test_q5k_rows_on_the_matrix_unit_match_same_codes_oracle(m, k, n):
    """loken_dense_q5k_imma_m8_plain: the fifth bit joins the nibble before the matrix instruction."""
    w = synth.weight(Q5K, n, k, seed=63, stream=1)
    x = synth.activation(m, k, seed=63)
    got = ops.dense_q4k_rows(dev(w), dev(x), n, q5=True).cpu().numpy()
    assert_close(got, oracle.ob_matmul(Q5K, x, w, n))
    # the mat-vec family reads the same blocks another way: same integers, different summation order
    if m <= 8:
        other = ops.mmvq(Q5K, dev(w), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
        assert (np.abs(got - other) <= 2e-5 * np.abs(other) + 1e-5 * np.abs(other).max()).all()


@pytest.mark.parametrize("m,k,n", [(3, 512, 70), (8, 2048, 130), (20, 1024, 64)])
@pytest.mark.parametrize("use_gelu", [False, True])
def test_q5k_gate_and_up_in_one_launch(m, k, n, use_gelu):
    gate = synth.weight(Q5K, n, k, seed=64, stream=1)
    up = synth.weight(Q5K, n, k, seed=64, stream=2)
    x = synth.activation(m, k, seed=64) * np.float32(4.0)
    g = oracle.ob_matmul(Q5K, x, gate, n).astype(np.float64)
    u = oracle.ob_matmul(Q5K, x, up, n).astype(np.float64)
    want = (gelu_tanh(g) if use_gelu else silu(g)) * u
    got = ops.dense_q4k_rows_actmul(dev(gate), dev(up), dev(x), n, use_gelu, q5=True).cpu().numpy()
    assert (np.abs(got - want) <= RTOL * np.abs(want) + ATOL * max(1.0, np.abs(want).max())).all()


Q6K = lib.TYPE_Q6_K


@pytest.mark.parametrize("m,k,n", [(1, 256, 32), (3, 512, 70), (8, 2048, 257), (8, 14336, 40), (9, 768, 64), (16, 1024, 130),
                                   (16, 14336, 33), (17, 512, 64), (32, 768, 33), (33, 512, 96), (70, 2048, 100)])
def test_q6k_rows_on_the_matrix_unit_match_same_codes_oracle(m, k, n):
    """Signed 6-bit codes through v_mfma_i32_32x32x32_i8, one 16-value group per lane half."""
    w = synth.weight(Q6K, n, k, seed=65, stream=1)
    x = synth.activation(m, k, seed=65)
    got = ops.dense_q6k_rows(dev(w), dev(x), n).cpu().numpy()
    assert_close(got, oracle.ob_matmul(Q6K, x, w, n))
    if m <= 8:   # the mat-vec family: the same integers, another summation order
        other = ops.mmvq(Q6K, dev(w), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
        assert (np.abs(got - other) <= 2e-5 * np.abs(other) + 1e-5 * np.abs(other).max()).all()


def test_q6k_rows_emit_the_exact_integers_on_crafted_inputs():
    """Activations on an integer grid with 127 in every block (d8 = 1), weights with d = 1 and scale
    1 in one group of each super-block and 0 elsewhere: the f32 output is that group's integer dot."""
    rng = np.random.default_rng(66)
    m, k, n = 8, 1024, 64
    nb = k // 256
    x = rng.integers(-127, 128, size=(m, k)).astype(np.float32)
    x.reshape(m, k // 32, 32)[:, :, 0] = 127.0
    w = np.zeros((n, nb, 210), np.uint8)
    w[:, :, :192] = rng.integers(0, 256, size=(n, nb, 192), dtype=np.uint8)
    group = rng.integers(0, 16, size=(n, nb))
    scales = np.zeros((n, nb, 16), np.int8)
    np.put_along_axis(scales, group[:, :, None], 1, axis=2)
    w[:, :, 192:208] = scales.view(np.uint8)
    w[:, :, 208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    got = ops.dense_q6k_rows(dev(w.reshape(n, -1)), dev(x), n).cpu().numpy()
    # the integer dot, from the format's layout
    ql, qh = w[:, :, :128].astype(np.int32), w[:, :, 128:192].astype(np.int32)
    codes = np.zeros((n, nb, 256), np.int32)
    for half in range(2):
        for qt in range(4):
            l = np.arange(32)
            nib = ql[:, :, 64 * half + 32 * (qt & 1) + l]
            nib = (nib >> 4) if qt & 2 else (nib & 15)
            hi = (qh[:, :, 32 * half + l] >> (2 * qt)) & 3
            codes[:, :, 128 * half + 32 * qt + l] = (nib | (hi << 4)) - 32
    mask = (np.arange(256)[None, None, :] // 16) == group[:, :, None]
    want = np.einsum("nbk,mbk->mn", (codes * mask).astype(np.int64), x.reshape(m, nb, 256).astype(np.int64))
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, got.astype(np.int64))


# ---------------------------------------------------------------------------------------------
# At most eight rows: 16-row tiles on v_mfma_i32_16x16x64_i8 (rows16_mfma.hip)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("m,k,n", [(1, 256, 1), (2, 256, 15), (3, 512, 17), (4, 768, 16), (7, 1024, 31), (8, 1280, 48),
                                   (8, 4096, 1000), (6, 4096, 4096), (8, 11008, 50), (5, 2048, 16400), (3, 256, 16500),
                                   (9, 256, 1), (10, 512, 17), (13, 1024, 31), (16, 1280, 48), (16, 4096, 1000), (12, 2048, 4096),
                                   (15, 11008, 50), (11, 2048, 16400), (16, 256, 16500)])
@pytest.mark.parametrize("wtype", [Q4K, lib.TYPE_Q5_K])
def test_eight_rows_or_fewer_in_sixteen_row_tiles(m, k, n, wtype):
    """Ragged tile edges (n not a multiple of 16), rows of one to 43 super-blocks (waves with no
    block of their own), every row count of the launch, and matrices of more than 1024 row tiles
    (four tiles per workgroup instead of two)."""
    w = synth.weight(wtype, n, k, seed=70, stream=1)
    x = synth.activation(m, k, seed=70)
    got = ops.dense_q4k_rows(dev(w), dev(x), n, q5=wtype != Q4K).cpu().numpy()
    assert_close(got, oracle.ob_matmul(wtype, x, w, n))


@pytest.mark.parametrize("m", [8, 16])
def test_eight_rows_emit_the_exact_integers_on_crafted_inputs(m):
    """Activations on an integer grid with 127 in every block (d8 = 1); weights with d = 1, dmin = 0
    and scale 1 in ONE sub-block of each super-block, 0 in the others: the f32 output is that
    sub-block's integer dot, so a code that strays into the neighbouring sub-block of its
    instruction (or a lane that should hold zeros and does not) shows."""
    rng = np.random.default_rng(71)
    k, n = 1024, 80
    nb = k // 256
    x = rng.integers(-127, 128, size=(m, k)).astype(np.float32)
    x.reshape(m, k // 32, 32)[:, :, 0] = 127.0
    w = np.zeros((n, nb, 144), np.uint8)
    w[:, :, 16:] = rng.integers(0, 256, size=(n, nb, 128), dtype=np.uint8)
    pick = rng.integers(0, 8, size=(n, nb))
    sc = (np.arange(8)[None, None, :] == pick[:, :, None]).astype(np.uint8)   # six-bit scales, mins 0
    # get_scale_min_k4: j < 4: sc = q[j] & 63; j >= 4: sc = (q[j + 4] & 15) | ((q[j - 4] >> 6) << 4)
    w[:, :, 4:8] = sc[:, :, 0:4]
    w[:, :, 12:16] = sc[:, :, 4:8]
    w[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    got = ops.dense_q4k_rows(dev(w.reshape(n, -1)), dev(x), n).cpu().numpy()
    qs = w[:, :, 16:].astype(np.int64).reshape(n, nb, 4, 32)
    codes = np.stack([qs & 15, qs >> 4], axis=3).reshape(n, nb, 8, 32)       # sub-block 2 p, 2 p + 1
    xs = x.reshape(m, nb, 8, 32).astype(np.int64)
    want = np.einsum("nbsk,mbsk,nbs->mn", codes, xs, sc.astype(np.int64))
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, got.astype(np.int64))


@pytest.mark.parametrize("m", [1, 5, 8, 11, 16, 19, 32, 33, 70])
@pytest.mark.parametrize("q5", [False, True])
def test_three_matrices_in_one_launch_carry_the_single_launches_bits(m, q5):
    """q + k + v: lk_dense_q4k_rows_multi against one lk_dense_q4k_rows per matrix."""
    k, sizes = 2048, (520, 130, 7)
    wtype = lib.TYPE_Q5_K if q5 else Q4K
    ws = [dev(synth.weight(wtype, n, k, seed=72, stream=i)) for i, n in enumerate(sizes)]
    x = dev(synth.activation(m, k, seed=72))
    outs = ops.dense_q4k_rows_multi(ws, x, sizes, q5=q5)
    for w, n, out in zip(ws, sizes, outs):
        assert torch.equal(out, ops.dense_q4k_rows(w, x, n, q5=q5))
    two = ops.dense_q4k_rows_multi(ws[:2], x, sizes[:2], q5=q5)
    assert torch.equal(two[0], outs[0]) and torch.equal(two[1], outs[1])


@pytest.mark.parametrize("m,k,n", [(8, 4096, 8200), (2, 512, 9000), (14, 2048, 8200)])
def test_gate_and_up_of_many_row_tiles(m, k, n):
    """The dual launch with four tiles (two gate, two up) per workgroup: bits of the plain launches."""
    gate, up = dev(synth.weight(Q4K, n, k, seed=73, stream=1)), dev(synth.weight(Q4K, n, k, seed=73, stream=2))
    x = dev(synth.activation(m, k, seed=73))
    g, u = ops.dense_q4k_rows(gate, x, n).double(), ops.dense_q4k_rows(up, x, n).double()
    want = g / (1.0 + torch.exp(-g)) * u
    got = ops.dense_q4k_rows_actmul(gate, up, x, n, False).double()
    assert ((got - want).abs() <= 2e-6 * want.abs() + 1e-30).all()
    w = synth.weight(Q4K, 64, k, seed=73, stream=1)
    assert_close(ops.dense_q4k_rows(gate[:64 * (k // 256) * 144], x, 64).cpu().numpy(), oracle.ob_matmul(Q4K, x.cpu().numpy(), w, 64))


@pytest.mark.parametrize("m,k,n", [(1, 2048, 32), (3, 4096, 96), (4, 2048, 6144), (8, 4096, 14336), (8, 2048, 160),
                                   (9, 4096, 64), (13, 2048, 6144), (16, 4096, 4128), (17, 2048, 6144), (33, 1024, 96),
                                   (64, 2048, 640), (100, 4096, 224)])
@pytest.mark.parametrize("q5", [False, True])
def test_gate_and_up_handed_on_as_q8_1_rows_are_the_quantizers_bytes(m, k, n, q5):
    """lk_dense_q4k_rows_actmul_q8_1 against lk_dense_q4k_rows_actmul followed by lk_quantize_q8_1, SiLU and GELU."""
    wt = lib.TYPE_Q5_K if q5 else Q4K
    gate, up = dev(synth.weight(wt, n, k, seed=77, stream=1)), dev(synth.weight(wt, n, k, seed=77, stream=2))
    x = dev(synth.activation(m, k, seed=77) * np.float32(3.0))
    for gelu in (False, True):
        h = ops.dense_q4k_rows_actmul(gate, up, x, n, gelu, q5=q5)
        want = ops.quantize_q8_1_rows(h, k_padded=n)
        got = ops.dense_q4k_rows_actmul_q8_1(gate, up, x, n, gelu, q5=q5)
        assert torch.equal(got.reshape(-1), want.reshape(-1))


def test_gate_and_up_as_q8_1_refuses_what_its_kernel_does_not_take():
    gate = dev(synth.weight(Q4K, 64, 1024, seed=78, stream=1))
    with pytest.raises(lib.LokenError):   # rows of 1024 values
        ops.dense_q4k_rows_actmul_q8_1(gate, gate, dev(synth.activation(4, 1024, seed=78)), 64, False)
    gate = dev(synth.weight(Q4K, 48, 2048, seed=78, stream=1))
    with pytest.raises(lib.LokenError):   # 48 output rows: not whole blocks
        ops.dense_q4k_rows_actmul_q8_1(gate, gate, dev(synth.activation(4, 2048, seed=78)), 48, False)


@pytest.mark.parametrize("m,k,n", [(1, 256, 1), (2, 512, 15), (3, 768, 17), (4, 1024, 33), (4, 14336, 48), (5, 256, 16), (7, 1280, 100),
                                   (8, 6144, 500), (6, 2048, 8300), (3, 512, 8300), (8, 512, 16500), (4, 256, 16500),
                                   (9, 2048, 17), (12, 6144, 500), (16, 4096, 100), (16, 2048, 8300), (13, 2048, 16500),
                                   (9, 14336, 48), (12, 14336, 100), (16, 14336, 33),
                                   (17, 2048, 100), (24, 6144, 500), (32, 4096, 33), (31, 14336, 48), (25, 2048, 8300),
                                   (64, 6144, 2048), (57, 2048, 1000), (40, 2048, 1024)])
def test_q6k_eight_rows_or_fewer_in_sixteen_row_tiles(m, k, n):
    """rows16_q6k.hip: both slot layouts (up to four rows, up to eight), ragged tile edges, rows of
    one super-block (waves with nothing to add), one, two and four tiles per workgroup; k = 14336 above
    eight rows: sixteen rows do not fit LDS and the rows go out as sets of eight over the launch's second grid
    axis, as do 17..32 rows of a matrix that L2 holds."""
    w = synth.weight(Q6K, n, k, seed=74, stream=1)
    x = synth.activation(m, k, seed=74)
    got = ops.dense_q6k_rows(dev(w), dev(x), n).cpu().numpy()
    assert_close(got, oracle.ob_matmul(Q6K, x, w, n))


@pytest.mark.parametrize("k", [1024, 4096])
@pytest.mark.parametrize("m", [3, 4, 7, 11, 16, 21, 32])
def test_q6k_few_rows_emit_the_exact_integers_on_crafted_inputs(m, k):
    """As test_q6k_rows_emit_the_exact_integers_on_crafted_inputs, for the launches of at most four
    and at most eight rows: one group of each super-block has scale 1, the others 0, so a code that
    strays into a neighbouring group of its instruction shows. k = 4096: rows of whole eight-block
    granules, whose super-blocks are read back from LDS at eight different byte offsets."""
    rng = np.random.default_rng(75 + m)
    n = 80
    nb = k // 256
    x = rng.integers(-127, 128, size=(m, k)).astype(np.float32)
    x.reshape(m, k // 32, 32)[:, :, 0] = 127.0
    w = np.zeros((n, nb, 210), np.uint8)
    w[:, :, :192] = rng.integers(0, 256, size=(n, nb, 192), dtype=np.uint8)
    group = rng.integers(0, 16, size=(n, nb))
    scales = np.zeros((n, nb, 16), np.int8)
    np.put_along_axis(scales, group[:, :, None], 1, axis=2)
    w[:, :, 192:208] = scales.view(np.uint8)
    w[:, :, 208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    got = ops.dense_q6k_rows(dev(w.reshape(n, -1)), dev(x), n).cpu().numpy()
    ql, qh = w[:, :, :128].astype(np.int32), w[:, :, 128:192].astype(np.int32)
    codes = np.zeros((n, nb, 256), np.int32)
    for half in range(2):
        for qt in range(4):
            l = np.arange(32)
            nib = ql[:, :, 64 * half + 32 * (qt & 1) + l]
            nib = (nib >> 4) if qt & 2 else (nib & 15)
            hi = (qh[:, :, 32 * half + l] >> (2 * qt)) & 3
            codes[:, :, 128 * half + 32 * qt + l] = (nib | (hi << 4)) - 32
    mask = (np.arange(256)[None, None, :] // 16) == group[:, :, None]
    want = np.einsum("nbk,mbk->mn", (codes * mask).astype(np.int64), x.reshape(m, nb, 256).astype(np.int64))
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, got.astype(np.int64))

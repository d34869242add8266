"""The timed CPU baseline's served Q4_K path (rows repacked eight at a time, one group dot per eight
columns, persistent worker pool) against the scalar oracle it is a faster statement of.

  * the repack is the reference's index map (repack_q4k.rs:44-68), checked byte by byte;
  * on inputs whose every factor is exactly representable the group dot returns the exact integer
    combination of the scalar definition (gemv_group_scalar, repack_q4k.rs:174-219): max abs 0;
  * on random inputs it stays inside the reference's own vector-vs-scalar bound
    1e-3 * max(|ref|, 1) (avx/parity.rs:50-56), for one row and for several;
  * the pool gives the same bits whatever its size (every output is one thread's own sum).
"""
import numpy as np
import pytest

import oracle
from loken_amd import synth

Q4K = oracle.Q4_K
pytestmark = pytest.mark.skipif(not oracle.lib().lko_cpu_has_avx2(), reason="needs AVX2")


def test_repack_places_every_byte_where_the_reference_puts_it():
    n, k = 16, 512
    nb = k // 256
    w = synth.weight(Q4K, n, k, seed=5)
    x8 = oracle.repack_q4k_x8(w, n, k).reshape(n // 8, nb, 1152)
    for g in range(n // 8):
        for b in range(nb):
            blk = x8[g, b]
            for j in range(8):
                src = w[g * 8 + j, b]
                assert np.array_equal(blk[2 * j:2 * j + 2], src[0:2])
                assert np.array_equal(blk[16 + 2 * j:18 + 2 * j], src[2:4])
                assert np.array_equal(blk[32 + 12 * j:44 + 12 * j], src[4:16])
                for p in range(128):
                    assert blk[128 + (p // 8) * 64 + j * 8 + p % 8] == src[16 + p]


def test_group_dot_is_the_exact_integer_combination():
    # d = dmin = 1, scales and mins small, activations integers with extreme -127: Q8_K's d is 1 and
    # its codes are the values, so every product and sum is an integer below 2^24
    rng = np.random.default_rng(11)
    n, k = 24, 1024
    nb = k // 256
    w = synth.weight(Q4K, n, k, seed=6)
    sc = rng.integers(0, 8, (n, nb, 8)).astype(np.uint8)
    mn = rng.integers(0, 8, (n, nb, 8)).astype(np.uint8)
    w[..., 4:16] = synth.pack_scales_mins(sc, mn)
    one = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    w[..., 0:2] = one
    w[..., 2:4] = one
    x = rng.integers(-127, 128, (3, k)).astype(np.float32)
    x[:, ::256] = -127.0
    qs = w[..., 16:144].reshape(n, nb, 4, 32)
    nibbles = np.stack([qs & 15, qs >> 4], axis=3).reshape(n, nb, 8, 32).astype(np.int64)   # [n, nb, sub-block, 32]
    a = x.astype(np.int64).reshape(3, nb, 8, 32)
    dots = np.einsum("nbsl,tbsl->tnbs", nibbles, a)
    want = (dots * sc[None].astype(np.int64)).sum(axis=(2, 3)) - (a.sum(axis=3)[:, None] * mn[None].astype(np.int64)).sum(axis=(2, 3))
    got = oracle.oa_matmul_q4k_x8(x, oracle.repack_q4k_x8(w, n, k), n)
    assert np.abs(want).max() < 2 ** 24
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("m", [1, 5])
def test_served_path_stays_inside_the_reference_bound(m):
    n, k = 264, 4096
    w = synth.weight(Q4K, n, k, seed=7)
    x = synth.activation(m, k, seed=7)
    ref = oracle.oa_matmul(Q4K, x, w, n)
    got = oracle.oa_matmul_q4k_x8(x, oracle.repack_q4k_x8(w, n, k), n)
    assert (np.abs(got - ref) <= 1e-3 * np.maximum(np.abs(ref), 1.0)).all()
    # the per-column vector driver shares the pool and the bound
    fast = oracle.oa_matmul(Q4K, x, w, n, fast_threads=3)
    assert (np.abs(fast - ref) <= 1e-3 * np.maximum(np.abs(ref), 1.0)).all()


def test_results_do_not_depend_on_the_pool_size():
    n, k = 512, 2048
    w = synth.weight(Q4K, n, k, seed=8)
    x = synth.activation(2, k, seed=8)
    x8 = oracle.repack_q4k_x8(w, n, k)
    outs = []
    for threads in (1, 2, 5, 0):
        assert oracle.pool_start(threads) >= 1
        outs.append(oracle.oa_matmul_q4k_x8(x, x8, n))
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])
    physical, logical = oracle.cpu_counts()
    assert 1 <= physical <= logical


def test_argument_errors():
    x = synth.activation(1, 256, seed=9)
    with pytest.raises(oracle.OracleError):
        oracle.oa_matmul_q4k_x8(x, np.zeros(1152 * 2, np.uint8), 12)   # n not a multiple of 8


def test_several_rows_per_pass_carry_the_one_row_kernels_bits():
    """vec_dot_q4k_q8k_many (avx/superblock.rs:425-490): out[t] is bit for bit the one-row kernel's."""
    k = 2048
    w = synth.weight(Q4K, 3, k, seed=12)
    x = synth.activation(7, k, seed=12)          # a pass of four, then a ragged one of three
    for row in range(3):
        many = oracle.dot_q4k_q8k_many(w[row], x)
        for t in range(7):
            one = np.float32(oracle.dot_q4k_q8k(w[row], x[t]))
            assert many[t] == one
    # and the one-row kernel is the scalar oracle's dot to the reference's vector-vs-scalar bound
    ref = oracle.oa_matmul(Q4K, x, w, 3)
    got = np.stack([oracle.dot_q4k_q8k_many(w[row], x) for row in range(3)], axis=1)
    assert (np.abs(got - ref) <= 1e-3 * np.maximum(np.abs(ref), 1.0)).all()


@pytest.mark.skipif(not oracle.lib().lko_cpu_has_avx512(), reason="needs AVX-512 with VNNI")
def test_the_512_bit_twin_returns_the_256_bit_kernels_bits():
    """avx512/superblock.rs:20-90: the same integer sums in wider registers, so the same float."""
    k = 4096
    w = synth.weight(Q4K, 16, k, seed=13)
    x = synth.activation(3, k, seed=13) * np.float32(5.0)
    for row in range(16):
        for t in range(3):
            assert oracle.dot_q4k_q8k(w[row], x[t], wide=True) == oracle.dot_q4k_q8k(w[row], x[t], wide=False)
    # extreme codes: every nibble 15, every activation at the quantizer's extreme
    w_hot = synth.weight(Q4K, 1, 512, seed=14)
    w_hot.reshape(-1, 144)[:, 16:] = 0xFF
    x_hot = np.full((1, 512), -3.0, np.float32)
    assert oracle.dot_q4k_q8k(w_hot[0], x_hot[0], wide=True) == oracle.dot_q4k_q8k(w_hot[0], x_hot[0], wide=False)


# ---- the served prefill forms (matmul_q4k_repacked_tiled / matmul_q6k_repacked_tiled, drivers.rs:231-406) ----

Q6K = oracle.Q6_K


@pytest.mark.parametrize("m", [1, 8, 19])
def test_tiled_q4k_prefill_carries_the_decode_drivers_bits_row_by_row(m):
    """A row's eight sums inside a tile are the decode path's group dot: the result of a row does not
    depend on how many rows travel with it, nor on the pool size."""
    n, k = 136, 1024
    w = synth.weight(Q4K, n, k, seed=21)
    x = synth.activation(m, k, seed=21)
    x8 = oracle.repack_q4k_x8(w, n, k)
    tiled = oracle.oa_matmul_q4k_x8_tiled(x, x8, n)
    for t in range(m):
        assert np.array_equal(tiled[t], oracle.oa_matmul_q4k_x8(x[t:t + 1], x8, n)[0])
    oracle.pool_start(3)
    assert np.array_equal(oracle.oa_matmul_q4k_x8_tiled(x, x8, n), tiled)
    oracle.pool_start(0)
    ref = oracle.oa_matmul(Q4K, x, w, n)
    assert (np.abs(tiled - ref) <= 1e-3 * np.maximum(np.abs(ref), 1.0)).all()


def test_q6k_repack_copies_each_columns_planes_verbatim():
    # BlockQ6Kx8 (repack_q6k.rs:17-64): d[8] f16, scales[8][16], ql[8][128], qh[8][64]
    n, k = 16, 512
    nb = k // 256
    w = synth.weight(Q6K, n, k, seed=22)
    x8 = oracle.repack_q6k_x8(w, n, k).reshape(n // 8, nb, 1680)
    for g in range(n // 8):
        for b in range(nb):
            blk = x8[g, b]
            for j in range(8):
                src = w[g * 8 + j, b]                      # ql[128] qh[64] scales[16] d
                assert np.array_equal(blk[2 * j:2 * j + 2], src[208:210])
                assert np.array_equal(blk[16 + 16 * j:32 + 16 * j], src[192:208])
                assert np.array_equal(blk[144 + 128 * j:272 + 128 * j], src[0:128])
                assert np.array_equal(blk[1168 + 64 * j:1232 + 64 * j], src[128:192])


def test_tiled_q6k_prefill_is_the_exact_integer_combination():
    # d = 1, scales small and of both signs, activations integers with an extreme of -127 per block so
    # that Q8_K's d is 1 and its codes are the values: every sum is an integer below 2^24. The
    # unsigned-codes-minus-zero-point arrangement of the vector kernel has to land on the same integer.
    rng = np.random.default_rng(23)
    n, k, m = 24, 1024, 11
    nb = k // 256
    w = synth.weight(Q6K, n, k, seed=23)
    w[..., 192:208] = rng.integers(-7, 8, (n, nb, 16)).astype(np.int8).view(np.uint8)
    w[..., 208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    x = rng.integers(-127, 128, (m, k)).astype(np.float32)
    x[:, ::256] = -127.0
    deq = oracle.dequantize(Q6K, w).reshape(n, k)
    assert np.array_equal(deq, np.round(deq)) and np.abs(deq).max() <= 32 * 7
    want = x.astype(np.int64) @ deq.astype(np.int64).T
    assert np.abs(want).max() < 2 ** 24
    got = oracle.oa_matmul_q6k_x8_tiled(x, oracle.repack_q6k_x8(w, n, k), n)
    assert np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("m", [1, 8, 19])
def test_tiled_q6k_prefill_stays_inside_the_reference_bound(m):
    n, k = 264, 2048
    nb = k // 256
    w = synth.weight(Q6K, n, k, seed=24)
    x = synth.activation(m, k, seed=24)
    x8 = oracle.repack_q6k_x8(w, n, k)
    ref = oracle.oa_matmul(Q6K, x, w, n)
    got = oracle.oa_matmul_q6k_x8_tiled(x, x8, n)
    assert (np.abs(got - ref) <= 1e-3 * np.maximum(np.abs(ref), 1.0)).all()
    # the vector tile against the reference's own scalar group dot (gemv_group_scalar, repack_q6k.rs:
    # 94-118): the integers are exact and the float fold is the same one product and one add per
    # block, so the two agree bit for bit
    for t in (0, m - 1):
        act = oracle.quantize_q8_k(x[t])
        for g in (0, n // 8 - 1):
            assert np.array_equal(oracle.gemv_group_q6k_x8_scalar(x8, g, nb, act), got[t, g * 8:g * 8 + 8])
    # a row's result does not depend on its companions in the tile or on the pool size
    oracle.pool_start(2)
    assert np.array_equal(oracle.oa_matmul_q6k_x8_tiled(x[m - 1:], x8, n)[0], got[m - 1])
    oracle.pool_start(0)


def test_tiled_argument_errors():
    x = synth.activation(2, 256, seed=25)
    with pytest.raises(oracle.OracleError):
        oracle.oa_matmul_q4k_x8_tiled(x, np.zeros(1152 * 2, np.uint8), 12)
    with pytest.raises(oracle.OracleError):
        oracle.oa_matmul_q6k_x8_tiled(x, np.zeros(1680 * 2, np.uint8), 12)


def test_pooled_expert_block_is_the_scalar_block_token_by_token():
    from loken_amd import workloads
    rng = np.random.default_rng(26)
    tokens, hidden, ffn, n_experts, topk = 13, 512, 256, 6, 2
    gate = synth.weight(Q4K, n_experts * ffn, hidden, seed=26)
    up = synth.weight(Q4K, n_experts * ffn, hidden, seed=27)
    down = synth.weight(Q6K, n_experts * hidden, ffn, seed=28)
    x = synth.activation(tokens, hidden, seed=26)
    ids = np.stack([rng.permutation(n_experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    weights = rng.random((tokens, topk)).astype(np.float32)
    for family in (0, 1):
        want = oracle.moe_forward(family, Q4K, Q6K, x, gate, up, down, ids, weights, n_experts, ffn)
        got = oracle.moe_forward_pool(family, Q4K, Q6K, x, gate, up, down, ids, weights, n_experts, ffn)
        assert np.array_equal(got, want)

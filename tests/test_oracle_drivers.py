"""The multi-expert CPU drivers of the served path (matmul_bytes_multi / matmul_bytes_grouped,
src/tensor/quant_cpu/drivers.rs:2144-2425) as the oracle states them.

The reference's contract is that each output is bit for bit the `dot` a single-matrix call gives
that (expert, row): that is what is checked, for K-quants and Q8_0, with ragged row counts and an
expert without rows, together with the error conditions the drivers name.
"""
import numpy as np
import pytest

import oracle
from loken_amd import synth

Q4K, Q6K, Q80 = oracle.Q4_K, oracle.Q6_K, oracle.Q8_0


@pytest.mark.parametrize("dtype", [Q4K, Q6K, Q80])
def test_multi_is_one_single_row_product_per_expert(dtype):
    k, n, ne = 512, 24, 5
    ws = [synth.weight(dtype, n, k, seed=90, stream=e) for e in range(ne)]
    xs = [synth.activation(1, k, seed=90, stream=e)[0] for e in range(ne)]
    outs = oracle.oa_matmul_multi(dtype, k, n, ws, xs)
    for e in range(ne):
        assert np.array_equal(outs[e], oracle.oa_matmul(dtype, xs[e][None, :], ws[e], n)[0])
    assert oracle.oa_matmul_multi(dtype, k, n, [], []) == []


@pytest.mark.parametrize("dtype", [Q4K, Q6K, Q80])
def test_grouped_is_one_product_per_expert_and_row(dtype):
    k, n = 256, 40
    rows = [3, 0, 1, 7]
    ws = [synth.weight(dtype, n, k, seed=91, stream=e) for e in range(len(rows))]
    xs = [synth.activation(max(r, 1), k, seed=91, stream=e)[:r] for e, r in enumerate(rows)]
    outs = oracle.oa_matmul_grouped(dtype, k, n, ws, xs)
    for e, r in enumerate(rows):
        assert outs[e].shape == (r, n)
        for i in range(r):
            assert np.array_equal(outs[e][i], oracle.oa_matmul(dtype, xs[e][i:i + 1], ws[e], n)[0])
        # and the multi driver on a row alone gives the same bits
        if r:
            assert np.array_equal(outs[e][0], oracle.oa_matmul_multi(dtype, k, n, [ws[e]], [xs[e][0]])[0])


def test_error_conditions_of_the_drivers():
    k, n = 256, 8
    w = synth.weight(Q4K, n, k, seed=92)
    x = synth.activation(2, k, seed=92)
    with pytest.raises(oracle.OracleError, match="multiple of the block"):
        oracle.oa_matmul_multi(Q4K, 200, n, [w], [x[0][:200]])
    with pytest.raises(oracle.OracleError, match="lhs entry"):
        oracle.oa_matmul_multi(Q4K, k, n, [w], [x.reshape(-1)])            # two rows where one is expected
    with pytest.raises(oracle.OracleError, match="outs entry"):
        oracle.oa_matmul_multi(Q4K, k, n, [w], [x[0]], out_lens=[n + 1])
    with pytest.raises(oracle.OracleError, match="rhs byte length"):
        oracle.oa_matmul_multi(Q4K, k, n, [w.reshape(-1)[:-144]], [x[0]])
    with pytest.raises(oracle.OracleError, match="lhs entry"):
        oracle.oa_matmul_grouped(Q4K, k, n, [w], [x.reshape(-1)[:k + 5]])  # not whole rows
    with pytest.raises(oracle.OracleError, match="outs entry"):
        oracle.oa_matmul_grouped(Q4K, k, n, [w], [x], out_shapes=[(3, n)])
    with pytest.raises(oracle.OracleError, match="dtype"):
        oracle.oa_matmul_grouped(99, k, n, [w], [x])

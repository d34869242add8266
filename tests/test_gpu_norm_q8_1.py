"""Decode-step producers that end in a Q8_1 row (lk_rmsnorm_q8_1, lk_add_rmsnorm_q8_1,
lk_post_norm_add_norm_q8_1, lk_split_act_mul_q8_1) against the oracle: the f32 rows bit for bit
for the norm family (same accumulation order, correctly rounded operations on both sides), within
1e-6 for the split activation (exp / tanh differ between the two math libraries in the last
place), and the Q8_1 rows byte for byte what the oracle's quantizer makes of the f32 row."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, ops, synth

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def q8_1_of(rows_f32):
    return np.stack([oracle.quantize_q8_1(r).reshape(-1, 36) for r in rows_f32])


def inputs(rows, cols, seed):
    x = (synth.normal(seed, 1, rows * cols) * 2.5).reshape(rows, cols)
    res = synth.normal(seed, 2, rows * cols).reshape(rows, cols)
    w = (1.0 + 0.2 * synth.normal(seed, 3, cols)).astype(np.float32)
    w2 = (1.0 + 0.2 * synth.normal(seed, 4, cols)).astype(np.float32)
    return x, res, w, w2


SHAPES = [(1, 512), (1, 4096), (3, 2048), (16, 6144), (2, 14336), (2, 20480)]


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_rmsnorm_row_and_its_q8_1(rows, cols):
    x, _, w, _ = inputs(rows, cols, 100 + cols)
    out, q = ops.rmsnorm_q8_1(dev(x), dev(w), 1e-5)
    assert np.array_equal(host(out), oracle.norm_rows(0, x, w, eps=1e-5))
    assert np.array_equal(host(q), q8_1_of(host(out)))
    # the blocks are what the stand-alone quantizer writes for that row
    assert torch.equal(q, ops.quantize_q8_1_rows(out))


@pytest.mark.parametrize("hidden", [512, 2048, 4096, 2080, 96, 14336])
def test_reference_named_single_row_launch_writes_the_same_blocks(hidden):
    # loken_rms_quantize_q8_1 / _bf16: Q8_1 only, any multiple of 32
    x, _, w, _ = inputs(1, hidden, 150 + hidden)
    want = oracle.norm_rows(0, x, w, eps=1e-5)
    q = ops.rms_quantize_q8_1(dev(x[0]), dev(w), 1e-5)
    assert np.array_equal(host(q), q8_1_of(want)[0])
    xb = dev(x[0]).to(torch.bfloat16)
    x_seen = xb.to(torch.float32).cpu().numpy()[None, :]
    qb = ops.rms_quantize_q8_1(xb, dev(w), 1e-5)
    assert np.array_equal(host(qb), q8_1_of(oracle.norm_rows(0, x_seen, w, eps=1e-5))[0])


def test_reference_named_single_row_launch_declines_bad_arguments():
    q = torch.full((4, 36), 7, dtype=torch.uint8, device="cuda")
    x = torch.ones(100, device="cuda")
    lib.load().loken_rms_quantize_q8_1(x.data_ptr(), x.data_ptr(), q.data_ptr(), 100, 1e-5, None)   # not a multiple of 32
    lib.load().loken_rms_quantize_q8_1(None, x.data_ptr(), q.data_ptr(), 96, 1e-5, None)
    torch.cuda.synchronize()
    assert (q == 7).all()


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_add_then_rmsnorm(rows, cols):
    x, res, w, _ = inputs(rows, cols, 200 + cols)
    total, out, q = ops.add_rmsnorm_q8_1(dev(x), dev(res), dev(w), 1e-6)
    want_total, want = oracle.norm_rows(1, x, w, residual=res, eps=1e-6)
    assert np.array_equal(host(total), want_total) and np.array_equal(host(out), want)
    assert np.array_equal(host(q), q8_1_of(want))


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_post_norm_add_norm(rows, cols):
    a, res, w_post, w_ffn = inputs(rows, cols, 300 + cols)
    x_out, out, q = ops.post_norm_add_norm_q8_1(dev(a), dev(w_post), dev(res), dev(w_ffn), 1e-5, 1e-6)
    want_x, want = oracle.norm_rows(2, a, w_ffn, w_first=w_post, residual=res, eps=1e-6, eps_first=1e-5)
    assert np.array_equal(host(x_out), want_x) and np.array_equal(host(out), want)
    assert np.array_equal(host(q), q8_1_of(want))


def test_a_zero_row_and_a_row_with_one_value():
    cols = 1024
    x = np.zeros((2, cols), np.float32)
    x[1, 700] = -3.0
    w = np.ones(cols, np.float32)
    out, q = ops.rmsnorm_q8_1(dev(x), dev(w), 1e-6)
    assert np.array_equal(host(out), oracle.norm_rows(0, x, w, eps=1e-6))
    assert np.array_equal(host(q), q8_1_of(host(out)))
    assert not host(q)[0].any()                       # zero blocks: d = 0, s = 0, codes 0
    assert host(q)[1, 700 // 32, 4 + 700 % 32] == 0x81  # the extreme maps to -127


@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("rows,n", [(1, 32), (1, 6144), (5, 14336), (2, 96)])
def test_split_activation_and_its_q8_1(act, rows, n):
    gu = (synth.normal(400 + n, act, rows * 2 * n) * 3.0).reshape(rows, 2 * n)
    out, q = ops.split_act_mul_q8_1(dev(gu), act)
    want = oracle.split_act_mul(gu, act)
    got = host(out)
    # 1 + tanh(.) cancels for a negative gate: the two math libraries' last-place differences in
    # tanh (and exp) then show at the scale of g * u, not of the result
    scale = np.abs(gu[:, :n] * gu[:, n:])
    assert (np.abs(got - want) <= 1e-6 * np.abs(want) + 2.5e-7 * scale + 1e-30).all()
    assert np.array_equal(host(q), q8_1_of(got))


def test_the_quantized_row_feeds_the_matvec_as_the_two_launch_path_does():
    n, k = 256, 2048
    w = dev(synth.weight(lib.TYPE_Q4_K, n, k, seed=7, stream=1))
    x, _, nw, _ = inputs(1, k, 500)
    out, q = ops.rmsnorm_q8_1(dev(x), dev(nw), 1e-5)
    assert torch.equal(ops.mmvq(lib.TYPE_Q4_K, w, q, k, n), ops.mmvq(lib.TYPE_Q4_K, w, ops.quantize_q8_1_rows(out), k, n))


def test_sizes_the_kernels_do_not_take_are_refused():
    l = lib.load()
    x = torch.zeros((1, 1000), device="cuda")
    q = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    assert l.lk_rmsnorm_q8_1(x.data_ptr(), x.data_ptr(), x.data_ptr(), q.data_ptr(), 1e-6, 1000, 1, 0) == lib.LK_ERR_ARG
    assert l.lk_rmsnorm_q8_1(x.data_ptr(), x.data_ptr(), x.data_ptr(), q.data_ptr(), 1e-6, 512 * 200, 1, 0) == lib.LK_ERR_ARG
    assert l.lk_rmsnorm_q8_1(None, x.data_ptr(), x.data_ptr(), q.data_ptr(), 1e-6, 512, 1, 0) == lib.LK_ERR_ARG
    assert l.lk_rmsnorm_q8_1(x.data_ptr(), x.data_ptr(), x.data_ptr(), q.data_ptr(), 1e-6, 512, 0, 0) == lib.LK_OK
    assert l.lk_split_act_mul_q8_1(x.data_ptr(), x.data_ptr(), q.data_ptr(), 40, 1, 0, 0) == lib.LK_ERR_ARG
    assert l.lk_split_act_mul_q8_1(x.data_ptr(), x.data_ptr(), q.data_ptr(), 64, 1, 2, 0) == lib.LK_ERR_TYPE

"""The benchmark configurations at their full shapes, against the same-codes oracle.

  config 0  Q4_K 4096 x 4096, one row, seed 0: every integer sub-block dot of every weight row, and
            the f32 output
  config 1  Llama-3-8B linears at 4 and 8 rows: gate/up 14336 x 4096 (Q4_K), down 4096 x 14336
            (Q6_K), lm_head 128256 x 4096 (Q8_0); the batch-1 forms live in test_gpu_mmvq.py
  config 3  the Qwen3-30B-A3B-shaped expert block at 16 tokens (1 and 256 live in test_gpu_moe.py)
  config 4  every Qwen3-1.7B linear shape at 1, 16 and 64 rows through the host mirror of
            QKernelMatMul::forward (whatever path it picks for the row count)

Large outputs are checked on a seeded sample of weight rows (every activation row): the oracle
runs on the sampled rows' blocks, the GPU on the whole matrix.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from moe_block_check import check_block
from loken_amd import lib, moe, ops, synth

pytestmark = pytest.mark.gpu

Q4K, Q6K, Q80 = lib.TYPE_Q4_K, lib.TYPE_Q6_K, lib.TYPE_Q8_0
X_TYPES = {torch.float32: lib.TYPE_F32}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(got, want, rtol=1e-3, atol=1e-4):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bad = np.abs(got - want) > rtol * np.abs(want) + atol
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; worst {np.abs(got - want).max()}"


_WEIGHTS = {}


def weight(wtype, n, k, stream):
    key = (wtype, n, k, stream)
    if key not in _WEIGHTS:
        if len(_WEIGHTS) > 3:
            _WEIGHTS.clear()
        w = synth.weight(wtype, n, k, seed=0, stream=stream)
        _WEIGHTS[key] = (w, dev(w))
    return _WEIGHTS[key]


def sample_rows(n, count, seed):
    if n <= count:
        return np.arange(n)
    rng = np.random.default_rng(seed)
    return np.sort(np.concatenate([[0, 1, n - 2, n - 1], rng.choice(np.arange(2, n - 2), count - 4, replace=False)]))


# ---------------------------------------------------------------- config 0
def test_config0_every_integer_subblock_dot_and_the_output():
    n = k = 4096
    w, wd = weight(Q4K, n, k, 0)
    x = synth.activation(1, k, seed=0)
    q = ops.quantize_q8_1_rows(dev(x))
    act = oracle.quantize_q8_1(x[0])
    assert np.array_equal(q.cpu().numpy().reshape(-1), act.reshape(-1))
    for r0 in range(0, n, 1024):   # the probe's grid takes up to 65535 rows; slices keep the host buffers small
        dots, sums = ops.mmvq_subdots(Q4K, wd[r0:r0 + 1024], q[0], k, 1024)
        want_dots, want_sums = oracle.ob_subdots(Q4K, k, 1024, w[r0:r0 + 1024], act)
        assert np.array_equal(dots.cpu().numpy(), want_dots)
        assert np.array_equal(sums.cpu().numpy(), want_sums)
    assert_close(ops.mmvq(Q4K, wd, q, k, n).cpu().numpy(), oracle.ob_matmul(Q4K, x, w, n))


# ---------------------------------------------------------------- config 1 at 4 and 8 rows
@pytest.mark.parametrize("wtype,n,k,stream", [(Q4K, 14336, 4096, 10), (Q6K, 4096, 14336, 10), (Q80, 128256, 4096, 10)])
@pytest.mark.parametrize("batch", [4, 8])
def test_config1_large_linears_at_4_and_8_rows(wtype, n, k, stream, batch):
    w, wd = weight(wtype, n, k, stream)
    x = synth.activation(batch, k, seed=batch)
    got = ops.mmvq(wtype, wd, ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
    rows = sample_rows(n, 1500, seed=n + batch)
    assert_close(got[:, rows], oracle.ob_matmul(wtype, x, w[rows], len(rows)))
    # and the fused-activation launch carries the same bits
    fused = ops.mmvq_fused(wtype, [wd], dev(x), [n])[0] if k <= 8192 else None
    if fused is not None:
        assert np.array_equal(fused.cpu().numpy(), got)


# ---------------------------------------------------------------- config 3 at 16 tokens
def test_config3_expert_block_at_16_tokens_full_shape():
    tokens, hidden, ffn, n_experts, topk = 16, 2048, 768, 128, 8
    gate = synth.weight(Q4K, n_experts * ffn, hidden, seed=0, stream=1)
    up = synth.weight(Q4K, n_experts * ffn, hidden, seed=0, stream=2)
    down = synth.weight(Q4K, n_experts * hidden, ffn, seed=0, stream=3)
    x = synth.activation(tokens, hidden, seed=0) * np.float32(30.0)
    ids, w = oracle.topk_softmax(synth.activation(tokens, n_experts, seed=0, stream=7), topk)
    want, want_h = oracle.moe_forward(1, Q4K, Q4K, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    slots = oracle.group_by_expert(ids)[0]
    want_slot = np.empty_like(want_h)
    want_slot[slots] = want_h   # the oracle's gated rows are in sorted order; the checks read slot order
    gd, ud, dd, xd, wd = dev(gate), dev(up), dev(down), dev(x), dev(w.reshape(-1))
    # per routed pair (what the layer code picks at this load: one row per expert on average)
    routing = moe.ExpertRouting(dev(ids))
    h = moe.moe_gemm_gguf_gate_up_silu_mul(Q4K, xd, gd, ud, routing, n_experts, ffn)
    assert (np.abs(h.cpu().numpy() - want_slot) <= 1e-3 * np.abs(want_slot) + 1e-4 * np.abs(want_slot).max()).all()
    out = moe.moe_gemm_gguf_down_reduce(Q4K, h, dd, routing, wd, n_experts, hidden).cpu().numpy()
    # 1e-3 / 1e-4 with the oracle's second stage fed the card's own gated rows; end to end, anything
    # outside that bound is attributed to a flipped Q8_1 code of those rows (tests/moe_block_check.py)
    check_block(out, h.cpu().numpy(), want, want_slot, Q4K, down, ids, w, n_experts, hidden)
    # and the expert-batched tiles over the same routing
    plan = moe.MmqRouting.from_choices(dev(ids), n_experts)
    h2 = plan.gate_up_silu(Q4K, xd, gd, ud, ffn)
    out2 = plan.down_fold(Q4K, h2, dd, hidden, wd).cpu().numpy()
    h2_slot = np.empty_like(want_h)
    h2_slot[plan.slots.cpu().numpy()] = h2.cpu().numpy()
    assert (np.abs(h2_slot - want_slot) <= 1e-3 * np.abs(want_slot) + 1e-4 * np.abs(want_slot).max()).all()
    check_block(out2, h2_slot, want, want_slot, Q4K, down, ids, w, n_experts, hidden)


# ---------------------------------------------------------------- config 4
class Linear:
    def __init__(self, wtype, w, n, k):
        self.l, self.w, self.n, self.k = lib.load(), w, n, k
        self.h = self.l.lkh_qkernel_matmul_new(wtype, n, k, w.data_ptr(), torch.cuda.current_device())

    def __call__(self, x):
        out = torch.empty((x.shape[0], self.n), dtype=x.dtype, device=x.device)
        lib.check("lkh_qkernel_matmul_forward",
                  self.l.lkh_qkernel_matmul_forward(self.h, x.data_ptr(), lib.TYPE_F32, x.shape[0], out.data_ptr(),
                                                    torch.cuda.current_stream().cuda_stream, 0))
        return out

    def close(self):
        self.l.lkh_qkernel_matmul_free(self.h)


QWEN3_1P7B = [("q_o", Q4K, 2048, 2048), ("k_v", Q4K, 1024, 2048), ("gate_up", Q4K, 6144, 2048),
              ("down", Q6K, 2048, 6144), ("lm_head", Q6K, 151936, 2048)]


@pytest.mark.parametrize("name,wtype,n,k", QWEN3_1P7B)
def test_config4_qwen3_1p7b_linears_at_1_16_64_rows(name, wtype, n, k):
    w, wd = weight(wtype, n, k, 40)
    lin = Linear(wtype, wd, n, k)
    rows = sample_rows(n, 1200, seed=n)
    try:
        for b in (1, 16, 64):
            x = synth.activation(b, k, seed=40 + b)
            got = lin(dev(x)).cpu().numpy()
            assert_close(got[:, rows], oracle.ob_matmul(wtype, x, w[rows], len(rows)))
    finally:
        lin.close()

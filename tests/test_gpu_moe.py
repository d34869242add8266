"""GPU parity of the MoE expert block against the CPU oracle.

The oracle (lko_moe_forward) follows loken's host path: gate/up per routed pair, SiLU, down,
fold in expert-run order (src/inference/moe_cuda_cpu/mod.rs:459-605, 1478-1660). The GPU fold
runs in slot order (cuda/moe/moe_mmq.cu:155-176), so only the final [tokens, hidden] is
comparable and only to float summation order; the intermediate GLU rows are compared in sorted
order, which both sides share.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, synth
from loken_amd.moe import MmqRouting

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-3, 1e-4


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(got, want, rtol=RTOL, atol=ATOL):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bad = np.abs(got - want) > rtol * np.abs(want) + atol
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; worst {np.abs(got - want).max()}"


def make_layer(tokens, hidden, ffn, n_experts, topk, seed, dt_down=lib.TYPE_Q4_K, x_scale=30.0):
    dt = lib.TYPE_Q4_K
    gate = synth.weight(dt, n_experts * ffn, hidden, seed=seed, stream=1)
    up = synth.weight(dt, n_experts * ffn, hidden, seed=seed, stream=2)
    down = synth.weight(dt_down, n_experts * hidden, ffn, seed=seed, stream=3)
    x = synth.activation(tokens, hidden, seed=seed) * np.float32(x_scale)
    logits = synth.activation(tokens, n_experts, seed=seed, stream=7)
    ids, w = oracle.topk_softmax(logits, topk)
    return gate, up, down, x, ids, w


def test_route_groups_pairs_stably_by_expert():
    rng = np.random.default_rng(50)
    tokens, topk, n_experts = 37, 4, 11
    choices = np.stack([rng.choice(n_experts, topk, replace=False) for _ in range(tokens)]).astype(np.int32)
    plan = MmqRouting.from_choices(dev(choices), n_experts)
    slots, experts = oracle.group_by_expert(choices)
    assert plan.slots.cpu().tolist() == slots.tolist()
    assert plan.src_rows.cpu().tolist() == (slots // topk).tolist()
    want_bounds = np.searchsorted(experts, np.arange(n_experts + 1))
    assert plan.bounds.cpu().tolist() == want_bounds.tolist()
    # the sorted-routing entry point builds the same plan
    plan2 = MmqRouting.new(dev(slots), dev(experts), topk, n_experts)
    assert torch.equal(plan2.bounds, plan.bounds) and torch.equal(plan2.slots, plan.slots)
    assert torch.equal(plan2.src_rows, plan.src_rows)


def test_route_with_experts_nobody_chose_and_one_token():
    choices = np.array([[5, 2]], np.int32)
    plan = MmqRouting.from_choices(dev(choices), 8)
    assert plan.bounds.cpu().tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2]
    assert plan.slots.cpu().tolist() == [1, 0]


@pytest.mark.parametrize("tokens,hidden,ffn,n_experts,topk", [(5, 512, 256, 6, 2), (40, 1024, 512, 8, 3),
                                                             (1, 256, 256, 4, 2), (70, 512, 768, 16, 4)])
@pytest.mark.parametrize("dt_down", [lib.TYPE_Q4_K, lib.TYPE_Q6_K])
def test_expert_batched_block_matches_oracle(tokens, hidden, ffn, n_experts, topk, dt_down):
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=51, dt_down=dt_down)
    want, want_h = oracle.moe_forward(1, lib.TYPE_Q4_K, dt_down, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    plan = MmqRouting.from_choices(dev(ids), n_experts)
    h = plan.gate_up_silu(lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), ffn)
    # GLU rows in sorted order; expf differs from libm's in the last place, and silu(g)*u inherits
    # the relative error of g and u where they nearly cancel: compare against the scale of a row
    got_h = h.cpu().numpy()
    assert (np.abs(got_h - want_h) <= 1e-3 * np.abs(want_h) + 1e-4 * np.abs(want_h).max()).all()
    out = plan.down_fold(dt_down, h, dev(down), hidden, dev(w.reshape(-1)))
    got = out.cpu().numpy()
    # the down projection re-quantizes h: a one-ulp difference in h can flip a Q8_1 code, so the
    # final bound is the quantization envelope of the reference's own tests, not 1e-3 relative
    scale = np.abs(want).max()
    assert (np.abs(got - want) <= 2e-3 * np.abs(want) + 2e-4 * scale).all()


def test_down_fold_alone_is_tight_when_fed_the_oracle_rows():
    # feeding the oracle's own GLU rows removes the re-quantization ambiguity: 1e-3 rel + 1e-4 abs
    tokens, hidden, ffn, n_experts, topk = 24, 512, 512, 8, 2
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=52)
    want, want_h = oracle.moe_forward(1, lib.TYPE_Q4_K, lib.TYPE_Q4_K, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    plan = MmqRouting.from_choices(dev(ids), n_experts)
    out = plan.down_fold(lib.TYPE_Q4_K, dev(want_h), dev(down), hidden, dev(w.reshape(-1)))
    assert_close(out.cpu().numpy(), want, atol=1e-4 * max(1.0, np.abs(want).max()))


def test_residual_is_the_starting_value_of_the_fold():
    tokens, hidden, ffn, n_experts, topk = 6, 256, 256, 4, 2
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=53)
    plan = MmqRouting.from_choices(dev(ids), n_experts)
    h = plan.gate_up_silu(lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), ffn)
    base = plan.down_fold(lib.TYPE_Q4_K, h, dev(down), hidden, dev(w.reshape(-1)))
    res = torch.randn((tokens, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))
    with_res = plan.down_fold(lib.TYPE_Q4_K, h, dev(down), hidden, dev(w.reshape(-1)), residual=res)
    # (res + a) + b against (0 + a + b) + res: float summation order only
    scale = base.abs().max().item() + res.abs().max().item()
    assert (with_res - (base + res)).abs().max().item() <= 1e-6 * scale


def test_result_does_not_depend_on_tile_width():
    tokens, hidden, ffn, n_experts, topk = 90, 512, 256, 4, 2
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=54)
    outs = []
    for width in (0, 32, 64, 128):
        plan = MmqRouting.from_choices(dev(ids), n_experts).with_tile_width(width)
        h = plan.gate_up_silu(lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), ffn)
        outs.append(plan.down_fold(lib.TYPE_Q4_K, h, dev(down), hidden, dev(w.reshape(-1))))
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


def test_glu_kernels():
    rng = np.random.default_rng(55)
    rows, width, n_experts = 13, 40, 3
    gu = rng.standard_normal((rows, 2 * width)).astype(np.float32) * 3
    l = lib.load()
    s = torch.cuda.current_stream().cuda_stream
    gud = dev(gu)
    out = torch.empty((rows, width), device="cuda")
    l.loken_moe_mmq_silu_mul(gud.data_ptr(), out.data_ptr(), rows, width, s)
    g, u = gu[:, :width].astype(np.float64), gu[:, width:].astype(np.float64)
    np.testing.assert_allclose(out.cpu().numpy(), g / (1 + np.exp(-g)) * u, rtol=2e-6, atol=1e-7)
    bounds = np.array([0, 4, 4, 13], np.int32)
    gb = rng.standard_normal((n_experts, width)).astype(np.float32)
    ub = rng.standard_normal((n_experts, width)).astype(np.float32)
    alpha, limit = 1.702, 7.0
    bd, gbd, ubd = dev(bounds), dev(gb), dev(ub)   # named: a temporary would be freed before the launch
    l.loken_moe_mmq_swiglu_oai(gud.data_ptr(), out.data_ptr(), rows, width, bd.data_ptr(), n_experts,
                               gbd.data_ptr(), ubd.data_ptr(), alpha, limit, s)
    e_of = np.array([0] * 4 + [2] * 9)
    xx = np.minimum(g + gb[e_of], limit)
    uc = np.clip(u + ub[e_of], -limit, limit)
    np.testing.assert_allclose(out.cpu().numpy(), xx / (1 + np.exp(-alpha * xx)) * (1 + uc), rtol=3e-6, atol=1e-6)


def test_fold_is_in_slot_order_with_bias():
    rng = np.random.default_rng(56)
    tokens, topk, cols, n_experts = 5, 3, 33, 4
    pairs = rng.standard_normal((tokens * topk, cols)).astype(np.float32)
    wts = rng.random(tokens * topk).astype(np.float32)
    choices = rng.integers(0, n_experts, tokens * topk).astype(np.int32)
    bias = rng.standard_normal((n_experts, cols)).astype(np.float32)
    start = rng.standard_normal((tokens, cols)).astype(np.float32)
    out = dev(start.copy())
    pd, wd, cd, bd = dev(pairs), dev(wts), dev(choices), dev(bias)
    lib.load().loken_moe_mmq_fold(pd.data_ptr(), wd.data_ptr(), cd.data_ptr(), bd.data_ptr(), out.data_ptr(),
                                  tokens, topk, cols, torch.cuda.current_stream().cuda_stream)
    want = start.copy()
    for t in range(tokens):
        for k in range(topk):
            p = t * topk + k
            want[t] = want[t] + wts[p] * (pairs[p] + bias[choices[p]])   # same f32 steps, same order
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=1e-6, atol=1e-6)


def test_benchmark_shape_256_tokens_against_sampled_oracle():
    # Qwen3-30B-A3B-shaped layer: 128 experts, hidden 2048, ffn 768, top-8
    tokens, hidden, ffn, n_experts, topk = 256, 2048, 768, 128, 8
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=0)
    plan = MmqRouting.from_choices(dev(ids), n_experts)
    h = plan.gate_up_silu(lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), ffn)
    out = plan.down_fold(lib.TYPE_Q4_K, h, dev(down), hidden, dev(w.reshape(-1))).cpu().numpy()
    # oracle on a sample of tokens (a token's output depends only on its own routed pairs)
    sample = [0, 17, 100, 255]
    want = oracle.moe_forward(1, lib.TYPE_Q4_K, lib.TYPE_Q4_K, x[sample], gate, up, down, ids[sample], w[sample],
                              n_experts, ffn)
    scale = np.abs(want).max()
    assert (np.abs(out[sample] - want) <= 2e-3 * np.abs(want) + 2e-4 * scale).all()
    # every routed pair landed somewhere: the per-expert load adds up
    bounds = plan.bounds.cpu().numpy()
    assert bounds[-1] == tokens * topk and (np.diff(bounds) >= 0).all()

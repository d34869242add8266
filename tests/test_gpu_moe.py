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
from loken_amd import lib, moe, ops, synth
from loken_amd.moe import MmqRouting
from moe_block_check import check_block

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-3, 1e-4


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(got, want, rtol=RTOL, atol=ATOL):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bad = np.abs(got - want) > rtol * np.abs(want) + atol
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; worst {np.abs(got - want).max()}"


def make_layer(tokens, hidden, ffn, n_experts, topk, seed, dt_down=lib.TYPE_Q4_K, x_scale=30.0, dt_gu=lib.TYPE_Q4_K):
    dt = dt_gu
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
@pytest.mark.parametrize("dt_down", [lib.TYPE_Q4_K, lib.TYPE_Q5_K, lib.TYPE_Q6_K])
@pytest.mark.parametrize("path", ["tiled", "rows"])
def test_expert_batched_block_matches_oracle(tokens, hidden, ffn, n_experts, topk, dt_down, path):
    """Both launch families of the expert-batched block: the tiled matmul, and (Q4_K stacks) the
    matrix-unit rows launch that serves short runs per expert."""
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=51, dt_down=dt_down)
    want, want_h = oracle.moe_forward(1, lib.TYPE_Q4_K, dt_down, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    plan = MmqRouting.from_choices(dev(ids), n_experts).with_path(path)
    assert plan.takes_rows_launch(lib.TYPE_Q4_K, hidden) == (path == "rows")
    h = plan.gate_up_silu(lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), ffn)
    # GLU rows in sorted order; expf differs from libm's in the last place, and silu(g)*u inherits
    # the relative error of g and u where they nearly cancel: compare against the scale of a row
    got_h = h.cpu().numpy()
    assert (np.abs(got_h - want_h) <= 1e-3 * np.abs(want_h) + 1e-4 * np.abs(want_h).max()).all()
    out = plan.down_fold(dt_down, h, dev(down), hidden, dev(w.reshape(-1)))
    # the strict bound with the oracle's second stage fed the card's own rows; end to end, whatever is
    # outside it belongs to a token with a flipped Q8_1 code of h (moe_block_check.py)
    slots = plan.slots.cpu().numpy()
    h_slot, want_h_slot = np.empty_like(got_h), np.empty_like(want_h)
    h_slot[slots], want_h_slot[slots] = got_h, want_h
    check_block(out.cpu().numpy(), h_slot, want, want_h_slot, dt_down, down, ids, w, n_experts, hidden)


NIBBLE_TILES = {"q4_0": lib.TYPE_Q4_0, "q4_1": lib.TYPE_Q4_1, "q5_0": lib.TYPE_Q5_0, "q5_1": lib.TYPE_Q5_1,
                "iq4_nl": lib.TYPE_IQ4_NL, "mxfp4": lib.TYPE_MXFP4, "iq4_xs": lib.TYPE_IQ4_XS, "q3_k": lib.TYPE_Q3_K,
                "q2_k": lib.TYPE_Q2_K,
                # the codebook formats only mixtures store (src/tensor/quantized/mmq.rs:335-343)
                "iq3_xxs": lib.TYPE_IQ3_XXS, "iq3_s": lib.TYPE_IQ3_S, "iq2_s": lib.TYPE_IQ2_S, "q2_0": lib.TYPE_Q2_0}


@pytest.mark.parametrize("tokens,hidden,ffn,n_experts,topk", [(40, 1024, 512, 8, 3), (70, 512, 768, 16, 4),
                                                             (1, 256, 256, 4, 2), (300, 512, 256, 3, 2)])
@pytest.mark.parametrize("name", sorted(NIBBLE_TILES))
def test_expert_batched_block_in_the_nibble_formats_matches_oracle(name, tokens, hidden, ffn, n_experts, topk):
    """The tiled launch for the 32-value formats, IQ4_XS and Q3_K; IQ4_NL, MXFP4 and IQ4_XS have no dense
    entry point. The last shape runs the 128-token tiles."""
    dt = NIBBLE_TILES[name]
    assert moe.moe_mmq_serves(dt, hidden)
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=53, dt_down=dt, dt_gu=dt, x_scale=4.0)
    want, want_h = oracle.moe_forward(1, dt, dt, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    plan = MmqRouting.from_choices(dev(ids), n_experts).with_path("tiled")
    h = plan.gate_up_silu(dt, dev(x), dev(gate), dev(up), ffn)
    got_h = h.cpu().numpy()
    assert (np.abs(got_h - want_h) <= 1e-3 * np.abs(want_h) + 1e-4 * np.abs(want_h).max()).all()
    # down from the oracle's own rows, so that a code flipped by the last place of h does not enter
    out = plan.down_fold(dt, dev(want_h), dev(down), hidden, dev(w.reshape(-1)))
    scale = np.abs(want).max()
    assert (np.abs(out.cpu().numpy() - want) <= 1e-3 * np.abs(want) + 1e-4 * scale).all()


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
    # The narrow tiles run the same int8 kernel, to the bit. The 128-token tile of Q4_K forms the
    # same integer dots on the f16 matrix unit and adds them up in another f32 order; the hidden
    # state is re-quantized between the two products, so a last-bit difference there can move a
    # code by one: a float tolerance, not equality.
    for o in outs[1:3]:
        assert torch.equal(o, outs[0])
    scale = outs[0].abs().max().item()
    assert (outs[3] - outs[0]).abs().max().item() <= 1e-4 * scale


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
    want, want_h = oracle.moe_forward(1, lib.TYPE_Q4_K, lib.TYPE_Q4_K, x[sample], gate, up, down, ids[sample], w[sample],
                                      n_experts, ffn, want_h=True)
    slots = plan.slots.cpu().numpy()
    h_slot = np.empty((tokens * topk, ffn), np.float32)
    h_slot[slots] = h.cpu().numpy()
    rows = (np.array(sample)[:, None] * topk + np.arange(topk)[None, :]).reshape(-1)
    want_h_slot = np.empty_like(want_h)
    want_h_slot[oracle.group_by_expert(ids[sample])[0]] = want_h
    check_block(out[sample], h_slot[rows], want, want_h_slot, lib.TYPE_Q4_K, down, ids[sample], w[sample], n_experts, hidden)
    # every routed pair landed somewhere: the per-expert load adds up
    bounds = plan.bounds.cpu().numpy()
    assert bounds[-1] == tokens * topk and (np.diff(bounds) >= 0).all()


# ---------------------------------------------------------------- decode (per routed pair)
from loken_amd.moe import (ExpertRouting, moe_forward, moe_gemm_gguf, moe_gemm_gguf_down_reduce,
                           moe_gemm_gguf_gate_up_silu_mul)


def slot_order(h_sorted, ids):
    """oracle rows are in sorted order; the decode kernels write slot order"""
    slots, _ = oracle.group_by_expert(ids)
    out = np.empty_like(h_sorted)
    out[slots] = h_sorted
    return out


@pytest.mark.parametrize("tokens,hidden,ffn,n_experts,topk", [(1, 2048, 768, 128, 8), (3, 512, 256, 6, 2),
                                                             (16, 1024, 768, 32, 4)])
@pytest.mark.parametrize("dt_down", [lib.TYPE_Q4_K, lib.TYPE_Q5_K, lib.TYPE_Q6_K])
def test_per_pair_decode_block_matches_oracle(tokens, hidden, ffn, n_experts, topk, dt_down):
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=57, dt_down=dt_down)
    want, want_h = oracle.moe_forward(1, lib.TYPE_Q4_K, dt_down, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    routing = ExpertRouting(dev(ids))
    slots, experts = oracle.group_by_expert(ids)
    assert routing.sorted_token_ids.cpu().tolist() == slots.tolist()
    assert routing.expert_ids.cpu().tolist() == experts.tolist()
    h = moe_gemm_gguf_gate_up_silu_mul(lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), routing, n_experts, ffn)
    want_slot = slot_order(want_h, ids)
    assert (np.abs(h.cpu().numpy() - want_slot) <= 1e-3 * np.abs(want_slot) + 1e-4 * np.abs(want_slot).max()).all()
    out = moe_gemm_gguf_down_reduce(dt_down, h, dev(down), routing, dev(w.reshape(-1)), n_experts, hidden)
    check_block(out.cpu().numpy(), h.cpu().numpy(), want, want_slot, dt_down, down, ids, w, n_experts, hidden)


# the rows of the reference's expert table (src/inference/moe_cuda/gemm.rs:23-39) beyond the K-quant engines
TABLE_TAIL = {"q2_k": lib.TYPE_Q2_K, "q3_k": lib.TYPE_Q3_K, "q5_0": lib.TYPE_Q5_0, "mxfp4": lib.TYPE_MXFP4,
              "q5_1": lib.TYPE_Q5_1, "iq4_nl": lib.TYPE_IQ4_NL, "iq4_xs": lib.TYPE_IQ4_XS,
              "iq3_xxs": lib.TYPE_IQ3_XXS, "iq3_s": lib.TYPE_IQ3_S, "iq2_s": lib.TYPE_IQ2_S, "q2_0": lib.TYPE_Q2_0,
              "iq2_xxs": lib.TYPE_IQ2_XXS,   # wire ids 11..15
              "q5_k": lib.TYPE_Q5_K}   # and Q5_K on the K-quant engine, short rows and long


@pytest.mark.parametrize("tokens,hidden,ffn,n_experts,topk", [(1, 1024, 768, 16, 4), (3, 512, 256, 6, 2), (2, 2560, 512, 4, 2)])
@pytest.mark.parametrize("name", sorted(TABLE_TAIL))
def test_per_pair_decode_block_in_the_tail_formats_matches_oracle(name, tokens, hidden, ffn, n_experts, topk):
    dt = TABLE_TAIL[name]
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=61, dt_down=dt, dt_gu=dt, x_scale=4.0)
    want, want_h = oracle.moe_forward(1, dt, dt, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    routing = ExpertRouting(dev(ids))
    h = moe_gemm_gguf_gate_up_silu_mul(dt, dev(x), dev(gate), dev(up), routing, n_experts, ffn)
    want_slot = slot_order(want_h, ids)
    assert (np.abs(h.cpu().numpy() - want_slot) <= 1e-3 * np.abs(want_slot) + 1e-4 * np.abs(want_slot).max()).all()
    # down from the oracle's own intermediate rows, so the two stages are checked apart
    bias = torch.randn((n_experts, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(7))
    out = moe_gemm_gguf_down_reduce(dt, dev(want_slot), dev(down), routing, dev(w.reshape(-1)), n_experts, hidden)
    scale = np.abs(want).max()
    assert (np.abs(out.cpu().numpy() - want) <= 1e-3 * np.abs(want) + 1e-4 * scale).all()
    with_bias = moe_gemm_gguf_down_reduce(dt, dev(want_slot), dev(down), routing, dev(w.reshape(-1)), n_experts, hidden,
                                          down_bias=bias)
    add = (dev(w).unsqueeze(-1) * bias[dev(ids).long()]).sum(1)
    assert (with_bias - (out + add)).abs().max().item() <= 1e-5 * (scale + add.abs().max().item())
    # the plain launcher over the same pairs: the gate product alone
    plain = moe_gemm_gguf(dt, dev(x), dev(gate), routing, n_experts, ffn)
    slots, experts = oracle.group_by_expert(ids)
    gate_rows = gate.reshape(n_experts, ffn, -1)
    for j in range(len(slots)):
        want_row = oracle.ob_matmul(dt, x[slots[j] // topk][None, :], gate_rows[experts[j]].reshape(-1), ffn)[0]
        got_row = plain[slots[j]].cpu().numpy()
        assert (np.abs(got_row - want_row) <= 1e-3 * np.abs(want_row) + 1e-4 * np.abs(want_row).max()).all()


@pytest.mark.parametrize("name", ["q4_k", "q6_k", "q8_0", "mxfp4", "q5_0", "q3_k"])
def test_gated_decode_launch_with_the_other_activations(name):
    """The gate and up products are the same-codes oracle's; the activation on top of them is the
    closed form the reference's kernels state (cuda/moe/moe_gguf.cu:994-1003, 1178-1184, 1280-1289)."""
    from loken_amd.moe import (moe_gemm_gguf_gate_up_gelu_mul_concat, moe_gemm_gguf_gate_up_swiglu_limited,
                               moe_gemm_gguf_gate_up_swiglu_oai)
    dt = {"q4_k": lib.TYPE_Q4_K, "q6_k": lib.TYPE_Q6_K, "q8_0": lib.TYPE_Q8_0, **TABLE_TAIL}[name]
    tokens, hidden, ffn, n_experts, topk = 3, 512, 256, 5, 2
    gate, up, _, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=63, dt_gu=dt, x_scale=4.0)
    routing = ExpertRouting(dev(ids))
    slots, experts = oracle.group_by_expert(ids)
    gate_rows, up_rows = gate.reshape(n_experts, ffn, -1), up.reshape(n_experts, ffn, -1)
    g = np.empty((tokens * topk, ffn), np.float64)
    u = np.empty((tokens * topk, ffn), np.float64)
    for j in range(len(slots)):
        row = x[slots[j] // topk][None, :]
        g[slots[j]] = oracle.ob_matmul(dt, row, gate_rows[experts[j]].reshape(-1), ffn)[0]
        u[slots[j]] = oracle.ob_matmul(dt, row, up_rows[experts[j]].reshape(-1), ffn)[0]
    e_of_slot = ids.reshape(-1)

    def close(got, want):
        got = got.cpu().numpy()
        assert (np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-4 * np.abs(want).max()).all()

    limit = float(np.quantile(np.abs(g), 0.7))   # so that both sides of every clamp occur
    alpha = 1.702
    gb = synth.normal(63, 11, n_experts * ffn).reshape(n_experts, ffn) * np.float32(0.1 * limit)
    ub = synth.normal(63, 12, n_experts * ffn).reshape(n_experts, ffn) * np.float32(0.1 * limit)
    for biased in (False, True):
        gg = g + (gb[e_of_slot] if biased else 0.0)
        uu = u + (ub[e_of_slot] if biased else 0.0)
        xx = np.minimum(gg, limit)
        want = xx / (1.0 + np.exp(-alpha * xx)) * (1.0 + np.clip(uu, -limit, limit))
        got = moe_gemm_gguf_gate_up_swiglu_oai(dt, dev(x), dev(gate), dev(up), routing, n_experts, ffn, alpha, limit,
                                               dev(gb) if biased else None, dev(ub) if biased else None)
        close(got, want)
    gl = np.minimum(g, limit)
    close(moe_gemm_gguf_gate_up_swiglu_limited(dt, dev(x), dev(gate), dev(up), routing, n_experts, ffn, limit),
          gl / (1.0 + np.exp(-gl)) * np.clip(u, -limit, limit))
    # one tensor per layer: every expert's gate rows, then its up rows
    both = np.concatenate([gate_rows, up_rows], axis=1)
    want = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3))) * u
    close(moe_gemm_gguf_gate_up_gelu_mul_concat(dt, dev(x), dev(np.ascontiguousarray(both)), routing, n_experts, ffn), want)


@pytest.mark.parametrize("name", ["q4_k", "mxfp4"])
def test_live_count_variants_run_the_first_pairs_only(name):
    from loken_amd.moe import moe_gemm_gguf_down_pairs_live, moe_gemm_gguf_gate_up_silu_mul_live
    dt = {"q4_k": lib.TYPE_Q4_K, **TABLE_TAIL}[name]
    tokens, hidden, ffn, n_experts, topk = 4, 512, 256, 5, 2
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=64, dt_down=dt, dt_gu=dt, x_scale=4.0)
    routing = ExpertRouting(dev(ids))
    slots = routing.sorted_token_ids.cpu().numpy()
    pairs = tokens * topk
    full_h = moe_gemm_gguf_gate_up_silu_mul(dt, dev(x), dev(gate), dev(up), routing, n_experts, ffn)
    flat_w = dev(w.reshape(-1))
    for count in (5, pairs, 0):
        live = torch.tensor([count], dtype=torch.int32, device="cuda")   # the card reads it as a uint32
        marker = torch.full((pairs, ffn), -7.0, device="cuda")
        h = moe_gemm_gguf_gate_up_silu_mul_live(dt, dev(x), dev(gate), dev(up), routing, n_experts, ffn, live, out=marker)
        ran, idle = slots[:count], slots[count:]
        assert torch.equal(h[ran], full_h[ran])
        assert (h[idle] == -7.0).all()
        rows = moe_gemm_gguf_down_pairs_live(dt, full_h, dev(down), routing, flat_w, n_experts, hidden, live)
        assert (rows[idle] == 0).all()
        if count == pairs:
            want = moe_gemm_gguf_down_reduce(dt, full_h, dev(down), routing, flat_w, n_experts, hidden)
            got = rows.reshape(tokens, topk, hidden).sum(1)
            assert (got - want).abs().max().item() <= 1e-6 * want.abs().max().item()
            all_rows = rows
    live = torch.tensor([5], dtype=torch.int32, device="cuda")
    rows5 = moe_gemm_gguf_down_pairs_live(dt, full_h, dev(down), routing, flat_w, n_experts, hidden, live)
    assert torch.equal(rows5[slots[:5]], all_rows[slots[:5]])


@pytest.mark.parametrize("name", ["q4_k", "q6_k", "mxfp4"])
def test_experts_over_two_tensors_match_the_one_tensor_launch(name):
    from loken_amd.moe import (moe_gemm_gguf_down_pairs_over, moe_gemm_gguf_down_reduce_over,
                               moe_gemm_gguf_gate_up_silu_mul_over)
    dt = {"q4_k": lib.TYPE_Q4_K, "q6_k": lib.TYPE_Q6_K, **TABLE_TAIL}[name]
    tokens, hidden, ffn, n_experts, topk, cut = 5, 512, 256, 6, 3, 4
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=65, dt_down=dt, dt_gu=dt, x_scale=4.0)
    routing = ExpertRouting(dev(ids))
    flat_w = dev(w.reshape(-1))
    want_h = moe_gemm_gguf_gate_up_silu_mul(dt, dev(x), dev(gate), dev(up), routing, n_experts, ffn)
    want = moe_gemm_gguf_down_reduce(dt, want_h, dev(down), routing, flat_w, n_experts, hidden)

    def halves(stack):   # experts 0..cut-1 in one allocation, cut.. in another
        per = stack.reshape(n_experts, -1)
        return dev(np.ascontiguousarray(per[:cut])), dev(np.ascontiguousarray(per[cut:]))

    (g0, g1), (u0, u1), (d0, d1) = halves(gate), halves(up), halves(down)
    h = moe_gemm_gguf_gate_up_silu_mul_over(dt, dev(x), g0, u0, g1, u1, cut, routing, n_experts, ffn)
    assert torch.equal(h, want_h)
    # the second pair named by addresses on the card; the host-side ones are then ignored
    at = torch.tensor([g1.data_ptr(), u1.data_ptr()], dtype=torch.int64, device="cuda")
    h2 = moe_gemm_gguf_gate_up_silu_mul_over(dt, dev(x), g0, u0, g0, u0, cut, routing, n_experts, ffn, more_at=at)
    assert torch.equal(h2, want_h)
    bias = torch.randn((n_experts, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))
    assert torch.equal(moe_gemm_gguf_down_reduce_over(dt, want_h, d0, d1, cut, routing, flat_w, n_experts, hidden), want)
    assert torch.equal(moe_gemm_gguf_down_reduce_over(dt, want_h, d0, d1, cut, routing, flat_w, n_experts, hidden, down_bias=bias),
                       moe_gemm_gguf_down_reduce(dt, want_h, dev(down), routing, flat_w, n_experts, hidden, down_bias=bias))
    rows = moe_gemm_gguf_down_pairs_over(dt, want_h, d0, d1, cut, routing, flat_w, n_experts, hidden)
    assert (rows.reshape(tokens, topk, hidden).sum(1) - want).abs().max().item() <= 1e-6 * want.abs().max().item()
    at_d = torch.tensor([d1.data_ptr(), 0], dtype=torch.int64, device="cuda")
    assert torch.equal(moe_gemm_gguf_down_pairs_over(dt, want_h, d0, d0, cut, routing, flat_w, n_experts, hidden, more_at=at_d), rows)


def test_decode_launchers_refuse_wire_ids_outside_the_table():
    tokens, hidden, ffn, n_experts, topk = 2, 512, 256, 4, 2
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=62)
    routing = ExpertRouting(dev(ids))
    L = lib.load()
    out = torch.empty((tokens * topk, ffn), device="cuda")
    for wire in (16, 17, 99, -1):   # the table ends at 15 (src/inference/moe_cuda/gemm.rs:23-39)
        rc = L.loken_moe_gemm_gguf(dev(x).data_ptr(), dev(gate).data_ptr(), routing.sorted_token_ids.data_ptr(),
                                   routing.expert_ids.data_ptr(), None, out.data_ptr(), n_experts, topk,
                                   tokens * topk, ffn, hidden, wire, None)
        assert rc == lib.LK_ERR_TYPE


def test_decode_down_reduce_is_tight_on_oracle_rows_and_folds_in_slot_order():
    tokens, hidden, ffn, n_experts, topk = 4, 512, 512, 8, 3
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=58)
    want, want_h = oracle.moe_forward(1, lib.TYPE_Q4_K, lib.TYPE_Q4_K, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    routing = ExpertRouting(dev(ids))
    h = dev(slot_order(want_h, ids))
    out = moe_gemm_gguf_down_reduce(lib.TYPE_Q4_K, h, dev(down), routing, dev(w.reshape(-1)), n_experts, hidden)
    assert_close(out.cpu().numpy(), want, atol=1e-4 * max(1.0, np.abs(want).max()))
    # residual as the starting value, add_after as a written sum, bias scaled by the router weight
    res = torch.randn((tokens, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(5))
    with_res = moe_gemm_gguf_down_reduce(lib.TYPE_Q4_K, h, dev(down), routing, dev(w.reshape(-1)), n_experts, hidden, residual=res)
    added = moe_gemm_gguf_down_reduce(lib.TYPE_Q4_K, h, dev(down), routing, dev(w.reshape(-1)), n_experts, hidden, add_after=res)
    scale = out.abs().max().item() + res.abs().max().item()
    assert (with_res - (out + res)).abs().max().item() <= 1e-6 * scale
    assert (added - (out + res)).abs().max().item() <= 1e-6 * scale
    bias = torch.randn((n_experts, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(6))
    biased = moe_gemm_gguf_down_reduce(lib.TYPE_Q4_K, h, dev(down), routing, dev(w.reshape(-1)), n_experts, hidden, down_bias=bias)
    wt = dev(w)
    extra = (wt.unsqueeze(-1) * bias[dev(ids).long()]).sum(dim=1)
    assert (biased - (out + extra)).abs().max().item() <= 1e-5 * (scale + extra.abs().max().item())


def test_generic_routed_product_with_and_without_weights():
    tokens, k, n, n_experts, topk = 5, 512, 96, 7, 2
    wq = synth.weight(lib.TYPE_Q8_0, n_experts * n, k, seed=59, stream=1)
    x = synth.activation(tokens, k, seed=59)
    ids, w = oracle.topk_softmax(synth.activation(tokens, n_experts, seed=59, stream=7), topk)
    routing = ExpertRouting(dev(ids))
    we = wq.reshape(n_experts, n, -1, 34)
    plain = moe_gemm_gguf(lib.TYPE_Q8_0, dev(x), dev(wq), routing, n_experts, n).cpu().numpy()
    for t in range(tokens):
        for j in range(topk):
            assert_close(plain[t * topk + j], oracle.ob_matmul(lib.TYPE_Q8_0, x[t:t + 1], we[ids[t, j]], n)[0])
    # with routing weights: one activation row per slot, output scaled
    xs = synth.activation(tokens * topk, k, seed=59, stream=8)
    scaled = moe_gemm_gguf(lib.TYPE_Q8_0, dev(xs), dev(wq), routing, n_experts, n, topk_weights=dev(w.reshape(-1))).cpu().numpy()
    for p in range(tokens * topk):
        e = ids.reshape(-1)[p]
        assert_close(scaled[p], w.reshape(-1)[p] * oracle.ob_matmul(lib.TYPE_Q8_0, xs[p:p + 1], we[e], n)[0])


@pytest.mark.parametrize("half", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name", ["q4_k", "q6_k", "q8_0", "q5_1"])
def test_prefill_form_takes_half_precision_rows(name, half):
    # loken_moe_gemm_gguf_prefill: the rows arrive as f16 / bf16; the oracle is fed the values they hold
    from loken_amd.moe import moe_gemm_gguf_prefill
    wtype = {"q4_k": lib.TYPE_Q4_K, "q6_k": lib.TYPE_Q6_K, "q8_0": lib.TYPE_Q8_0, "q5_1": lib.TYPE_Q5_1}[name]
    tokens, k, n, n_experts, topk = 9, 512, 96, 6, 2
    wq = synth.weight(wtype, n_experts * n, k, seed=61, stream=1)
    ids, w = oracle.topk_softmax(synth.activation(tokens, n_experts, seed=61, stream=7), topk)
    routing = ExpertRouting(dev(ids))
    we = wq.reshape(n_experts, -1)   # an expert's n rows of blocks
    xh = dev(synth.activation(tokens, k, seed=61)).to(half)
    x_seen = xh.to(torch.float32).cpu().numpy()
    got = moe_gemm_gguf_prefill(wtype, xh, dev(wq), routing, n_experts, n).cpu().numpy()
    for t in range(tokens):
        for j in range(topk):
            assert_close(got[t * topk + j], oracle.ob_matmul(wtype, x_seen[t:t + 1], we[ids[t, j]], n)[0])
    # the same values as f32 rows through the decode-form launch: the same bits
    same = moe_gemm_gguf(wtype, xh.to(torch.float32), dev(wq), routing, n_experts, n).cpu().numpy()
    assert np.array_equal(got, same)
    # with routing weights: one activation row per slot, output scaled
    xs = dev(synth.activation(tokens * topk, k, seed=61, stream=8)).to(half)
    scaled = moe_gemm_gguf_prefill(wtype, xs, dev(wq), routing, n_experts, n, topk_weights=dev(w.reshape(-1))).cpu().numpy()
    xs_seen = xs.to(torch.float32).cpu().numpy()
    for p in range(tokens * topk):
        e = ids.reshape(-1)[p]
        assert_close(scaled[p], w.reshape(-1)[p] * oracle.ob_matmul(wtype, xs_seen[p:p + 1], we[e], n)[0])
    # an input width the launch does not know is a status, not a launch
    L = lib.load()
    assert L.loken_moe_gemm_gguf_prefill(xh.data_ptr(), dev(wq).data_ptr(), routing.sorted_token_ids.data_ptr(),
                                         routing.expert_ids.data_ptr(), None, dev(np.zeros(4, np.float32)).data_ptr(),
                                         n_experts, topk, tokens * topk, n, k, 2, 1, None) == lib.LK_ERR_TYPE


@pytest.mark.parametrize("tokens,hidden,ffn,n_experts,topk", [(1, 2048, 768, 128, 8), (16, 2048, 768, 128, 8),
                                                              (5, 100, 512, 9, 4), (7, 264, 1024, 12, 6),
                                                              (3, 77, 768, 5, 1), (40, 96, 512, 16, 8), (64, 64, 512, 16, 8)])
@pytest.mark.parametrize("name", ["q4_k", "q5_k", "q6_k"])
def test_down_and_fold_in_one_launch_gives_the_bits_of_the_two_launches(name, tokens, hidden, ffn, n_experts, topk, knobs):
    """Short K-quant rows at a handful of tokens take one launch (down + fold); with that launch switched
    off the same call takes the per-pair mat-vec and the fold kernel. Same bits, and both on the oracle."""
    dt, block_bytes = {"q4_k": (lib.TYPE_Q4_K, 144), "q5_k": (lib.TYPE_Q5_K, 176), "q6_k": (lib.TYPE_Q6_K, 210)}[name]
    down = synth.weight(dt, n_experts * hidden, ffn, seed=61, stream=3)
    ids, w = oracle.topk_softmax(synth.activation(tokens, n_experts, seed=61, stream=7), topk)
    h = synth.activation(tokens * topk, ffn, seed=61, stream=4) * np.float32(5.0)
    routing = ExpertRouting(dev(ids))
    bias = torch.randn((n_experts, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(9))
    res = torch.randn((tokens, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(10))
    down_d, h_d, w_d = dev(down), dev(h), dev(w.reshape(-1))

    def run(**kw):
        return moe_gemm_gguf_down_reduce(dt, h_d, down_d, routing, w_d, n_experts, hidden, **kw)

    cases = ({}, {"residual": res}, {"add_after": res}, {"down_bias": bias}, {"down_bias": bias, "add_after": res})
    one = [run(**kw) for kw in cases]
    # a pair whose expert is out of range, in the one launch
    keep = routing.expert_ids[0].item()
    routing.expert_ids[0] = -1
    one_dropped = run()
    knobs.set("LK_TUNE_DOWN_FOLD_OFF")
    two_dropped = run()
    routing.expert_ids[0] = keep
    two = [run(**kw) for kw in cases]
    for a, b in zip(one, two):
        assert torch.equal(a, b)
    assert torch.equal(one_dropped, two_dropped)
    we = down.reshape(n_experts, hidden, -1, block_bytes)
    want = np.zeros((tokens, hidden), np.float32)
    for t in range(tokens):
        for j in range(topk):
            p = t * topk + j
            want[t] += w[t, j] * oracle.ob_matmul(dt, h[p:p + 1], we[ids[t, j]], hidden)[0]
    assert_close(one[0].cpu().numpy(), want, atol=1e-4 * max(1.0, np.abs(want).max()))


def test_pairs_the_routing_leaves_out_add_nothing():
    tokens, hidden, ffn, n_experts, topk = 3, 256, 256, 4, 2
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=60)
    routing = ExpertRouting(dev(ids))
    h = moe_gemm_gguf_gate_up_silu_mul(lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), routing, n_experts, ffn)
    full = moe_gemm_gguf_down_reduce(lib.TYPE_Q4_K, h, dev(down), routing, dev(w.reshape(-1)), n_experts, hidden)
    # mark the first sorted pair as belonging to no expert: the fold must see zeros for it
    dropped = routing.sorted_token_ids[0].item()
    routing.expert_ids[0] = n_experts + 3
    part = moe_gemm_gguf_down_reduce(lib.TYPE_Q4_K, h, dev(down), routing, dev(w.reshape(-1)), n_experts, hidden)
    t = dropped // topk
    others = [i for i in range(tokens) if i != t]
    assert torch.equal(part[others], full[others])
    assert not torch.equal(part[t], full[t])


def test_launchers_report_bad_arguments_and_formats():
    l = lib.load()
    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p, s = buf.data_ptr(), torch.cuda.current_stream().cuda_stream
    assert l.loken_moe_gemm_gguf(p, p, p, p, None, p, 4, 2, 4, 8, 256, 16, s) == lib.LK_ERR_TYPE    # past the table's last row
    assert l.loken_moe_gemm_gguf(p, p, p, p, None, p, 4, 2, 4, 8, 250, 1, s) == lib.LK_ERR_ARG      # k not whole blocks
    assert l.loken_moe_gemm_gguf(p, p, p, p, None, p, 4, 2, 5, 8, 256, 1, s) == lib.LK_ERR_ARG      # pairs % topk
    assert l.loken_moe_gemm_gguf_down_reduce(p, p, p, p, None, p, 4, 2, 4, 8, 256, 1, None, None, s) == lib.LK_ERR_ARG
    assert l.loken_moe_gemm_gguf(p, p, p, p, None, p, 4, 2, 0, 8, 256, 1, s) == lib.LK_OK           # nothing routed
    l.loken_stream_scratch_release()


@pytest.mark.parametrize("tokens", [1, 16, 256])
def test_layer_entry_picks_a_path_and_both_agree(tokens):
    hidden, ffn, n_experts, topk = 512, 256, 16, 4
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=61)
    args = (lib.TYPE_Q4_K, lib.TYPE_Q4_K, dev(x), dev(gate), dev(up), dev(down), dev(ids), dev(w), n_experts, ffn)
    got, rows = moe_forward(*args, return_rows=True)
    want, want_h = oracle.moe_forward(1, lib.TYPE_Q4_K, lib.TYPE_Q4_K, x, gate, up, down, ids, w, n_experts, ffn, want_h=True)
    want_slot = slot_order(want_h, ids)
    sample = None if tokens <= 16 else np.arange(0, tokens, 16)
    check_block(got.cpu().numpy(), rows.cpu().numpy(), want, want_slot, lib.TYPE_Q4_K, down, ids, w, n_experts, hidden,
                tokens=sample)


# ---------------------------------------------------------------- router
@pytest.mark.parametrize("tokens,experts,topk,renorm", [(1, 128, 8, True), (16, 128, 8, True), (256, 128, 8, False),
                                                        (7, 60, 4, True), (5, 512, 64, True), (3, 8, 8, False)])
def test_router_topk_softmax_matches_oracle(tokens, experts, topk, renorm):
    logits = synth.normal(90, tokens * 1000 + experts, tokens * experts).astype(np.float32).reshape(tokens, experts)
    want_ids, want_w = oracle.topk_softmax(logits, topk, renorm)
    w, ids = moe.topk_softmax(dev(logits), topk, renorm)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.allclose(w.cpu().numpy(), want_w, rtol=1e-5, atol=1e-7)


def test_router_ties_go_to_the_lower_expert_and_weights_descend():
    logits = np.zeros((2, 128), np.float32)
    logits[1, [5, 40, 41, 100]] = [2.0, 3.0, 3.0, 2.0]
    w, ids = moe.topk_softmax(dev(logits), 8, True)
    ids, w = ids.cpu().numpy(), w.cpu().numpy()
    assert ids[0].tolist() == list(range(8)) and np.allclose(w[0], 1.0 / 8)
    assert ids[1, :4].tolist() == [40, 41, 5, 100] and ids[1, 4:].tolist() == [0, 1, 2, 3]
    assert (np.diff(w[1]) <= 0).all() and abs(w[1].sum() - 1.0) < 1e-6


@pytest.mark.parametrize("tokens,topk,n_experts", [(3, 2, 5), (8, 4, 16), (1, 8, 128)])
def test_q4k_pair_rows_over_caller_quantized_rows_with_one_expert_per_pair(tokens, topk, n_experts):
    """loken_moe_q4k_imma_m8_gate_up and loken_moe_q4k_imma_m8_down: Q8_1 rows from the caller,
    expert ids per pair (one of them out of range), GELU on the gate. The products are the
    same-codes oracle's (cuda/moe/moe_q4k_imma_m8.cu:273-296, moe_q4k_imma_m8_down.cu:196-230)."""
    from loken_amd.moe import moe_q4k_imma_m8_down_reduce, moe_q4k_imma_m8_gate_up
    hidden, ffn = 512, 256
    gate, up, down, x, ids, w = make_layer(tokens, hidden, ffn, n_experts, topk, seed=66, x_scale=4.0)
    slots, experts = oracle.group_by_expert(ids)
    experts = experts.copy()
    dropped = len(slots) // 2
    experts[dropped] = n_experts + 3          # a pair the routing leaves out
    gate_rows, up_rows = gate.reshape(n_experts, ffn, -1), up.reshape(n_experts, ffn, -1)
    both = np.ascontiguousarray(np.concatenate([gate_rows, up_rows], axis=1))
    pairs = tokens * topk
    want_h = np.zeros((pairs, ffn), np.float64)
    for j in range(pairs):
        if experts[j] >= n_experts:
            continue
        row = x[slots[j] // topk][None, :]
        g = oracle.ob_matmul(lib.TYPE_Q4_K, row, gate_rows[experts[j]].reshape(-1), ffn)[0].astype(np.float64)
        u = oracle.ob_matmul(lib.TYPE_Q4_K, row, up_rows[experts[j]].reshape(-1), ffn)[0].astype(np.float64)
        want_h[slots[j]] = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3))) * u
    sd, ed = dev(slots.astype(np.int32)), dev(experts.astype(np.int32))
    h = moe_q4k_imma_m8_gate_up(dev(x), dev(both), sd, ed, n_experts, topk, ffn)
    got_h = h.cpu().numpy()
    assert (got_h[slots[dropped]] == 0).all()
    assert (np.abs(got_h - want_h) <= 1e-3 * np.abs(want_h) + 1e-4 * np.abs(want_h).max()).all()

    # down from the device's own h, so that the two sides quantize the same rows
    down_rows = down.reshape(n_experts, hidden, -1)
    flat_w = w.reshape(-1).astype(np.float32)
    want = np.zeros((tokens, hidden), np.float64)
    for slot in range(pairs):                 # slot order: the fold's order
        j = int(np.nonzero(slots == slot)[0][0])
        if experts[j] >= n_experts:
            continue
        y = oracle.ob_matmul(lib.TYPE_Q4_K, got_h[slot][None, :], down_rows[experts[j]].reshape(-1), hidden)[0]
        want[slot // topk] += (y * flat_w[slot]).astype(np.float64)
    got = moe_q4k_imma_m8_down_reduce(h, dev(down), sd, ed, dev(flat_w), n_experts, topk, hidden).cpu().numpy()
    assert (np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-4 * np.abs(want).max()).all()


@pytest.mark.parametrize("hint", [1, 9, 40])
# a wave per 16-row tile (2, 3, 4, 8 super-blocks: every load depth), a wave per 32-row tile (1, 5, 6), or four
# waves splitting a tile's super-blocks (10)
@pytest.mark.parametrize("k", [256, 512, 768, 1024, 1280, 1536, 2048, 2560])
def test_rows_launch_serves_any_run_length_whatever_the_hint(hint, k):
    """lk_moe_q4k_rows_grouped: the hint only picks the pass width (8, 16 or 32 rows); an expert with
    more rows takes more passes, one without rows none, and gather / scatter follow the routing."""
    rng = np.random.default_rng(67)
    n_experts, n, tokens = 5, 100, 30
    counts = [37, 0, 1, 9, 13]                              # sorted rows per expert
    rows = sum(counts)
    bounds = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    src = rng.integers(0, tokens, rows).astype(np.int32)    # sorted row -> token
    dst_map = rng.permutation(rows).astype(np.int32)        # sorted row -> output row
    w = synth.weight(lib.TYPE_Q4_K, n_experts * n, k, seed=67, stream=1)
    w2 = synth.weight(lib.TYPE_Q4_K, n_experts * n, k, seed=67, stream=2)
    x = synth.activation(tokens, k, seed=67) * np.float32(4.0)
    q = ops.quantize_q8_1_rows(dev(x), k_padded=k)
    expert_of = np.repeat(np.arange(n_experts), counts)
    per = w.reshape(n_experts, n, -1), w2.reshape(n_experts, n, -1)
    prod = [np.stack([oracle.ob_matmul(lib.TYPE_Q4_K, x[src[i]][None, :], m[expert_of[i]].reshape(-1), n)[0]
                      for i in range(rows)]).astype(np.float64) for m in per]
    L = lib.load()
    s = torch.cuda.current_stream().cuda_stream
    wd, w2d, bd, sd, dd = dev(w), dev(w2), dev(bounds), dev(src), dev(dst_map)
    # plain product, scattered
    out = torch.full((rows, n), -9.0, device="cuda")
    lib.check("lk_moe_q4k_rows_grouped", L.lk_moe_q4k_rows_grouped(
        wd.data_ptr(), None, 0, q.data_ptr(), k // 32, bd.data_ptr(), sd.data_ptr(), dd.data_ptr(), out.data_ptr(), n,
        n_experts, n * (k // 256) * 144, n, k, hint, s))
    got = out.cpu().numpy()
    want = np.empty_like(prod[0])
    want[dst_map] = prod[0]
    assert (np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-4).all()
    # gate and up with SiLU, rows left in sorted order
    out2 = torch.full((rows, n), -9.0, device="cuda")
    lib.check("lk_moe_q4k_rows_grouped", L.lk_moe_q4k_rows_grouped(
        wd.data_ptr(), w2d.data_ptr(), 0, q.data_ptr(), k // 32, bd.data_ptr(), sd.data_ptr(), None, out2.data_ptr(), n,
        n_experts, n * (k // 256) * 144, n, k, hint, s))
    g, u = prod
    want2 = g / (1.0 + np.exp(-g)) * u
    got2 = out2.cpu().numpy()
    assert (np.abs(got2 - want2) <= 1e-3 * np.abs(want2) + 1e-4 * np.abs(want2).max()).all()

"""The entry point that allocates nothing, loken_moe_gemm_gguf_down_reduce_static, against the
entry point it is a variant of (loken_moe_gemm_gguf_down_reduce): same arguments through the C
ABI, bit-identical outputs, on two calls in a row, the second with a smaller input, for a format
whose kernels read the f32 rows themselves (only the pairs' rows use the fixed array) and for one
that also keeps its Q8_1 rows there. A call past the array's size is refused with LK_ERR_SIZE."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, moe, synth

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def call(fn_name, wire, h, down, routing, w, n_experts, hidden, bias, add):
    l = lib.load()
    pairs, k = h.shape
    out = torch.full((pairs // routing.topk, hidden), 3.0, dtype=torch.float32, device="cuda")
    rc = getattr(l, fn_name)(h.data_ptr(), down.data_ptr(), routing.sorted_token_ids.data_ptr(),
                             routing.expert_ids.data_ptr(), w.data_ptr(), out.data_ptr(), n_experts, routing.topk, pairs,
                             hidden, k, wire, bias.data_ptr() if bias is not None else None,
                             add.data_ptr() if add is not None else None, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return rc, out


@pytest.mark.parametrize("wtype", [lib.TYPE_Q4_K, lib.TYPE_Q5_0])
def test_static_scratch_entry_matches_the_allocating_one_twice_in_a_row(wtype):
    n_experts, hidden, ffn, topk = 8, 512, 256, 2
    wire = moe.EXPERT_QUANT_CODES[wtype]
    down = dev(synth.weight(wtype, n_experts * hidden, ffn, seed=90, stream=3))
    bias = dev(synth.activation(n_experts, hidden, seed=90, stream=5))
    for tokens in (12, 5):   # the second call is smaller: the array still holds the first call's rows
        h = dev(synth.activation(tokens * topk, ffn, seed=90 + tokens) * np.float32(3.0))
        ids, w = oracle.topk_softmax(synth.activation(tokens, n_experts, seed=90 + tokens, stream=7), topk)
        routing = moe.ExpertRouting(dev(ids))
        wd = dev(w.reshape(-1))
        add = dev(synth.activation(tokens, hidden, seed=91, stream=9))
        for b, a in ((None, None), (bias, add)):
            rc0, want = call("loken_moe_gemm_gguf_down_reduce", wire, h, down, routing, wd, n_experts, hidden, b, a)
            rc1, got = call("loken_moe_gemm_gguf_down_reduce_static", wire, h, down, routing, wd, n_experts, hidden, b, a)
            assert rc0 == 0 and rc1 == 0
            assert torch.equal(got, want)


def test_static_scratch_entry_refuses_what_does_not_fit():
    l = lib.load()
    # size_m * size_n * 4 bytes of pair rows alone pass the array: nothing may be launched
    size_m, size_n, size_k = 1024, 4096, 256
    assert size_m * size_n * 4 > lib.STATIC_SCRATCH_BYTES
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    out = torch.full((16,), 5.0, device="cuda")
    p = buf.data_ptr()
    rc = l.loken_moe_gemm_gguf_down_reduce_static(p, p, p, p, p, out.data_ptr(), 4, 2, size_m, size_n, size_k, 1, None, None,
                                                  torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == lib.LK_ERR_SIZE
    assert (out == 5.0).all()


def test_static_scratch_entry_recorded_into_a_graph_replays_to_the_eager_bits():
    """What the entry point is for: the call recorded into a HIP graph (after one eager call on the device,
    which resolves the fixed array's address), replayed three times with the program's own eager work and
    synchronizations between the replays, every replay bit for bit the eager result."""
    n_experts, hidden, ffn, topk, tokens = 8, 512, 256, 2, 9
    for wtype in (lib.TYPE_Q4_K, lib.TYPE_Q5_0):
        wire = moe.EXPERT_QUANT_CODES[wtype]
        down = dev(synth.weight(wtype, n_experts * hidden, ffn, seed=95, stream=3))
        h = dev(synth.activation(tokens * topk, ffn, seed=96) * np.float32(3.0))
        ids, w = oracle.topk_softmax(synth.activation(tokens, n_experts, seed=96, stream=7), topk)
        routing = moe.ExpertRouting(dev(ids))
        wd = dev(w.reshape(-1))
        add = dev(synth.activation(tokens, hidden, seed=97, stream=9))
        rc, want = call("loken_moe_gemm_gguf_down_reduce_static", wire, h, down, routing, wd, n_experts, hidden, None, add)
        assert rc == 0
        l = lib.load()
        out = torch.zeros((tokens, hidden), dtype=torch.float32, device="cuda")
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                rc = l.loken_moe_gemm_gguf_down_reduce_static(
                    h.data_ptr(), down.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
                    wd.data_ptr(), out.data_ptr(), n_experts, topk, tokens * topk, hidden, ffn, wire, None, add.data_ptr(),
                    side.cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        for replay in range(3):
            out.fill_(7.0)
            # eager work of the program between the replays: another call through the same array, smaller
            rc2, _ = call("loken_moe_gemm_gguf_down_reduce_static", wire, h[: 2 * topk], down,
                          moe.ExpertRouting(dev(ids[:2])), dev(w[:2].reshape(-1)), n_experts, hidden, None, add[:2].contiguous())
            assert rc2 == 0
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want), f"replay {replay}"

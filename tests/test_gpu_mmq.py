"""GPU parity of the prefill path (workspace quantizer + int8-MFMA tiled matmul).

Same bars as the decode path: workspace codes / scales / sums bit-exact with loken's
BlockQ8_1::quantize; f32 outputs within 1e-3 relative + 1e-4 absolute of the same-codes oracle;
and the family-vs-family check the reference runs (tiled matmul vs mat-vec on the same weights,
src/tensor/quantized/tests.rs:848-921), here to a much tighter bound since both families see
identical integer codes.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, ops, synth

pytestmark = pytest.mark.gpu

DT = {"q4_k": lib.TYPE_Q4_K, "q5_k": lib.TYPE_Q5_K, "q6_k": lib.TYPE_Q6_K, "q8_0": lib.TYPE_Q8_0,
      "q4_0": lib.TYPE_Q4_0, "q4_1": lib.TYPE_Q4_1, "q5_0": lib.TYPE_Q5_0, "q5_1": lib.TYPE_Q5_1,
      "q3_k": lib.TYPE_Q3_K, "q2_k": lib.TYPE_Q2_K}
SERVED = [name for name in DT if hasattr(lib.load(), ops.MMQ_LAUNCHER[DT[name]])]
RTOL, ATOL = 1e-3, 1e-4


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    bad = np.abs(got - want) > RTOL * np.abs(want) + ATOL
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; worst {np.abs(got - want).max()}"


def unpack_workspace(ws: np.ndarray, rows: int, k_padded: int):
    """-> codes int8 [rows, k_padded], d f16 [rows, k_padded/32], sums int16 [rows, k_padded/32]"""
    nkb = k_padded // 256
    rec = ws[: nkb * rows * 288].reshape(nkb, rows, 288)
    codes = rec[:, :, :256].copy().view(np.int8).transpose(1, 0, 2).reshape(rows, k_padded)
    d = rec[:, :, 256:272].copy().view(np.float16).transpose(1, 0, 2).reshape(rows, nkb * 8)
    sums = rec[:, :, 272:288].copy().view(np.int16).transpose(1, 0, 2).reshape(rows, nkb * 8)
    return codes, d, sums


@pytest.mark.parametrize("rows,k", [(1, 256), (7, 1000), (130, 4096), (33, 768)])
@pytest.mark.parametrize("f16", [False, True])
def test_workspace_quantizer_is_bit_exact(rows, k, f16):
    x = synth.activation(rows, k, seed=41) * np.float32(1.7)
    xt = dev(x).to(torch.float16) if f16 else dev(x)
    x_seen = xt.to(torch.float32).cpu().numpy()
    kp = ops.pad_to(k, 512)
    ws = ops.mmq_quantize(lib.TYPE_Q4_K, xt).cpu().numpy()
    codes, d, sums = unpack_workspace(ws, rows, kp)
    padded = np.zeros((rows, kp), np.float32)
    padded[:, :k] = x_seen
    want = oracle.quantize_q8_1(padded).reshape(rows, kp // 32, 36)
    assert np.array_equal(codes.reshape(rows, kp // 32, 32), want[:, :, 4:].view(np.int8))
    assert np.array_equal(d.view(np.uint16), want[:, :, 0:2].copy().view(np.uint16).reshape(rows, -1))
    assert np.array_equal(sums.astype(np.int32), want[:, :, 4:].view(np.int8).astype(np.int32).sum(axis=2))


def test_workspace_quantizer_gathers_rows():
    x = synth.activation(9, 512, seed=42)
    ids = np.array([3, 3, 0, 8, 1, 1, 1, 7], np.int32)
    ws = ops.mmq_quantize(lib.TYPE_Q4_K, dev(x), gather=dev(ids)).cpu().numpy()
    codes, d, _ = unpack_workspace(ws, len(ids), 512)
    want = oracle.quantize_q8_1(x[ids]).reshape(len(ids), 16, 36)
    assert np.array_equal(codes.reshape(len(ids), 16, 32), want[:, :, 4:].view(np.int8))
    assert np.array_equal(d.view(np.uint16), want[:, :, 0:2].copy().view(np.uint16).reshape(len(ids), -1))


SHAPES = [(6, 256, 128), (8, 512, 64), (33, 768, 130), (64, 1024, 256), (65, 1024, 129), (128, 2048, 384),
          (200, 4096, 300), (1, 256, 1), (129, 256, 257)]


@pytest.mark.parametrize("name", SERVED)
@pytest.mark.parametrize("m,k,n", SHAPES)
def test_tiled_matmul_matches_same_codes_oracle(name, m, k, n):
    wtype = DT[name]
    w = synth.weight(wtype, n, k, seed=43, stream=1)
    x = synth.activation(m, k, seed=43)
    got = ops.mmq_forward(wtype, dev(w), dev(x), n).cpu().numpy()
    assert_close(got, oracle.ob_matmul(wtype, x, w, n))


@pytest.mark.parametrize("name", SERVED)
def test_tiled_matmul_agrees_with_matvec_family(name):
    wtype = DT[name]
    m, k, n = 40, 2048, 520
    w = dev(synth.weight(wtype, n, k, seed=44, stream=2))
    x = dev(synth.activation(m, k, seed=44))
    tiled = ops.mmq_forward(wtype, w, x, n)
    q = ops.quantize_q8_1_rows(x)
    rows = torch.cat([ops.mmvq(wtype, w, q[i:i + 8], k, n) for i in range(0, m, 8)])
    # same integers on both sides: only f32 summation order differs
    scale = rows.abs().max().item()
    assert (tiled - rows).abs().max().item() <= 2e-5 * scale


@pytest.mark.parametrize("name", SERVED)
@pytest.mark.parametrize("m,k,n", [(20, 1280, 132), (64, 2048, 256), (100, 1280, 512), (300, 3584, 264), (7, 7168, 8)])
def test_cut_k_follows_the_oracle_and_the_plain_launch(name, m, k, n):
    # Given the caller's tmp_fixup (FIXUP_BYTES of src/tensor/quantized/kernel_matmul/mmq.rs:42) a product of
    # few tiles is launched over ranges of K (5, 8, 14 and 28 blocks here: uneven ranges too) and the
    # partial products are added in ascending order: the same integers, another order of f32 sums, and
    # nothing that depends on which workgroup finished first.
    wtype = DT[name]
    w = dev(synth.weight(wtype, n, k, seed=47, stream=5))
    xh = synth.activation(m, k, seed=47)
    x = dev(xh)
    plain = ops.mmq_forward(wtype, w, x, n, fixup=False)
    cut = ops.mmq_forward(wtype, w, x, n)
    again = ops.mmq_forward(wtype, w, x, n)
    assert torch.equal(cut, again)
    assert_close(cut.cpu().numpy(), oracle.ob_matmul(wtype, xh, w.cpu().numpy(), n))
    assert (cut - plain).abs().max().item() <= 2e-5 * plain.abs().max().item()


@pytest.mark.parametrize("m,k,n", [(100, 1280, 2052), (40, 1792, 2304), (200, 3584, 2048)])
def test_cut_k_on_the_f16_tiles_of_q4k_follows_the_oracle(m, k, n):
    # 2048 weight rows or more and 33 token rows or more: the 64-token f16 tiles, here few enough to have K
    # cut (5, 7 and 14 blocks: uneven ranges)
    wtype = lib.TYPE_Q4_K
    wh = synth.weight(wtype, n, k, seed=49, stream=8)
    xh = synth.activation(m, k, seed=49)
    w, x = dev(wh), dev(xh)
    plain = ops.mmq_forward(wtype, w, x, n, fixup=False)
    cut = ops.mmq_forward(wtype, w, x, n)
    assert torch.equal(cut, ops.mmq_forward(wtype, w, x, n))
    assert not torch.equal(cut, plain)
    pick = np.sort(np.random.default_rng(49).choice(n, 256, replace=False))
    assert_close(cut.cpu().numpy()[:, pick], oracle.ob_matmul(wtype, xh, wh[pick], len(pick)))
    assert (cut - plain).abs().max().item() <= 2e-5 * plain.abs().max().item()


@pytest.mark.parametrize("name,m,k,n", [("q6_k", 48, 2048, 260), ("q4_k", 100, 1792, 2304)])
def test_cut_k_recorded_into_a_graph_replays_to_the_eager_bits(name, m, k, n):
    # The cut-K call is two launches and nothing else (no fill, no allocation): recorded into a HIP graph
    # and replayed three times, with eager calls of another size through the same tmp_fixup between the
    # replays, every replay carries the eager call's bits.
    wtype = DT[name]
    w = dev(synth.weight(wtype, n, k, seed=50, stream=9))
    x = dev(synth.activation(m, k, seed=50))
    want = ops.mmq_forward(wtype, w, x, n)
    assert not torch.equal(want, ops.mmq_forward(wtype, w, x, n, fixup=False))   # K was cut
    ws = ops.mmq_quantize(wtype, x)
    out = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    fn = getattr(lib.load(), ops.MMQ_LAUNCHER[wtype])
    i = ops.MMQ_DEVICE_INFO
    fix = ops.mmq_fixup(x.device)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            launched = fn(fix.data_ptr(), w.data_ptr(), ws.data_ptr(), out.data_ptr(), k, n, m, k // synth.BLOCK_LEN[wtype], n,
                          i["cc"], i["nsm"], i["smpbo"], i["warp_size"], side.cuda_stream)
    assert launched != 0
    torch.cuda.synchronize()
    for replay in range(3):
        out.fill_(7.0)
        ops.mmq_forward(wtype, w, x[: m // 2].contiguous(), n)   # the program's own work through the same buffer
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {replay}"


@pytest.mark.parametrize("name,splits", [("q4_k", 3), ("q6_k", 7), ("q8_0", 2), ("q4_k", 64)])
def test_forced_range_counts_and_what_keeps_k_whole(name, splits, knobs):
    # LK_TUNE_MMQ_SPLITS asks for a range count (capped so that a range keeps two blocks); -1, no buffer,
    # or a row length that is not a multiple of four floats leave K whole: then the bits are the plain launch's.
    wtype = DT[name]
    m, k, n = 70, 2560, 260
    w = dev(synth.weight(wtype, n, k, seed=48, stream=6))
    xh = synth.activation(m, k, seed=48)
    x = dev(xh)
    plain = ops.mmq_forward(wtype, w, x, n, fixup=False)
    knobs.set("LK_TUNE_MMQ_SPLITS", str(splits))
    cut = ops.mmq_forward(wtype, w, x, n)
    knobs.set("LK_TUNE_MMQ_SPLITS", "-1")
    whole = ops.mmq_forward(wtype, w, x, n)
    knobs.clear("LK_TUNE_MMQ_SPLITS")
    assert torch.equal(whole, plain)
    assert not torch.equal(cut, plain)
    assert_close(cut.cpu().numpy(), oracle.ob_matmul(wtype, xh, w.cpu().numpy(), n))
    w_odd = dev(synth.weight(wtype, 130, k, seed=48, stream=7))
    assert torch.equal(ops.mmq_forward(wtype, w_odd, x, 130), ops.mmq_forward(wtype, w_odd, x, 130, fixup=False))


@pytest.mark.parametrize("m,k,n", [(65, 256, 2049), (40, 512, 2050), (130, 2048, 2056), (300, 1024, 2304), (500, 512, 8450)])
def test_q4k_wide_tiles_agree_with_int8_tiles_and_matvec(m, k, n, knobs):
    # Above 32 token rows of a matrix of 2048 rows or more Q4_K forms its sub-block dots on the f16 matrix
    # unit (scale folded into the weight operand; 64-token tiles, K cut into ranges where they are few; the
    # last shape has enough 128-token tiles for the kernel that expands the token side once per call);
    # LK_MMQ_I8 sends the same call to the int8 tiles. Same integers either way, so only the f32
    # summation order may differ.
    wtype = lib.TYPE_Q4_K
    w = dev(synth.weight(wtype, n, k, seed=46, stream=4))
    x = dev(synth.activation(m, k, seed=46))
    wide = ops.mmq_forward(wtype, w, x, n)
    knobs.set("LK_MMQ_I8")
    int8 = ops.mmq_forward(wtype, w, x, n)
    knobs.clear("LK_MMQ_I8")
    q = ops.quantize_q8_1_rows(x)
    rows = torch.cat([ops.mmvq(wtype, w, q[i:i + 8], k, n) for i in range(0, m, 8)])
    scale = rows.abs().max().item()
    assert (wide - int8).abs().max().item() <= 2e-5 * scale
    assert (wide - rows).abs().max().item() <= 2e-5 * scale


@pytest.mark.parametrize("name", SERVED)
def test_exact_activation_grid_leaves_only_summation_order(name):
    # activations n * 2^-6 with one |n| = 127 per block quantize exactly
    # (the construction of src/inference/moe_cuda/imma_reference.rs:17-29)
    wtype = DT[name]
    m, k, n = 16, 1024, 96
    rng = np.random.default_rng(45)
    a = rng.integers(-127, 128, (m, k))
    a[:, ::32] = 127
    x = (a * 2.0 ** -6).astype(np.float32)
    w = synth.weight(wtype, n, k, seed=45, stream=3)
    got = ops.mmq_forward(wtype, dev(w), dev(x), n).cpu().numpy()
    ref = oracle.ob_matmul_f64(wtype, x, w, n)
    wd = np.abs(oracle.dequantize(wtype, w).reshape(n, k).astype(np.float64))
    bound = 1e-5 * (np.abs(x.astype(np.float64)) @ wd.T)
    assert (np.abs(got - ref) <= bound + 1e-9).all()


@pytest.mark.parametrize("name", SERVED)
def test_launcher_declines_what_it_cannot_tile(name):
    wtype = DT[name]
    fn = getattr(lib.load(), ops.MMQ_LAUNCHER[wtype])
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    i = ops.MMQ_DEVICE_INFO
    s = torch.cuda.current_stream().cuda_stream
    p = buf.data_ptr()
    blk = synth.BLOCK_LEN[wtype]
    # k not a multiple of 256, a row stride shorter than the row, no rows: 0 = nothing ran
    assert fn(None, p, p, p, 128, 4, 4, 128 // blk, 4, i["cc"], i["nsm"], i["smpbo"], 64, s) == 0
    assert fn(None, p, p, p, 256, 4, 4, 256 // blk - 1, 4, i["cc"], i["nsm"], i["smpbo"], 64, s) == 0
    assert fn(None, p, p, p, 256, 4, 0, 256 // blk, 4, i["cc"], i["nsm"], i["smpbo"], 64, s) == 0
    assert fn(None, None, p, p, 256, 4, 4, 256 // blk, 4, i["cc"], i["nsm"], i["smpbo"], 64, s) == 0


@pytest.mark.parametrize("name,m,k,n", [("q4_k", 512, 4096, 14336), ("q6_k", 2048, 14336, 4096)])
def test_full_benchmark_size_against_matvec_and_sampled_oracle(name, m, k, n):
    if name not in SERVED:
        pytest.skip(f"{name} tile kernel not built")
    wtype = DT[name]
    w = synth.weight(wtype, n, k, seed=0, stream=20)
    x = synth.activation(m, k, seed=0, stream=21)
    wd, xd = dev(w), dev(x)
    tiled = ops.mmq_forward(wtype, wd, xd, n)
    # 1. a sample of token rows against the mat-vec family over ALL weight rows
    rows = [0, 1, 2, 3, m // 2, m // 2 + 1, m - 2, m - 1]
    q = ops.quantize_q8_1_rows(xd[rows].contiguous())
    vec = ops.mmvq(wtype, wd, q, k, n)
    assert (tiled[rows] - vec).abs().max().item() <= 2e-5 * vec.abs().max().item()
    # 2. a sample of (token, weight row) pairs against the CPU oracle
    rng = np.random.default_rng(46)
    tok = np.sort(rng.choice(m, 12, replace=False))
    wr = np.sort(rng.choice(n, 300, replace=False))
    want = oracle.ob_matmul(wtype, x[tok], w[wr], len(wr))
    assert_close(tiled.cpu().numpy()[np.ix_(tok, wr)], want)
    # 3. size-independent property: permuting token rows permutes output rows, bit for bit
    perm = torch.randperm(m, device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    assert torch.equal(ops.mmq_forward(wtype, wd, xd[perm].contiguous(), n), tiled[perm])

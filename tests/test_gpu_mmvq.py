"""GPU parity of the decode path (Q8_1 quantizer + mat-vec) against the CPU oracle.

Bars: Q8_1 bytes and integer sub-block dots bit-exact; f32 outputs within 1e-3 relative +
1e-4 absolute of the same-codes oracle (O-B); and within the reference's own quantization
envelope 1e-3 * sum|x.w| + 1e-3 (src/tensor/quantized/tests.rs:715-724) of the served CPU path
(O-A), whose activation codes differ by design (Q8_K per 256 vs Q8_1 per 32).
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, ops, synth

pytestmark = pytest.mark.gpu

DT = {"q4_k": lib.TYPE_Q4_K, "q5_k": lib.TYPE_Q5_K, "q6_k": lib.TYPE_Q6_K, "q8_0": lib.TYPE_Q8_0}
# the 32-value nibble formats: served by lk_mmvq and the sub-dot probe only
LEGACY = {"q4_0": lib.TYPE_Q4_0, "q4_1": lib.TYPE_Q4_1, "q5_0": lib.TYPE_Q5_0, "q5_1": lib.TYPE_Q5_1,
          "iq4_nl": lib.TYPE_IQ4_NL, "mxfp4": lib.TYPE_MXFP4}
RTOL, ATOL = 1e-3, 1e-4


def dev(a: np.ndarray) -> "torch.Tensor":
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    bad = np.abs(got - want) > RTOL * np.abs(want) + ATOL
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside 1e-3 rel + 1e-4 abs; worst {np.abs(got - want).max()}"


# ---------------------------------------------------------------- quantizer
@pytest.mark.parametrize("rows,k", [(1, 4096), (3, 1000), (8, 14336), (2, 32), (1, 33), (5, 2048)])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_q8_1_quantizer_is_bit_exact(rows, k, dtype):
    x = synth.activation(rows, k, seed=31) * np.float32(2.5)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    xt = dev(x).to(tdt)
    x_seen = xt.to(torch.float32).cpu().numpy()  # what the kernel reads, widened exactly
    kp = ops.pad_to(k, 512)
    got = ops.quantize_q8_1_rows(xt).cpu().numpy()
    assert got.shape == (rows, kp // 32, 36)
    padded = np.zeros((rows, kp), np.float32)
    padded[:, :k] = x_seen
    want = oracle.quantize_q8_1(padded).reshape(rows, kp // 32, 36)
    assert np.array_equal(got, want)


def test_q8_1_quantizer_edge_values():
    x = np.zeros((4, 64), np.float32)
    x[1, 0] = 127.0
    x[1, 1:9] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5]   # exact ties at d = 1
    x[2] = 1e-30                                                  # tiny but nonzero
    x[3, 5] = -3.0e38                                             # near f32 max
    got = ops.quantize_q8_1_rows(dev(x), k_padded=64).cpu().numpy()
    want = oracle.quantize_q8_1(x).reshape(4, 2, 36)
    assert np.array_equal(got, want)
    assert got[1, 0, 4:13].view(np.int8).tolist() == [127, 1, 2, 3, -1, -2, -3, 64, -64]


def test_quantizer_rejects_what_it_cannot_take():
    x = torch.zeros((2, 64), device="cuda")
    with pytest.raises(lib.LokenError):
        ops.quantize_q8_1_rows(x, k_padded=48)      # not whole blocks
    with pytest.raises(lib.LokenError):
        ops.quantize_q8_1_rows(x, k_padded=32)      # shorter than the row


# ---------------------------------------------------------------- integer sub-block dots
@pytest.mark.parametrize("name,n,k", [("q4_k", 16, 1024), ("q4_k", 5, 768), ("q4_k", 64, 4096),
                                      ("q5_k", 16, 1024), ("q5_k", 5, 768), ("q5_k", 33, 4096),
                                      ("q6_k", 16, 1024), ("q6_k", 7, 2304), ("q8_0", 16, 1024),
                                      ("q8_0", 9, 96), ("q8_0", 4, 4096)])
def test_integer_subblock_dots_are_bit_exact(name, n, k):
    wtype = DT[name]
    w = synth.weight(wtype, n, k, seed=32, stream=1)
    x = synth.activation(1, k, seed=32)
    q = ops.quantize_q8_1_rows(dev(x))
    dots, sums = ops.mmvq_subdots(wtype, dev(w), q[0], k, n)
    want_dots, want_sums = oracle.ob_subdots(wtype, k, n, w, oracle.quantize_q8_1(x))
    assert np.array_equal(dots.cpu().numpy(), want_dots)
    assert np.array_equal(sums.cpu().numpy(), want_sums)


def test_q4k_extreme_subdot_on_gpu():
    w = np.zeros((1, 1, 144), np.uint8)
    w[..., 16:] = 0xFF
    x = np.full((1, 256), 127.0, np.float32)
    dots, sums = ops.mmvq_subdots(lib.TYPE_Q4_K, dev(w), ops.quantize_q8_1_rows(dev(x))[0], 256, 1)
    assert dots.cpu().tolist() == [[60960] * 8] and sums.cpu().tolist() == [127 * 32] * 8


@pytest.mark.parametrize("name", sorted(LEGACY))
@pytest.mark.parametrize("n,k", [(16, 1024), (5, 96), (3, 32), (70, 4096)])
def test_legacy_integer_block_dots_are_bit_exact(name, n, k):
    wtype = LEGACY[name]
    w = synth.weight(wtype, n, k, seed=70, stream=1)
    x = synth.activation(1, k, seed=70)
    q = ops.quantize_q8_1_rows(dev(x))
    dots, sums = ops.mmvq_subdots(wtype, dev(w), q[0], k, n)
    want_dots, want_sums = oracle.ob_subdots(wtype, k, n, w, oracle.quantize_q8_1(x))
    assert np.array_equal(dots.cpu().numpy(), want_dots)
    assert np.array_equal(sums.cpu().numpy(), want_sums)


@pytest.mark.parametrize("name", sorted(LEGACY))
@pytest.mark.parametrize("n,k", [(4096, 4096), (33, 96), (1, 32), (257, 2080), (1000, 14336)])
@pytest.mark.parametrize("batch", [1, 3, 4, 7, 8])
def test_legacy_matvec_matches_same_codes_oracle(name, n, k, batch):
    wtype = LEGACY[name]
    w = synth.weight(wtype, n, k, seed=71, stream=2)
    x = synth.activation(batch, k, seed=71)
    got = ops.mmvq(wtype, dev(w), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
    assert_close(got, oracle.ob_matmul(wtype, x, w, n))


@pytest.mark.parametrize("name", sorted(LEGACY))
def test_legacy_matvec_extremes_bias_and_half_outputs(name):
    wtype = LEGACY[name]
    n, k = 40, 256
    # every code at its maximum against every activation code at +-127
    w = synth.weight(wtype, n, k, seed=72, stream=3)
    qs_at = {"q4_0": 2, "q4_1": 4, "q5_0": 6, "q5_1": 8, "iq4_nl": 2, "mxfp4": 1}[name]
    w[:, :, qs_at - (4 if name.startswith("q5") else 0):] = 0xFF
    x = np.where(np.arange(k) % 2 == 0, 127.0, -127.0).astype(np.float32).reshape(1, k) * np.float32(0.5)
    q = ops.quantize_q8_1_rows(dev(x))
    got = ops.mmvq(wtype, dev(w), q, k, n)
    assert_close(got.cpu().numpy(), oracle.ob_matmul(wtype, x, w, n))
    bias = dev(synth.normal(72, 9, n))
    with_bias = ops.mmvq(wtype, dev(w), q, k, n, bias=bias)
    assert torch.equal(with_bias, got + bias)
    for t in (torch.float16, torch.bfloat16):
        assert torch.equal(ops.mmvq(wtype, dev(w), q, k, n, out_dtype=t), got.to(t))


@pytest.mark.parametrize("name", sorted(LEGACY))
def test_legacy_matvec_within_the_reference_envelope(name):
    wtype = LEGACY[name]
    n, k = 256, 4096
    w = synth.weight(wtype, n, k, seed=73, stream=4)
    x = synth.activation(2, k, seed=73)
    got = ops.mmvq(wtype, dev(w), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
    wd = oracle.dequantize(wtype, w).reshape(n, k).astype(np.float64)
    truth = x.astype(np.float64) @ wd.T
    envelope = 1e-3 * (np.abs(x.astype(np.float64)) @ np.abs(wd).T) + 1e-3
    assert (np.abs(got - truth) <= envelope).all()
    assert (np.abs(oracle.oa_matmul(wtype, x, w, n) - truth) <= envelope).all()


LOWBIT = {"q2_k": lib.TYPE_Q2_K, "q3_k": lib.TYPE_Q3_K, "iq4_xs": lib.TYPE_IQ4_XS,
          # the codebook expert formats: runs of 32 under a scale per half (two integers per run)
          "iq2_xxs": lib.TYPE_IQ2_XXS, "iq3_xxs": lib.TYPE_IQ3_XXS, "iq3_s": lib.TYPE_IQ3_S, "iq2_s": lib.TYPE_IQ2_S,
          "q2_0": lib.TYPE_Q2_0}


@pytest.mark.parametrize("name", sorted(LOWBIT))
@pytest.mark.parametrize("n,k", [(16, 1024), (5, 768), (3, 256), (40, 4096)])
def test_two_bit_integer_subblock_dots_are_bit_exact(name, n, k):
    wtype = LOWBIT[name]
    w = synth.weight(wtype, n, k, seed=74, stream=1)
    x = synth.activation(1, k, seed=74)
    q = ops.quantize_q8_1_rows(dev(x))
    dots, sums = ops.mmvq_subdots(wtype, dev(w), q[0], k, n)
    want_dots, want_sums = oracle.ob_subdots(wtype, k, n, w, oracle.quantize_q8_1(x))
    assert np.array_equal(dots.cpu().numpy(), want_dots)
    assert np.array_equal(sums.cpu().numpy(), want_sums)


@pytest.mark.parametrize("name", sorted(LOWBIT))
@pytest.mark.parametrize("n,k", [(4096, 4096), (33, 768), (1, 256), (257, 2048), (500, 14336)])
@pytest.mark.parametrize("batch", [1, 3, 4, 8])
def test_two_bit_matvec_matches_same_codes_oracle(name, n, k, batch):
    wtype = LOWBIT[name]
    w = synth.weight(wtype, n, k, seed=75, stream=2)
    x = synth.activation(batch, k, seed=75)
    got = ops.mmvq(wtype, dev(w), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
    assert_close(got, oracle.ob_matmul(wtype, x, w, n))


@pytest.mark.parametrize("name", sorted(LOWBIT))
def test_two_bit_matvec_within_the_reference_envelope_and_outputs(name):
    wtype = LOWBIT[name]
    n, k = 256, 4096
    w = synth.weight(wtype, n, k, seed=76, stream=4)
    x = synth.activation(2, k, seed=76)
    q = ops.quantize_q8_1_rows(dev(x))
    got_t = ops.mmvq(wtype, dev(w), q, k, n)
    got = got_t.cpu().numpy()
    wd = oracle.dequantize(wtype, w).reshape(n, k).astype(np.float64)
    truth = x.astype(np.float64) @ wd.T
    envelope = 1e-3 * (np.abs(x.astype(np.float64)) @ np.abs(wd).T) + 1e-3
    assert (np.abs(got - truth) <= envelope).all()
    assert (np.abs(oracle.oa_matmul(wtype, x, w, n) - truth) <= envelope).all()
    bias = dev(synth.normal(76, 9, n))
    assert torch.equal(ops.mmvq(wtype, dev(w), q, k, n, bias=bias), got_t + bias)
    assert torch.equal(ops.mmvq(wtype, dev(w), q, k, n, out_dtype=torch.bfloat16), got_t.to(torch.bfloat16))


# ---------------------------------------------------------------- f32 outputs
SHAPES = [
    ("q4_k", 4096, 4096), ("q4_k", 1024, 4096), ("q4_k", 33, 768), ("q4_k", 1, 256), ("q4_k", 257, 2048),
    ("q5_k", 4096, 4096), ("q5_k", 33, 768), ("q5_k", 1, 256), ("q5_k", 257, 2048), ("q5_k", 130, 14336),
    ("q6_k", 4096, 2048), ("q6_k", 19, 2304), ("q6_k", 1, 256), ("q6_k", 130, 14336),
    ("q8_0", 1000, 4096), ("q8_0", 3, 32), ("q8_0", 65, 1056),
]


@pytest.mark.parametrize("name,n,k", SHAPES)
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 5, 8])
def test_matvec_matches_same_codes_oracle(name, n, k, batch):
    wtype = DT[name]
    w = synth.weight(wtype, n, k, seed=33, stream=2)
    x = synth.activation(batch, k, seed=33)
    q = ops.quantize_q8_1_rows(dev(x))
    got = ops.mmvq(wtype, dev(w), q, k, n).cpu().numpy()
    want = oracle.ob_matmul(wtype, x, w, n)
    assert_close(got, want)


@pytest.mark.parametrize("name", sorted(DT))
def test_matvec_within_reference_envelope_of_served_cpu_path(name):
    wtype = DT[name]
    n, k = 512, 4096
    w = synth.weight(wtype, n, k, seed=34, stream=3)
    x = synth.activation(4, k, seed=34)
    got = ops.mmvq(wtype, dev(w), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
    served = oracle.oa_matmul(wtype, x, w, n)
    # The reference's bound on a quantized product is against the f64 product of the unquantized
    # activation with the blocks' own values (src/tensor/quantized/tests.rs:707-731): what remains
    # is one 8-bit activation step per term. The served CPU path (Q8_K / Q8_0 codes) and this one
    # (Q8_1 codes) each sit inside it, with independent activation noise, so twice apart at most.
    wd = oracle.dequantize(wtype, w).reshape(n, k).astype(np.float64)
    truth = x.astype(np.float64) @ wd.T
    envelope = 1e-3 * (np.abs(x.astype(np.float64)) @ np.abs(wd).T) + 1e-3
    assert (np.abs(got - truth) <= envelope).all()
    assert (np.abs(served - truth) <= envelope).all()
    assert (np.abs(got - served) <= 2 * envelope).all()


@pytest.mark.parametrize("name", sorted(DT))
def test_rows_do_not_depend_on_batch(name):
    # decode order: a row of a batched launch carries the bits of its own batch-1 launch
    wtype = DT[name]
    n, k = 300, 2048
    w = dev(synth.weight(wtype, n, k, seed=35, stream=4))
    q = ops.quantize_q8_1_rows(dev(synth.activation(6, k, seed=35)))
    full = ops.mmvq(wtype, w, q, k, n, decode_order=True)
    for j in range(6):
        one = ops.mmvq(wtype, w, q[j:j + 1], k, n)
        assert torch.equal(one[0], full[j])


@pytest.mark.parametrize("out", ["f16", "bf16"])
def test_bias_and_narrow_outputs(out):
    wtype, n, k = lib.TYPE_Q4_K, 200, 1024
    w = synth.weight(wtype, n, k, seed=36, stream=5)
    x = synth.activation(2, k, seed=36)
    bias = synth.activation(1, n, seed=36, stream=9)[0]
    q = ops.quantize_q8_1_rows(dev(x))
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[out]
    f32 = ops.mmvq(wtype, dev(w), q, k, n, bias=dev(bias))
    want = oracle.ob_matmul(wtype, x, w, n) + bias[None, :]
    assert_close(f32.cpu().numpy(), want)
    narrow = ops.mmvq(wtype, dev(w), q, k, n, out_dtype=tdt, bias=dev(bias))
    assert torch.equal(narrow, f32.to(tdt))


def test_strided_destination_and_activation():
    # dst rows further apart than n, activation rows further apart than k/32
    wtype, n, k = lib.TYPE_Q6_K, 40, 512
    w = synth.weight(wtype, n, k, seed=37, stream=6)
    x = synth.activation(3, k, seed=37)
    q = ops.quantize_q8_1_rows(dev(x), k_padded=1024)
    out = torch.full((3, 64), 7.0, device="cuda")
    wd = dev(w)
    lib.check("lk_mmvq", lib.load().lk_mmvq(wtype, wd.data_ptr(), q.data_ptr(), out.data_ptr(),
                                            lib.TYPE_F32, k, n, 3, 1024 // 32, 64, None, 0,
                                            torch.cuda.current_stream().cuda_stream))
    got = out.cpu().numpy()
    assert_close(got[:, :n], oracle.ob_matmul(wtype, x, w, n))
    assert (got[:, n:] == 7.0).all()


# ---------------------------------------------------------------- full benchmark sizes
@pytest.mark.parametrize("name,n,k", [("q4_k", 14336, 4096), ("q6_k", 4096, 14336), ("q8_0", 128256, 4096)])
def test_full_size_matvec_against_oracle(name, n, k):
    wtype = DT[name]
    w = synth.weight(wtype, n, k, seed=0, stream=10)
    x = synth.activation(1, k, seed=0)
    got = ops.mmvq(wtype, dev(w), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
    assert_close(got, oracle.ob_matmul(wtype, x, w, n))
    # size-independent property: the product is linear in the block scale d, so doubling every
    # d (exact in f16) doubles every output bit for bit
    w2 = w.copy()
    off = {"q4_k": 0, "q6_k": 208, "q8_0": 0}[name]
    d = w2[:, :, off:off + 2].copy().view(np.float16)
    w2[:, :, off:off + 2] = (d * np.float16(2)).view(np.uint8)
    if name == "q4_k":
        dm = w2[:, :, 2:4].copy().view(np.float16)
        w2[:, :, 2:4] = (dm * np.float16(2)).view(np.uint8)
    got2 = ops.mmvq(wtype, dev(w2), ops.quantize_q8_1_rows(dev(x)), k, n).cpu().numpy()
    assert np.array_equal(got2, 2 * got)


# ---------------------------------------------------------------- fused neighbours
@pytest.mark.parametrize("name", sorted(DT))
@pytest.mark.parametrize("batch", [1, 3])
def test_multi_launch_rows_carry_the_bits_of_their_own_launch(name, batch):
    wtype = DT[name]
    k, ns = 2048, [512, 128, 130]
    ws = [dev(synth.weight(wtype, n, k, seed=38, stream=10 + i)) for i, n in enumerate(ns)]
    q = ops.quantize_q8_1_rows(dev(synth.activation(batch, k, seed=38)))
    outs = ops.mmvq_multi(wtype, ws, q, k, ns)
    for w, n, o in zip(ws, ns, outs):
        assert torch.equal(o, ops.mmvq(wtype, w, q, k, n))


@pytest.mark.parametrize("name", sorted(DT))
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_gate_up_pair_with_activation_in_the_store(name, act):
    wtype = DT[name]
    k, n = 1024, 300
    g = synth.weight(wtype, n, k, seed=39, stream=1)
    u = synth.weight(wtype, n, k, seed=39, stream=2)
    x = synth.activation(2, k, seed=39) * np.float32(20.0)
    q = ops.quantize_q8_1_rows(dev(x))
    got = ops.mmvq_pair_act(wtype, dev(g), dev(u), q, k, n, act=act).cpu().numpy()
    gg = oracle.ob_matmul(wtype, x, g, n).astype(np.float64)
    uu = oracle.ob_matmul(wtype, x, u, n).astype(np.float64)
    if act == "silu":
        want = gg / (1.0 + np.exp(-gg)) * uu
    else:
        want = 0.5 * gg * (1.0 + np.tanh(0.7978845608028654 * gg * (1.0 + 0.044715 * gg * gg))) * uu
    # act(g)*u inherits the relative error of g and u: bound against the row scale
    assert (np.abs(got - want) <= 2e-3 * np.abs(want) + 1e-4 * np.abs(want).max()).all()
    # and it is exactly the two single launches combined the same way
    gs = ops.mmvq(wtype, dev(g), q, k, n)
    us = ops.mmvq(wtype, dev(u), q, k, n)
    if act == "silu":
        torch.testing.assert_close(torch.from_numpy(got).cuda(), gs / (1 + torch.exp(-gs)) * us, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("name", sorted(DT))
def test_grouped_launch_each_weight_over_its_own_row(name):
    wtype = DT[name]
    groups, k, n = 5, 1024, 96
    ws = [dev(synth.weight(wtype, n, k, seed=40, stream=20 + g)) for g in range(groups)]
    table = torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device="cuda")
    q = ops.quantize_q8_1_rows(dev(synth.activation(groups, k, seed=40)))   # k is a multiple of 512
    got = ops.mmvq_grouped(wtype, table, q, k, n)
    for g in range(groups):
        assert torch.equal(got[g], ops.mmvq(wtype, ws[g], q[g:g + 1], k, n)[0])


@pytest.mark.parametrize("name,k", [("q4_k", 4096), ("q4_k", 768), ("q5_k", 4096), ("q5_k", 768), ("q6_k", 2304), ("q8_0", 1056), ("q8_0", 4096)])
@pytest.mark.parametrize("batch", [1, 4])
def test_quantize_in_kernel_path_carries_the_bits_of_the_two_launch_path(name, k, batch):
    wtype = DT[name]
    ns = [300, 64]
    ws = [dev(synth.weight(wtype, n, k, seed=62, stream=30 + i)) for i, n in enumerate(ns)]
    x = dev(synth.activation(batch, k, seed=62) * np.float32(3.0))
    fused = ops.mmvq_fused(wtype, ws, x, ns)
    q = ops.quantize_q8_1_rows(x)
    for w, n, o in zip(ws, ns, fused):
        assert torch.equal(o, ops.mmvq(wtype, w, q, k, n))


# ---------------------------------------------------------------- gate/up pair handing on Q8_1
@pytest.mark.parametrize("name,n,k,b,act", [("q4_k", 64, 512, 1, "silu"), ("q4_k", 14336, 4096, 1, "silu"),
                                            ("q4_k", 96, 768, 3, "gelu"), ("q6_k", 128, 1024, 2, "silu"),
                                            ("q8_0", 160, 256, 4, "silu")])
def test_pair_launch_writes_the_quantizers_q8_1_of_its_own_f32_result(name, n, k, b, act):
    """The Q8_1 blocks of the pair launch are, byte for byte, what the stand-alone quantizer makes of
    the f32 result of the same pair launch; and feeding them to a mat-vec equals the two-step path."""
    wtype = DT[name]
    gate = dev(synth.weight(wtype, n, k, seed=70, stream=1))
    up = dev(synth.weight(wtype, n, k, seed=70, stream=2))
    x = dev(synth.activation(b, k, seed=70))
    q = ops.quantize_q8_1_rows(x)
    h = ops.mmvq_pair_act(wtype, gate, up, q, k, n, act=act)
    want = ops.quantize_q8_1_rows(h, k_padded=n)
    for src in (x, q):   # f32 rows quantized in the kernel, or Q8_1 rows
        got = ops.mmvq_pair_act_q8_1(wtype, gate, up, src, k, n, act=act)
        assert torch.equal(got, want)


def test_pair_q8_1_launch_declines_partial_blocks():
    gate = dev(synth.weight(lib.TYPE_Q4_K, 40, 256, seed=71))
    x = dev(synth.activation(1, 256, seed=71))
    with pytest.raises(lib.LokenError):
        ops.mmvq_pair_act_q8_1(lib.TYPE_Q4_K, gate, gate, x, 256, 40)


def test_the_reference_batch1_matrix_unit_name_is_the_q4k_matvec():
    """q4k_mmvq_imma (cuda/q4k_mmvq_imma.cu:149-175): same arguments, the mat-vec family's bits."""
    n, k = 300, 2048
    w = synth.weight(lib.TYPE_Q4_K, n, k, seed=71, stream=1)
    x = synth.activation(1, k, seed=71)
    wd = torch.from_numpy(w).cuda()
    q = ops.quantize_q8_1_rows(torch.from_numpy(x).cuda(), k_padded=k)
    out = torch.full((n,), -3.0, dtype=torch.float32, device="cuda")
    lib.load().q4k_mmvq_imma(wd.data_ptr(), q.data_ptr(), out.data_ptr(), k, n, torch.cuda.current_stream().cuda_stream)
    assert torch.equal(out, ops.mmvq(lib.TYPE_Q4_K, wd, q, k, n)[0])
    want = oracle.ob_matmul(lib.TYPE_Q4_K, x, w, n)[0]
    assert (np.abs(out.cpu().numpy() - want) <= 1e-3 * np.abs(want) + 1e-4).all()


@pytest.mark.parametrize("name,n,k,rows", [("q4_k", 33, 1024, 3), ("q4_k", 5, 256, 1), ("q4_k", 64, 4096, 2), ("q4_k", 7, 17408, 1),
                                           ("q6_k", 33, 1024, 3), ("q6_k", 5, 256, 1), ("q6_k", 40, 14336, 2), ("q6_k", 7, 17408, 1)])
def test_exact_mode_carries_the_bits_of_the_cpu_exact_fold(name, n, k, rows):
    """lk_mmvq_exact over Q8_K rows quantized on the host against dot_exact of the CPU statement (the reference's
    cross-device contract, blocks.rs:80-96): bit for bit, rows of more than 64 super-blocks included."""
    wtype = {"q4_k": lib.TYPE_Q4_K, "q6_k": lib.TYPE_Q6_K}[name]
    w = synth.weight(wtype, n, k, seed=80, stream=1)
    x = synth.activation(rows, k, seed=80) * np.float32(9.0)
    x[0, :256] = 0.0   # a super-block of zeros: d8 = 0
    want = oracle.oa_matmul(wtype, x, w, n, exact=True)
    q8k = np.stack([oracle.quantize_q8_k(x[r]).reshape(-1, 292) for r in range(rows)])
    got = ops.mmvq_exact(wtype, dev(w), dev(q8k), n).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_exact_mode_refuses_other_formats():
    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    out = torch.zeros(4, device="cuda")
    rc = lib.load().lk_mmvq_exact(lib.TYPE_Q8_0, buf.data_ptr(), buf.data_ptr(), out.data_ptr(), 256, 4, 1,
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == lib.LK_ERR_TYPE


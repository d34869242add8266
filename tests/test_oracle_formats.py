"""Pins the oracle's block layouts, f16 conversion and dequantizers against ggml's own bytes.

Same judge as the reference's oracle_parity test (src/tensor/oracle_parity.rs:122-212): the
QUANT bytes ggml wrote must decode, bit for bit, to the DEQUANT values ggml computed.
"""
import numpy as np
import pytest

import oracle

TYPES = {"q2_K": oracle.Q2_K, "q3_K": oracle.Q3_K, "mxfp4": oracle.MXFP4, "q4_0": oracle.Q4_0, "q4_1": oracle.Q4_1, "q5_0": oracle.Q5_0, "q5_1": oracle.Q5_1, "q4_K": oracle.Q4_K, "q5_K": oracle.Q5_K, "q6_K": oracle.Q6_K, "q8_0": oracle.Q8_0, "q8_K": oracle.Q8_K}


@pytest.mark.parametrize("name", sorted(TYPES))
def test_dequantize_matches_ggml_bits(ggml_vectors, name):
    rec = ggml_vectors[name]
    assert rec["block_bytes"] == oracle.BLOCK_BYTES[TYPES[name]]
    assert rec["block_elems"] == oracle.BLOCK_LEN[TYPES[name]]
    got = oracle.dequantize(TYPES[name], rec["quant"])
    assert got.view(np.uint32).tolist() == rec["dequant"].view(np.uint32).tolist()


@pytest.mark.parametrize("name,dtype", [("q2_k", oracle.Q2_K), ("q3_k", oracle.Q3_K), ("iq4_nl", oracle.IQ4_NL), ("iq4_xs", oracle.IQ4_XS), ("mxfp4", oracle.MXFP4), ("q4_0", oracle.Q4_0), ("q4_1", oracle.Q4_1), ("q5_0", oracle.Q5_0), ("q5_1", oracle.Q5_1),
                                        ("q4_k", oracle.Q4_K), ("q5_k", oracle.Q5_K), ("q6_k", oracle.Q6_K), ("q8_0", oracle.Q8_0)])
def test_ggml_written_blocks_decode_to_ggml_rows(ggml_encode, name, dtype):
    f = ggml_encode["formats"][name]
    cols, read = ggml_encode["cols"], ggml_encode["read"]
    per_row = cols // oracle.BLOCK_LEN[dtype] * oracle.BLOCK_BYTES[dtype]
    assert f["blocks"].size == ggml_encode["rows"] * per_row
    got = oracle.dequantize(dtype, f["blocks"][: read * per_row])
    assert got.view(np.uint32).tolist() == f["expected"].view(np.uint32).tolist()
    # and the decoded rows are a quantization of x, not of something else
    x = ggml_encode["x"][: read * cols]
    # (MXFP4's sixteen levels step by up to a third of a value)
    assert np.abs(got - x).max() <= {"mxfp4": 0.2, "q2_k": 0.4, "q3_k": 0.2}.get(name, 0.1) * np.abs(x).max()


def test_f16_round_trip_is_exhaustively_consistent():
    # every finite half survives f16 -> f32 -> f16; numpy's IEEE conversion is the second witness
    halves = np.arange(0, 1 << 16, dtype=np.uint16)
    as_f32 = halves.view(np.float16).astype(np.float32)
    for h in list(range(0, 1 << 16, 7)) + [0x0001, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0x8001, 0xFBFF]:
        f = oracle.f16_to_f32(h)
        if np.isnan(as_f32[h]):
            assert np.isnan(f)
            continue
        assert np.float32(f).view(np.uint32) == as_f32[h].view(np.uint32), hex(h)
        assert oracle.f32_to_f16(f) == h, hex(h)


def test_f32_to_f16_rounds_to_nearest_even_like_numpy():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(1e-3),
        rng.standard_normal(4000).astype(np.float32) * np.float32(100.0),
        np.array([65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, 0.0, -0.0], np.float32),
        # exact ties between two halves
        (np.arange(1024, 1100, dtype=np.float32) + np.float32(0.5)) * np.float32(2.0 ** -10),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(float(v)) for v in vals], np.uint16)
    assert got.tolist() == want.tolist()


def test_scale_pack_unpack_round_trip_exhaustive_per_field():
    # every value of every one of the 16 six-bit fields, against a varied background
    rng = np.random.default_rng(2)
    for field in range(16):
        for v in range(64):
            sc = rng.integers(0, 64, 8).astype(np.uint8)
            mn = rng.integers(0, 64, 8).astype(np.uint8)
            (sc if field < 8 else mn)[field % 8] = v
            packed = oracle.pack_scales_mins(sc, mn)
            sc2, mn2 = oracle.unpack_scales_mins(packed)
            assert sc2.tolist() == sc.tolist() and mn2.tolist() == mn.tolist()


def test_scale_unpack_matches_the_second_statement_of_the_layout():
    # get_scale_min_k4 as the GPU header spells it (cuda/moe/gguf.cuh:271-285): an independent
    # formula over the same 12 bytes.
    rng = np.random.default_rng(3)
    for _ in range(500):
        p = rng.integers(0, 256, 12).astype(np.uint8)
        sc, mn = oracle.unpack_scales_mins(p)
        for j in range(8):
            if j < 4:
                d, m = p[j] & 63, p[j + 4] & 63
            else:
                d = (p[j + 4] & 0xF) | ((p[j - 4] >> 6) << 4)
                m = (p[j + 4] >> 4) | ((p[j] >> 6) << 4)
            assert (sc[j], mn[j]) == (d, m)


def test_synth_packing_agrees_with_oracle_packing():
    from loken_amd import synth
    rng = np.random.default_rng(4)
    sc = rng.integers(0, 64, (50, 8))
    mn = rng.integers(0, 64, (50, 8))
    packed = synth.pack_scales_mins(sc, mn)
    for i in range(50):
        assert packed[i].tolist() == oracle.pack_scales_mins(sc[i], mn[i]).tolist()

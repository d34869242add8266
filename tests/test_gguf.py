"""GGUF container reader (``lkh_gguf_*``) on the host: header, metadata, tensor directory, payload
offsets, header facts, malformed files. The cases follow the reference's own reader tests
(src/tensor/quantized/gguf_file.rs:1016-1108) and its layout rules (:135-204, :868-901); the first
test assembles a file byte by byte so the writer used elsewhere is itself checked."""
import struct

import numpy as np
import pytest

from loken_amd import gguf, lib, synth


def s(text):
    raw = text.encode()
    return struct.pack("<Q", len(raw)) + raw


def test_a_file_assembled_by_hand_is_read_field_by_field(tmp_path):
    payload_a = bytes(range(144)) * 2            # 2 Q4_K super-blocks: a [2, 256] tensor
    payload_b = bytes(range(34)) * 3             # 3 Q8_0 blocks: a [3, 32] tensor
    head = b"GGUF" + struct.pack("<IQQ", 3, 2, 4)
    head += s("general.architecture") + struct.pack("<I", 8) + s("llama")
    head += s("llama.block_count") + struct.pack("<II", 4, 32)
    head += s("llama.rope.freq_base") + struct.pack("<If", 6, 10000.0)
    head += s("tokenizer.ggml.scores") + struct.pack("<IIQ", 9, 6, 3) + struct.pack("<3f", 0.5, -1.0, 2.0)
    # dimensions are stored innermost first: a row-major [2, 256] is written 256, 2
    head += s("a.weight") + struct.pack("<IQQIQ", 2, 256, 2, 12, 0)
    head += s("b.weight") + struct.pack("<IQQIQ", 2, 32, 3, 8, 288)
    pad = -len(head) % 32
    image = head + b"\0" * pad + payload_a + payload_b
    path = tmp_path / "hand.gguf"
    path.write_bytes(image)

    for g in (gguf.GgufFile(path=path), gguf.GgufFile(data=image)):
        assert (g.version, g.alignment, g.tensor_count, g.kv_count) == (3, 32, 2, 4)
        assert g.data_offset == len(head) + pad and g.data_offset % 32 == 0
        assert g.keys() == ["general.architecture", "llama.block_count", "llama.rope.freq_base", "tokenizer.ggml.scores"]
        assert g.get("general.architecture") == "llama"
        assert g.get("llama.block_count") == 32 and g.kind("llama.block_count") == gguf.U32
        assert g.get("llama.rope.freq_base") == 10000.0
        assert g.get("tokenizer.ggml.scores") == [0.5, -1.0, 2.0]
        assert g.kind("tokenizer.ggml.scores") == (gguf.ARRAY, gguf.F32)
        assert g.get("absent.key", "dflt") == "dflt"
        a, b = g.tensor("a.weight"), g.tensor("b.weight")
        assert (a.dims, a.dtype, a.offset, a.nbytes) == ((2, 256), 12, 0, 288)
        assert (b.dims, b.dtype, b.offset, b.nbytes) == ((3, 32), 8, 288, 102)
        assert g.tensor_bytes("a.weight") == payload_a and g.tensor_bytes(1) == payload_b
        with pytest.raises(gguf.GgufError):
            g.tensor("c.weight")
        g.close()

    # the writer the other tests use states the same layout
    same = gguf.write_bytes(
        [("general.architecture", gguf.STRING, "llama"), ("llama.block_count", gguf.U32, 32),
         ("llama.rope.freq_base", gguf.F32, 10000.0), ("tokenizer.ggml.scores", gguf.ARRAY, (gguf.F32, [0.5, -1.0, 2.0]))],
        [("a.weight", (2, 256), 12, payload_a), ("b.weight", (3, 32), 8, payload_b)])
    assert same[:len(image)] == image and set(same[len(image):]) <= {0}


@pytest.mark.parametrize("version", [2, 3])
@pytest.mark.parametrize("alignment", [None, 64, 4096])
def test_the_payload_starts_at_the_first_multiple_of_the_alignment(version, alignment):
    w0 = synth.weight(lib.TYPE_Q6_K, 3, 512, seed=5).tobytes()
    w1 = synth.weight(lib.TYPE_Q4_K, 1, 256, seed=6).tobytes()
    image = gguf.write_bytes([("general.name", gguf.STRING, "x" * 7)],
                             [("blk.0.ffn_down.weight", (3, 512), 14, w0), ("blk.0.attn_q.weight", (1, 256), 12, w1)],
                             version=version, alignment=alignment)
    g = gguf.GgufFile(data=image)
    align = alignment or 32
    assert g.version == version and g.alignment == align and g.data_offset % align == 0
    t0, t1 = g.tensors()
    assert t0.offset == 0 and t1.offset % align == 0 and t1.offset >= len(w0)
    assert g.tensor_bytes(0) == w0 and g.tensor_bytes(1) == w1


def test_every_metadata_kind_and_the_reference_conversions():
    kvs = [("u8", gguf.U8, 200), ("i8", gguf.I8, -100), ("u16", gguf.U16, 60000), ("i16", gguf.I16, -30000),
           ("u32", gguf.U32, 4000000000), ("i32", gguf.I32, -2000000000), ("f32", gguf.F32, 0.25),
           ("yes", gguf.BOOL, 1), ("no", gguf.BOOL, 0), ("str", gguf.STRING, "héllo"),
           ("u64", gguf.U64, 2 ** 63 + 5), ("i64", gguf.I64, -2 ** 62), ("f64", gguf.F64, 1e300),
           ("strs", gguf.ARRAY, (gguf.STRING, ["a", "", "ccc"])), ("ints", gguf.ARRAY, (gguf.I32, [-1, 0, 7])),
           ("none", gguf.ARRAY, (gguf.U8, [])), ("small_u64", gguf.U64, 9)]
    g = gguf.GgufFile(data=gguf.write_bytes(kvs, []))
    for key, kind, want in kvs:
        if kind == gguf.ARRAY:
            assert g.get(key) == want[1] and g.kind(key) == (gguf.ARRAY, want[0])
        elif kind == gguf.BOOL:
            assert g.get(key) is bool(want)
        else:
            assert g.get(key) == want and g.kind(key) == kind
    # whole-number kinds convert when the value fits the target; floats, strings and bools never do
    assert g.as_u64("u8") == 200 and g.as_u64("i64") is None and g.as_u64("i8") is None and g.as_u64("u64") == 2 ** 63 + 5
    assert g.as_i64("i32") == -2000000000 and g.as_i64("u32") == 4000000000
    assert g.as_u64("f32") is None and g.as_u64("str") is None and g.as_u64("yes") is None
    assert g.as_i64("u64") is None and g.as_i64("small_u64") is None   # a U64 is refused whatever it holds
    assert g.tensor_count == 0 and g.facts().parameter_count is None


def test_a_declared_count_ends_the_walk_at_the_vocabulary():
    g = gguf.GgufFile(data=gguf.write_bytes(
        [("general.architecture", gguf.STRING, "llama"), ("general.tags", gguf.ARRAY, (gguf.STRING, ["chat", "code"])),
         ("general.file_type", gguf.U32, 15), ("general.parameter_count", gguf.U32, 7),
         ("tokenizer.ggml.tokens", gguf.ARRAY, (gguf.STRING, ["a", "b", "c"])), ("split.count", gguf.U32, 4)], []))
    f = g.facts()
    assert (f.architecture, f.file_type, f.parameter_count) == ("llama", 15, 7)
    assert f.split_parts is None     # behind the vocabulary: the walk had already stopped


def test_a_missing_count_is_summed_from_the_directory():
    g = gguf.GgufFile(data=gguf.write_bytes(
        [("general.architecture", gguf.STRING, "qwen3moe"), ("tokenizer.ggml.tokens", gguf.ARRAY, (gguf.STRING, ["a", "b"]))],
        [("token_embd.weight", (1000, 64), 0, b""), ("blk.0.attn_q.weight", (64, 64), 0, b""),
         ("blk.0.ffn_up_exps.weight", (8, 64, 64), 0, b"")]))
    f = g.facts()
    assert f.architecture == "qwen3moe" and f.parameter_count == 1000 * 64 + 64 * 64 + 8 * 64 * 64
    # the directory names more bytes than the image holds: data is refused, the header still reads
    with pytest.raises(gguf.GgufError):
        g.tensor_bytes("token_embd.weight")


def test_a_split_part_reports_the_set_it_belongs_to():
    g = gguf.GgufFile(data=gguf.write_bytes(
        [("general.architecture", gguf.STRING, "qwen3moe"), ("split.count", gguf.U32, 2), ("split.no", gguf.U32, 0)],
        [("blk.0.attn_q.weight", (64, 64), 0, b"")]))
    f = g.facts()
    assert f.split_parts == 2 and f.parameter_count == 64 * 64


def test_a_pooling_type_under_the_architecture_is_read():
    tokens = ("tokenizer.ggml.tokens", gguf.ARRAY, (gguf.STRING, ["a"]))
    g = gguf.GgufFile(data=gguf.write_bytes(
        [("general.architecture", gguf.STRING, "nomic-bert"), ("nomic-bert.pooling_type", gguf.U32, 1), tokens], []))
    assert g.facts().pools
    g = gguf.GgufFile(data=gguf.write_bytes(
        [("general.architecture", gguf.STRING, "llama"), ("bert.pooling_type", gguf.U32, 1)], []))
    assert not g.facts().pools
    g = gguf.GgufFile(data=gguf.write_bytes(
        [("general.architecture", gguf.STRING, "qwen3"), ("general.parameter_count", gguf.U32, 600_000_000), tokens], []))
    assert g.facts().parameter_count == 600_000_000 and not g.facts().pools


def test_malformed_files_are_refused_with_a_message(tmp_path):
    good = gguf.write_bytes([("general.architecture", gguf.STRING, "llama")],
                            [("w", (1, 256), 12, synth.weight(lib.TYPE_Q4_K, 1, 256).tobytes())])
    with pytest.raises(gguf.GgufError, match="not a GGUF file"):
        gguf.GgufFile(data=b"GGML" + good[4:])
    for version in (1, 4):
        with pytest.raises(gguf.GgufError, match=f"unsupported GGUF version {version}"):
            gguf.GgufFile(data=good[:4] + struct.pack("<I", version) + good[8:])
    # cut anywhere inside the header: a read error, never a read past the image
    header_len = gguf.GgufFile(data=good).data_offset - 20
    for cut in list(range(0, 40)) + list(range(40, header_len, 7)):
        with pytest.raises(gguf.GgufError):
            gguf.GgufFile(data=good[:cut] or b"\0")
    # a string length that runs past the file
    bad = bytearray(good)
    bad[24:32] = struct.pack("<Q", 2 ** 40)
    with pytest.raises(gguf.GgufError, match="failed to fill"):
        gguf.GgufFile(data=bytes(bad))
    with pytest.raises(gguf.GgufError, match="unknown value type"):
        gguf.GgufFile(data=gguf.write_bytes([], [])[:16] + struct.pack("<Q", 1) + s("k") + struct.pack("<I", 13))
    with pytest.raises(gguf.GgufError, match="unsupported ggml dtype id 99"):
        gguf.GgufFile(data=gguf.write_bytes([], [("w", (4,), 99, b"")]))
    with pytest.raises(gguf.GgufError, match="alignment is zero"):
        gguf.GgufFile(data=gguf.write_bytes([("general.alignment", gguf.U32, 0)], []))
    with pytest.raises(gguf.GgufError, match="open"):
        gguf.GgufFile(path=tmp_path / "absent.gguf")
    (tmp_path / "empty.gguf").write_bytes(b"")
    with pytest.raises(gguf.GgufError):
        gguf.GgufFile(path=tmp_path / "empty.gguf")


def test_tensor_bytes_follow_the_block_table():
    # id -> (values, bytes) per block, as the kernels' own constants state them for the served formats
    assert gguf.BLOCKS[lib.TYPE_Q4_K] == (256, 144) and gguf.BLOCKS[lib.TYPE_Q6_K] == (256, 210)
    assert gguf.BLOCKS[lib.TYPE_Q8_0] == (32, 34)
    tensors = [(f"t{dt}", (4, 512), dt, b"") for dt in sorted(gguf.BLOCKS)]
    g = gguf.GgufFile(data=gguf.write_bytes([], tensors))
    for t in g.tensors():
        values, nbytes = gguf.BLOCKS[t.dtype]
        assert t.nbytes == 4 * 512 // values * nbytes
    assert synth.weight_bytes(lib.TYPE_Q6_K, 4, 512) == g.tensor("t14").nbytes


def test_a_repeated_name_finds_the_later_entry_and_keeps_file_order():
    g = gguf.GgufFile(data=gguf.write_bytes([("k", gguf.U32, 1), ("k", gguf.U32, 2)], []))
    assert g.keys() == ["k", "k"] and g.get("k") == 2


def test_header_arithmetic_from_the_file_is_not_trusted():
    q4k = synth.weight(lib.TYPE_Q4_K, 1, 256).tobytes()
    # dimensions that are zero, negative as int64, or whose product wraps
    for dims in ((0, 256), (2 ** 63, 2), (2 ** 62, 4), (2 ** 32, 2 ** 32)):
        with pytest.raises(gguf.GgufError, match="dimension"):
            gguf.GgufFile(data=gguf.write_bytes([], [("w", dims, 12, q4k)]))
    with pytest.raises(gguf.GgufError, match="dimensions"):
        gguf.GgufFile(data=gguf.write_bytes([], [("w", (1,) * 9, 0, b"")]))
    # a row that is not whole blocks of its type
    with pytest.raises(gguf.GgufError, match="not whole blocks"):
        gguf.GgufFile(data=gguf.write_bytes([], [("w", (1, 250), 12, q4k)]))
    # an alignment that is not a power of two, or larger than the file
    with pytest.raises(gguf.GgufError, match="power of two"):
        gguf.GgufFile(data=gguf.write_bytes([("general.alignment", gguf.U32, 48)], []))
    with pytest.raises(gguf.GgufError, match="power of two"):
        gguf.GgufFile(data=_with_u64_alignment(2 ** 62))
    # a 30-byte file that claims an array of 2^60 items: refused before anything is reserved
    head = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + s("a") + struct.pack("<IIQ", 9, 4, 2 ** 60)
    with pytest.raises(gguf.GgufError, match="longer than the file"):
        gguf.GgufFile(data=head)


def _with_u64_alignment(value):
    return b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + s("general.alignment") + struct.pack("<IQ", 10, value) + b"\0" * 64

"""GGUF tensors on the card: the uploaded blob (blocks + 4096 zero bytes, the rule of
src/tensor/quantized/mod.rs:35 and kernel_matmul.rs:218-236) and a QKernelMatMul built straight from
a file (kernel_matmul.rs:213-275), checked against the oracle on the file's own bytes."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import gguf, lib, synth

pytestmark = pytest.mark.gpu

HIP_D2H = 2


def model_file(tmp_path):
    shapes = {"blk.0.attn_q.weight": (lib.TYPE_Q4_K, 192, 1024), "blk.0.ffn_down.weight": (lib.TYPE_Q6_K, 160, 768),
              "output.weight": (lib.TYPE_Q8_0, 320, 512), "blk.0.attn_v.weight": (lib.TYPE_Q5_K, 96, 1024),
              "blk.0.attn_k.weight": (lib.TYPE_Q4_0, 64, 1024), "blk.0.ffn_up.weight": (lib.TYPE_MXFP4, 128, 512)}
    blocks = {name: synth.weight(dt, n, k, seed=90, stream=i) for i, (name, (dt, n, k)) in enumerate(shapes.items())}
    norm = np.arange(1024, dtype=np.float32)
    tensors = [(name, (n, k), dt, blocks[name].tobytes()) for name, (dt, n, k) in shapes.items()]
    tensors.insert(1, ("blk.0.attn_norm.weight", (1024,), 0, norm.tobytes()))
    path = tmp_path / "tiny.gguf"
    path.write_bytes(gguf.write_bytes([("general.architecture", gguf.STRING, "llama")], tensors, alignment=64))
    return path, shapes, blocks


def test_an_uploaded_tensor_is_its_blocks_followed_by_4096_zero_bytes(tmp_path):
    path, shapes, blocks = model_file(tmp_path)
    g = gguf.GgufFile(path=path)
    torch.cuda.init()
    for name in shapes:
        want = blocks[name].tobytes()
        ptr, nbytes = g.upload(name)
        try:
            assert nbytes == len(want) + 4096
            back = torch.empty(nbytes, dtype=torch.uint8)
            # the runtime torch and the library already share (same soname: the loader returns that one)
            rc = C.CDLL("libamdhip64.so.7").hipMemcpy(C.c_void_p(back.data_ptr()), C.c_void_p(ptr), C.c_size_t(nbytes), HIP_D2H)
            assert rc == 0
            got = back.numpy().tobytes()
            assert got[:len(want)] == want and got[len(want):] == bytes(4096)
        finally:
            gguf.free_blob(ptr)


@pytest.mark.parametrize("rows", [1, 6, 96])
def test_a_linear_built_from_the_file_matches_the_oracle_on_the_files_bytes(tmp_path, rows):
    path, shapes, blocks = model_file(tmp_path)
    g = gguf.GgufFile(path=path)
    l = lib.load()
    for name, (dt, n, k) in shapes.items():
        x = synth.activation(rows, k, seed=91)
        xd = torch.from_numpy(x).cuda()
        out = torch.empty((rows, n), dtype=torch.float32, device="cuda")
        h, blob = g.linear(name)
        try:
            rc = l.lkh_qkernel_matmul_forward(h, xd.data_ptr(), lib.TYPE_F32, rows, out.data_ptr(),
                                              torch.cuda.current_stream().cuda_stream, 0)
            assert rc == 0
            torch.cuda.synchronize()
            want = oracle.ob_matmul(dt, x, np.frombuffer(g.tensor_bytes(name), dtype=np.uint8), n)
            got = out.cpu().numpy().astype(np.float64)
            assert (np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-4).all()
        finally:
            l.lkh_qkernel_matmul_free(h)
            gguf.free_blob(blob)


def test_tensors_the_card_path_does_not_serve_are_refused(tmp_path):
    path, _, _ = model_file(tmp_path)
    g = gguf.GgufFile(path=path)
    with pytest.raises(gguf.GgufError, match="2-D"):
        g.linear("blk.0.attn_norm.weight")
    with pytest.raises(gguf.GgufError, match="no tensor"):
        g.linear("blk.9.attn_q.weight")
    wide = gguf.GgufFile(data=gguf.write_bytes([], [("w", (4, 64), 0, bytes(1024))]))
    with pytest.raises(gguf.GgufError, match="not served"):
        wide.linear("w")

"""The C++ host mirror of QKernelMatMul (include/loken_host.hpp) through its C symbols: path chosen
by row count, results equal to the launchers called one by one, workspace rules."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle
from loken_amd import lib, ops, synth

pytestmark = pytest.mark.gpu

DT = {"q4_k": lib.TYPE_Q4_K, "q5_k": lib.TYPE_Q5_K, "q6_k": lib.TYPE_Q6_K, "q8_0": lib.TYPE_Q8_0,
      "q4_0": lib.TYPE_Q4_0, "q4_1": lib.TYPE_Q4_1, "q5_0": lib.TYPE_Q5_0, "q5_1": lib.TYPE_Q5_1, "iq4_nl": lib.TYPE_IQ4_NL, "mxfp4": lib.TYPE_MXFP4, "q2_k": lib.TYPE_Q2_K, "q3_k": lib.TYPE_Q3_K}
PATH = {1: "matvec-fused", 2: "matvec", 3: "rows-on-matrix-unit", 4: "tiled"}
X_TYPES = {torch.float32: lib.TYPE_F32, torch.float16: lib.TYPE_F16, torch.bfloat16: lib.TYPE_BF16}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


class Linear:
    def __init__(self, wtype, w, n, k):
        self.l = lib.load()
        self.w = w   # keeps the blob alive
        self.n, self.k = n, k
        self.h = self.l.lkh_qkernel_matmul_new(wtype, n, k, w.data_ptr(), torch.cuda.current_device())

    def __call__(self, x, decode_order=False, stream=None):
        out = torch.empty((x.shape[0], self.n), dtype=x.dtype, device=x.device)
        s = stream if stream is not None else torch.cuda.current_stream().cuda_stream
        rc = self.l.lkh_qkernel_matmul_forward(self.h, x.data_ptr(), X_TYPES[x.dtype], x.shape[0], out.data_ptr(), s,
                                               int(decode_order))
        if rc:
            raise lib.LokenError("lkh_qkernel_matmul_forward", rc)
        return out

    @property
    def path(self):
        return PATH.get(self.l.lkh_qkernel_matmul_last_path(self.h), "none")

    def close(self):
        self.l.lkh_qkernel_matmul_free(self.h)


def close(got, want, rtol=1e-3, atol=1e-4):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return bool((np.abs(got - want) <= rtol * np.abs(want) + atol).all())


@pytest.mark.parametrize("name,rows,n,expect", [
    ("q4_k", 1, 200, "matvec-fused"), ("q4_k", 2, 200, "matvec-fused"), ("q4_k", 5, 200, "matvec"),
    ("q4_k", 8, 200, "matvec"), ("q4_k", 9, 200, "rows-on-matrix-unit"), ("q4_k", 40, 200, "rows-on-matrix-unit"),
    # a handful of rows over a matrix large enough to pay for staging them in every workgroup
    ("q4_k", 2, 4000, "matvec-fused"), ("q4_k", 3, 4000, "rows-on-matrix-unit"), ("q4_k", 8, 1100, "rows-on-matrix-unit"),
    ("q5_k", 4, 2100, "rows-on-matrix-unit"), ("q5_k", 4, 2000, "matvec"),
    # above 16 rows the rows kernel keeps a matrix too small to fill the chip with tiles (n x rows up to 450 thousand)
    ("q4_k", 80, 200, "rows-on-matrix-unit"), ("q4_k", 80, 24000, "tiled"),
    ("q6_k", 1, 200, "matvec-fused"), ("q6_k", 8, 200, "matvec"), ("q6_k", 20, 200, "rows-on-matrix-unit"),
    ("q6_k", 40, 200, "rows-on-matrix-unit"), ("q6_k", 200, 24000, "tiled"),
    ("q8_0", 3, 200, "matvec"), ("q8_0", 16, 200, "matvec"), ("q8_0", 17, 200, "tiled"), ("q5_k", 1, 200, "matvec-fused"), ("q5_k", 8, 200, "matvec"),
    ("q5_k", 20, 200, "rows-on-matrix-unit"), ("q5_k", 200, 200, "rows-on-matrix-unit"), ("q5_k", 80, 24000, "tiled"), ("q5_k", 18, 24000, "rows-on-matrix-unit"),
    ("q4_0", 1, 200, "matvec"), ("q4_0", 12, 200, "matvec"), ("q5_1", 9, 200, "matvec"), ("iq4_nl", 3, 200, "matvec"),
    # four of the 32-value formats have tiles: from 16 rows, or from 9 over 48 M weights
    ("q4_0", 50, 200, "tiled"), ("q5_0", 16, 200, "tiled"), ("q5_1", 30, 12000, "tiled"), ("q4_1", 12, 12000, "matvec"),
    ("q4_0", 9, 49152, "tiled"),
    ("q4_1", 130, 300, "tiled"), ("iq4_nl", 60, 200, "matvec"), ("q3_k", 41, 200, "tiled"), ("q3_k", 17, 12000, "tiled"),
    ("q2_k", 50, 200, "tiled"),
    ("mxfp4", 17, 200, "matvec"), ("q2_k", 12, 200, "matvec"), ("q3_k", 1, 200, "matvec")])
def test_forward_takes_the_path_of_its_row_count_and_matches_the_oracle(name, rows, n, expect):
    wtype, k = DT[name], 1024
    w = synth.weight(wtype, n, k, seed=80, stream=1)
    x = synth.activation(rows, k, seed=80)
    lin = Linear(wtype, dev(w), n, k)
    try:
        got = lin(dev(x))
        assert lin.path == expect
        pick = np.arange(n) if n <= 400 else np.sort(np.random.default_rng(80).choice(n, 300, replace=False))
        assert close(got.cpu().numpy()[:, pick], oracle.ob_matmul(wtype, x, w[pick], len(pick)))
    finally:
        lin.close()


def test_decode_order_keeps_every_row_on_the_matvec_family_and_rows_independent():
    wtype, n, k = lib.TYPE_Q4_K, 300, 2048
    w = dev(synth.weight(wtype, n, k, seed=81, stream=1))
    x = dev(synth.activation(20, k, seed=81))
    lin = Linear(wtype, w, n, k)
    try:
        batch = lin(x, decode_order=True)
        assert lin.path == "matvec"
        q = ops.quantize_q8_1_rows(x)
        for r in (0, 7, 8, 19):
            assert torch.equal(batch[r:r + 1], ops.mmvq(wtype, w, q[r:r + 1], k, n))
    finally:
        lin.close()


def test_half_inputs_stay_in_their_type_on_the_matvec_family():
    wtype, n, k = lib.TYPE_Q6_K, 64, 512
    w = dev(synth.weight(wtype, n, k, seed=82, stream=1))
    lin = Linear(wtype, w, n, k)
    try:
        x = dev(synth.activation(3, k, seed=82)).to(torch.bfloat16)
        y = lin(x)
        assert y.dtype == torch.bfloat16 and lin.path == "matvec"
        want = ops.mmvq(wtype, w, ops.quantize_q8_1_rows(x), k, n, out_dtype=torch.bfloat16)
        assert torch.equal(y, want)
    finally:
        lin.close()


@pytest.mark.parametrize("half", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name,rows,n,expect", [
    ("q6_k", 50, 64, "rows-on-matrix-unit"), ("q4_k", 20, 200, "rows-on-matrix-unit"), ("q4_k", 4, 4000, "rows-on-matrix-unit"),
    ("q4_k", 130, 24000, "tiled"), ("q4_k", 300, 6000, "tiled"), ("q6_k", 200, 24000, "tiled"), ("q8_0", 40, 200, "tiled"),
    ("q5_1", 60, 200, "tiled"), ("q5_k", 90, 24000, "tiled")])
def test_half_rows_above_the_matvec_family_follow_the_oracle_and_leave_in_their_type(name, rows, n, expect, half):
    # the reference's forward serves f16 / bf16 rows at every row count and returns their type
    # (src/tensor/quantized/kernel_matmul.rs:1086-1714): the oracle is fed the values the rows hold, and
    # the result is the f32 call's result rounded once to the narrow type
    wtype, k = DT[name], 1024
    w = synth.weight(wtype, n, k, seed=83, stream=1)
    xh = dev(synth.activation(rows, k, seed=83)).to(half)
    x_seen = xh.to(torch.float32)
    lin = Linear(wtype, dev(w), n, k)
    try:
        got = lin(xh)
        assert got.dtype == half and lin.path == expect
        wide = lin(x_seen)
        assert lin.path == expect
        assert torch.equal(got, wide.to(half))
        pick = np.arange(n) if n <= 400 else np.sort(np.random.default_rng(83).choice(n, 300, replace=False))
        want = oracle.ob_matmul(wtype, x_seen.cpu().numpy(), w[pick], len(pick))
        eps = 2.0 ** -8 if half == torch.bfloat16 else 2.0 ** -11   # one rounding to the narrow type
        gotf = got.to(torch.float32).cpu().numpy()[:, pick].astype(np.float64)
        assert (np.abs(gotf - want) <= (1e-3 + eps) * np.abs(want) + 1e-4).all()
    finally:
        lin.close()


def test_workspace_grows_outside_a_capture_only_and_replays_then():
    wtype, n, k = lib.TYPE_Q4_K, 128, 1024
    w = dev(synth.weight(wtype, n, k, seed=83, stream=1))
    lin = Linear(wtype, w, n, k)
    lib.load().lkh_release_workspaces()
    try:
        x = dev(synth.activation(12, k, seed=83))
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with pytest.raises(lib.LokenError) as err:      # nothing reserved yet: refused while recording
                with torch.cuda.graph(graph, stream=side):
                    lin(x, stream=side.cuda_stream)
            assert "LK_ERR_NOMEM" in str(err.value)
        torch.cuda.synchronize()
        eager = lin(x)                                       # reserves the workspace
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        out = torch.empty((12, n), device="cuda")
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                rc = lib.load().lkh_qkernel_matmul_forward(lin.h, x.data_ptr(), lib.TYPE_F32, 12, out.data_ptr(),
                                                           side.cuda_stream, 0)
                assert rc == 0
        for _ in range(3):
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
    finally:
        lin.close()


def test_argument_errors_are_status_codes():
    l = lib.load()
    assert l.lkh_matvec_rows(lib.TYPE_Q4_K, 4096) == 8 and l.lkh_matvec_rows(lib.TYPE_Q6_K, 4096) == 8
    assert l.lkh_matvec_rows(lib.TYPE_Q8_0, 4096) == 16
    h = l.lkh_qkernel_matmul_new(99, 8, 256, 16, 0)
    assert l.lkh_qkernel_matmul_forward(h, 16, lib.TYPE_F32, 1, 16, None, 0) == lib.LK_ERR_TYPE
    l.lkh_qkernel_matmul_free(h)
    h = l.lkh_qkernel_matmul_new(lib.TYPE_Q4_K, 8, 250, 16, 0)
    assert l.lkh_qkernel_matmul_forward(h, 16, lib.TYPE_F32, 1, 16, None, 0) == lib.LK_ERR_ARG
    assert l.lkh_qkernel_matmul_forward(h, 16, lib.TYPE_F32, 0, 16, None, 0) == lib.LK_OK
    l.lkh_qkernel_matmul_free(h)


def test_rows_too_long_for_the_matrix_unit_rows_kernel_go_to_the_tiles():
    # 12 rows of 40960 values: the rows kernel's scale tables do not fit LDS; the call must end on the
    # tiled matmul with a written buffer, and the direct wrapper must raise instead of returning
    wtype, n, k, rows = lib.TYPE_Q4_K, 64, 40960, 12
    w = synth.weight(wtype, n, k, seed=84, stream=1)
    x = synth.activation(rows, k, seed=84)
    lin = Linear(wtype, dev(w), n, k)
    try:
        out = torch.full((rows, n), float("nan"), device="cuda")
        rc = lib.load().lkh_qkernel_matmul_forward(lin.h, dev(x).data_ptr(), lib.TYPE_F32, rows, out.data_ptr(),
                                                   torch.cuda.current_stream().cuda_stream, 0)
        assert rc == 0 and lin.path == "tiled"
        # 160 blocks per row summed one after the other in f32: held to the row scale, not element by
        # element (the test is about which kernel ran and that it wrote the buffer)
        want = oracle.ob_matmul(wtype, x, w, n)
        assert np.abs(out.cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max() + 1e-4
    finally:
        lin.close()
    with pytest.raises(lib.LokenError):
        ops.dense_q4k_rows(dev(w), dev(x), n)


@pytest.mark.parametrize("name,rows,n", [("q4_k", 1, 300), ("q4_k", 2, 300), ("q4_k", 7, 300), ("q6_k", 5, 260), ("q8_0", 12, 200),
                                        ("q5_k", 1, 130), ("q4_0", 6, 200), ("q3_k", 3, 200)])
@pytest.mark.parametrize("xt", [torch.float32, torch.float16])
def test_an_activation_quantized_once_serves_several_weights_with_the_bits_of_forward(name, rows, n, xt):
    # quantize_for_matvec / forward_quantized of the reference (src/tensor/quantized/kernel_matmul.rs:695-812):
    # the Q8_1 rows are made once and every weight over them returns what its own forward returns
    l = lib.load()
    wtype, k = DT[name], 1024
    lins = [Linear(wtype, dev(synth.weight(wtype, n + 8 * i, k, seed=90 + i, stream=1)), n + 8 * i, k) for i in range(2)]
    x = dev(synth.activation(rows, k, seed=90)).to(xt)
    q81 = torch.empty(l.lkh_quantized_activation_bytes(k, rows), dtype=torch.uint8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    try:
        assert l.lkh_qkernel_matmul_quantize_for_matvec(lins[0].h, x.data_ptr(), X_TYPES[xt], rows, q81.data_ptr(), s, 0) == 0
        for lin in lins:
            out = torch.empty((rows, lin.n), dtype=xt, device="cuda")
            assert l.lkh_qkernel_matmul_forward_quantized(lin.h, q81.data_ptr(), X_TYPES[xt], rows, out.data_ptr(), s, 0) == 0
            assert lin.path == "matvec"
            assert torch.equal(out, lin(x))
    finally:
        for lin in lins:
            lin.close()


def test_a_pair_of_weights_over_one_quantized_row_in_one_launch():
    # forward_quantized_pair (kernel_matmul.rs:814-876): one f32-born row, two weights of one format and k
    l = lib.load()
    k = 2048
    a = Linear(lib.TYPE_Q4_K, dev(synth.weight(lib.TYPE_Q4_K, 520, k, seed=91, stream=1)), 520, k)
    b = Linear(lib.TYPE_Q4_K, dev(synth.weight(lib.TYPE_Q4_K, 136, k, seed=92, stream=1)), 136, k)
    c = Linear(lib.TYPE_Q6_K, dev(synth.weight(lib.TYPE_Q6_K, 136, k, seed=93, stream=1)), 136, k)
    x = dev(synth.activation(1, k, seed=91))
    q81 = torch.empty(l.lkh_quantized_activation_bytes(k, 1), dtype=torch.uint8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    try:
        assert l.lkh_qkernel_matmul_quantize_for_matvec(a.h, x.data_ptr(), lib.TYPE_F32, 1, q81.data_ptr(), s, 0) == 0
        oa, ob = torch.empty((1, 520), device="cuda"), torch.empty((1, 136), device="cuda")
        assert l.lkh_qkernel_matmul_forward_quantized_pair(a.h, b.h, q81.data_ptr(), oa.data_ptr(), ob.data_ptr(), s) == 0
        assert torch.equal(oa, a(x)) and torch.equal(ob, b(x))
        # two formats do not pair: the reference's None
        assert l.lkh_qkernel_matmul_forward_quantized_pair(a.h, c.h, q81.data_ptr(), oa.data_ptr(), ob.data_ptr(), s) == lib.LK_NOT_TAKEN
    finally:
        for lin in (a, b, c):
            lin.close()


def test_rows_that_forward_serves_another_way_are_not_quantized_for_the_matvec():
    l = lib.load()
    s = torch.cuda.current_stream().cuda_stream
    k = 1024
    x = dev(synth.activation(40, k, seed=94))
    q81 = torch.empty(l.lkh_quantized_activation_bytes(k, 40), dtype=torch.uint8, device="cuda")
    out = torch.empty((40, 4000), device="cuda")
    big = Linear(lib.TYPE_Q4_K, dev(synth.weight(lib.TYPE_Q4_K, 4000, k, seed=94, stream=1)), 4000, k)
    try:
        # 40 rows go to the matrix-unit kernels, 4 rows over this matrix to the 16-row tiles
        for rows in (40, 4):
            assert l.lkh_qkernel_matmul_quantize_for_matvec(big.h, x.data_ptr(), lib.TYPE_F32, rows, q81.data_ptr(), s, 0) == lib.LK_NOT_TAKEN
            assert l.lkh_qkernel_matmul_forward_quantized(big.h, q81.data_ptr(), lib.TYPE_F32, rows, out.data_ptr(), s, 0) == lib.LK_NOT_TAKEN
        # in decode order every row count stays on the mat-vec kernels
        assert l.lkh_qkernel_matmul_quantize_for_matvec(big.h, x.data_ptr(), lib.TYPE_F32, 40, q81.data_ptr(), s, 1) == 0
        assert l.lkh_qkernel_matmul_forward_quantized(big.h, q81.data_ptr(), lib.TYPE_F32, 40, out.data_ptr(), s, 1) == 0
        assert torch.equal(out, big(x, decode_order=True))
        assert l.lkh_qkernel_matmul_quantize_for_matvec(big.h, x.data_ptr(), 77, 2, q81.data_ptr(), s, 0) == lib.LK_ERR_TYPE
        assert l.lkh_qkernel_matmul_quantize_for_matvec(big.h, None, lib.TYPE_F32, 2, q81.data_ptr(), s, 0) == lib.LK_ERR_ARG
    finally:
        big.close()


@pytest.mark.parametrize("name,rows,expect", [("q4_k", 12, "tiled"), ("q5_k", 16, "tiled"), ("q6_k", 12, "rows-on-matrix-unit"),
                                               ("q4_k", 8, "matvec")])
def test_long_rows_at_nine_to_sixteen_activation_rows(name, rows, expect):
    # rows of 8192 values: Q4_K / Q5_K leave the 16-row tiles for the tiled matmul (K cut into ranges) from nine rows
    wtype, n, k = DT[name], 2048, 8192
    w = synth.weight(wtype, n, k, seed=96, stream=1)
    x = synth.activation(rows, k, seed=96)
    lin = Linear(wtype, dev(w), n, k)
    try:
        got = lin(dev(x))
        assert lin.path == expect
        pick = np.sort(np.random.default_rng(96).choice(n, 200, replace=False))
        assert close(got.cpu().numpy()[:, pick], oracle.ob_matmul(wtype, x, w[pick], len(pick)))
    finally:
        lin.close()

"""Host layer over the C ABI for callers that hold torch device tensors.

torch is used for device memory and the current stream only; every computation goes through
``libloken_gfx950.so``. Function names follow the reference's Rust launch surface
(src/tensor/cuda/quant.rs of loken): ``quantize_q8_1_rows`` (:19-26,112-151), ``mmvq_f32``
(:173-184, 3264-3298).
"""
from __future__ import annotations

import torch

from . import lib as _lib
from .synth import BLOCK_BYTES, BLOCK_LEN

ROW_PADDING = 512

_X_TYPES = {torch.float32: _lib.TYPE_F32, torch.float16: _lib.TYPE_F16, torch.bfloat16: _lib.TYPE_BF16}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def pad_to(v: int, m: int) -> int:
    return (v + m - 1) // m * m


def quantize_q8_1_rows(x: torch.Tensor, k_padded: int | None = None) -> torch.Tensor:
    """``[rows, k]`` f32/f16/bf16 -> ``[rows, k_padded/32, 36]`` uint8 Q8_1 blocks."""
    if not x.is_cuda or x.dim() != 2 or not x.is_contiguous():
        raise ValueError("q8_1 quantize: a contiguous 2-D device tensor is required")
    rows, k = x.shape
    k_padded = pad_to(k, ROW_PADDING) if k_padded is None else k_padded
    out = torch.empty((rows, k_padded // 32, 36), dtype=torch.uint8, device=x.device)
    _lib.check("lk_quantize_q8_1", _lib.load().lk_quantize_q8_1(
        x.data_ptr(), _X_TYPES[x.dtype], out.data_ptr(), k, k_padded, rows, _stream()))
    return out


def _q8_1_rows(rows: int, cols: int, device) -> torch.Tensor:
    return torch.empty((rows, cols // 32, 36), dtype=torch.uint8, device=device)


def rmsnorm_q8_1(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """rms_norm_f32 with the row also quantized (src/tensor/cuda/gemm.rs:561-590) -> (out, q8_1)."""
    rows, cols = x.shape
    out, q = torch.empty_like(x), _q8_1_rows(rows, cols, x.device)
    _lib.check("lk_rmsnorm_q8_1", _lib.load().lk_rmsnorm_q8_1(
        x.data_ptr(), weight.data_ptr(), out.data_ptr(), q.data_ptr(), eps, cols, rows, _stream()))
    return out, q


def rms_quantize_q8_1(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """loken_rms_quantize_q8_1 / _bf16 (src/inference/moe_cuda/norm.rs:154, 206): one f32 or bf16 row of
    `hidden` values -> its RMS-normed Q8_1 blocks ``[hidden / 32, 36]`` (no f32 copy)."""
    hidden = x.numel()
    q = torch.zeros((hidden // 32, 36), dtype=torch.uint8, device=x.device)
    fn = {torch.float32: "loken_rms_quantize_q8_1", torch.bfloat16: "loken_rms_quantize_q8_1_bf16"}[x.dtype]
    getattr(_lib.load(), fn)(x.data_ptr(), weight.data_ptr(), q.data_ptr(), hidden, eps, _stream())
    return q


def add_rmsnorm_q8_1(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """fused_add_rmsnorm_dual (src/inference/kernel/fused/buffers/conv.rs:1043-1110) -> (sum, norm, q8_1)."""
    rows, cols = x.shape
    total, out, q = torch.empty_like(x), torch.empty_like(x), _q8_1_rows(rows, cols, x.device)
    _lib.check("lk_add_rmsnorm_q8_1", _lib.load().lk_add_rmsnorm_q8_1(
        x.data_ptr(), residual.data_ptr(), weight.data_ptr(), total.data_ptr(), out.data_ptr(), q.data_ptr(), eps,
        cols, rows, _stream()))
    return total, out, q


def post_norm_add_norm_q8_1(a: torch.Tensor, w_post: torch.Tensor, residual: torch.Tensor, w_ffn: torch.Tensor,
                            eps_post: float, eps_ffn: float):
    """fused_post_norm_add_norm (src/inference/kernel/fused/buffers/conv.rs:975-1035) -> (x, norm, q8_1)."""
    rows, cols = a.shape
    x_out, out, q = torch.empty_like(a), torch.empty_like(a), _q8_1_rows(rows, cols, a.device)
    _lib.check("lk_post_norm_add_norm_q8_1", _lib.load().lk_post_norm_add_norm_q8_1(
        a.data_ptr(), w_post.data_ptr(), residual.data_ptr(), w_ffn.data_ptr(), x_out.data_ptr(), out.data_ptr(),
        q.data_ptr(), eps_post, eps_ffn, cols, rows, _stream()))
    return x_out, out, q


def split_act_mul_q8_1(gu: torch.Tensor, act: int = 0):
    """``[rows, 2 n]`` gate|up -> (act(gate) * up ``[rows, n]``, its Q8_1 rows); act 0 SiLU, 1 tanh-GELU."""
    rows, two_n = gu.shape
    n = two_n // 2
    out = torch.empty((rows, n), dtype=torch.float32, device=gu.device)
    q = _q8_1_rows(rows, n, gu.device)
    _lib.check("lk_split_act_mul_q8_1", _lib.load().lk_split_act_mul_q8_1(
        gu.data_ptr(), out.data_ptr(), q.data_ptr(), n, rows, act, _stream()))
    return out, q


def mmvq(wtype: int, weight: torch.Tensor, q8_1: torch.Tensor, k: int, n: int, *,
         out_dtype: torch.dtype = torch.float32, bias: torch.Tensor | None = None,
         decode_order: bool = False) -> torch.Tensor:
    """``weight`` (uint8 blob of ``n`` rows of ``k`` values) x ``q8_1`` ``[b, k_padded/32, 36]``
    -> ``[b, n]``."""
    b = q8_1.shape[0]
    expect = n * (k // BLOCK_LEN[wtype]) * BLOCK_BYTES[wtype] if wtype in BLOCK_LEN else -1
    if weight.numel() < expect:
        raise ValueError(f"mmvq: weight holds {weight.numel()} bytes, {expect} needed")
    out = torch.empty((b, n), dtype=out_dtype, device=weight.device)
    _lib.check("lk_mmvq", _lib.load().lk_mmvq(
        wtype, weight.data_ptr(), q8_1.data_ptr(), out.data_ptr(), _X_TYPES[out_dtype], k, n, b,
        q8_1.shape[1], n, bias.data_ptr() if bias is not None else None, int(decode_order), _stream()))
    return out


def mmvq_multi(wtype: int, weights, q8_1: torch.Tensor, k: int, ns, *, out_dtype: torch.dtype = torch.float32):
    """Several matrices (same format, same k) over the same Q8_1 rows in one launch -> list of
    ``[b, n_i]`` outputs (forward_quantized_pair of the reference generalised to 4)."""
    import ctypes as C
    b = q8_1.shape[0]
    count = len(weights)
    outs = [torch.empty((b, n), dtype=out_dtype, device=q8_1.device) for n in ns]
    stride = max(ns)
    if any(n != stride for n in ns) and b > 1:
        # one destination row stride serves every matrix: give each its own launch-wide stride
        outs = [torch.empty((b, stride), dtype=out_dtype, device=q8_1.device) for _ in ns]
    vx = (C.c_void_p * count)(*[w.data_ptr() for w in weights])
    dst = (C.c_void_p * count)(*[o.data_ptr() for o in outs])
    nn = (C.c_int * count)(*ns)
    _lib.check("lk_mmvq_multi", _lib.load().lk_mmvq_multi(
        wtype, count, vx, q8_1.data_ptr(), dst, _X_TYPES[out_dtype], k, nn, b, q8_1.shape[1], stride, None, _stream()))
    return [o[:, :n] for o, n in zip(outs, ns)]


def mmvq_fused(wtype: int, weights, x: torch.Tensor, ns, *, out_dtype: torch.dtype = torch.float32):
    """Quantize-and-multiply in one launch: f32 rows ``x`` ``[b, k]`` against several matrices."""
    import ctypes as C
    b, k = x.shape
    count = len(weights)
    stride = max(ns)
    outs = [torch.empty((b, stride), dtype=out_dtype, device=x.device) for _ in ns]
    vx = (C.c_void_p * count)(*[w.data_ptr() for w in weights])
    dst = (C.c_void_p * count)(*[o.data_ptr() for o in outs])
    nn = (C.c_int * count)(*ns)
    _lib.check("lk_mmvq_fused", _lib.load().lk_mmvq_fused(
        wtype, count, vx, x.data_ptr(), x.stride(0), dst, _X_TYPES[out_dtype], k, nn, b, stride, None, _stream()))
    return [o[:, :n] for o, n in zip(outs, ns)]


def mmvq_pair_act(wtype: int, gate: torch.Tensor, up: torch.Tensor, q8_1: torch.Tensor, k: int, n: int, *,
                  act: str = "silu", out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``act(gate . x) * (up . x)`` in one launch (fast_mmvq::try_fused)."""
    b = q8_1.shape[0]
    out = torch.empty((b, n), dtype=out_dtype, device=q8_1.device)
    _lib.check("lk_mmvq_pair_act", _lib.load().lk_mmvq_pair_act(
        wtype, gate.data_ptr(), up.data_ptr(), q8_1.data_ptr(), out.data_ptr(), _X_TYPES[out_dtype], k, n, b,
        q8_1.shape[1], n, {"silu": 0, "gelu": 1}[act], _stream()))
    return out


def mmvq_pair_act_q8_1(wtype: int, gate: torch.Tensor, up: torch.Tensor, x: torch.Tensor, k: int, n: int, *,
                       act: str = "silu") -> torch.Tensor:
    """``Q8_1(act(gate . x) * (up . x))`` as ``[b, n/32, 36]`` bytes; ``x`` is f32 ``[b, k]`` or Q8_1
    ``[b, k_padded/32, 36]``."""
    is_f32 = x.dtype == torch.float32
    b = x.shape[0]
    out = torch.empty((b, n // 32, 36), dtype=torch.uint8, device=gate.device)
    _lib.check("lk_mmvq_pair_act_q8_1", _lib.load().lk_mmvq_pair_act_q8_1(
        wtype, gate.data_ptr(), up.data_ptr(), x.data_ptr(), int(is_f32), x.stride(0) if is_f32 else x.shape[1],
        out.data_ptr(), n // 32, k, n, b, {"silu": 0, "gelu": 1}[act], _stream()))
    return out


def mmvq_grouped(wtype: int, table: torch.Tensor, q8_1: torch.Tensor, k: int, n: int) -> torch.Tensor:
    """``groups`` same-shape weights (device address table, uint64) each over its own Q8_1 row."""
    groups = table.numel()
    out = torch.empty((groups, n), dtype=torch.float32, device=q8_1.device)
    _lib.check("lk_mmvq_grouped", _lib.load().lk_mmvq_grouped(
        wtype, table.data_ptr(), groups, q8_1.data_ptr(), out.data_ptr(), k, n, _stream()))
    return out


def mmvq_subdots(wtype: int, weight: torch.Tensor, q8_1_row: torch.Tensor, k: int, n: int):
    """Integer sub-block dots of every weight row against ONE Q8_1 row (parity probe)."""
    per = 16 if wtype in (_lib.TYPE_Q6_K, _lib.TYPE_Q2_K, _lib.TYPE_Q3_K, _lib.TYPE_IQ2_XXS, _lib.TYPE_IQ3_XXS, _lib.TYPE_IQ3_S,
                          _lib.TYPE_IQ2_S, _lib.TYPE_Q2_0) else 32
    dots = torch.empty((n, k // per), dtype=torch.int32, device=weight.device)
    sums = torch.empty((k // 32,), dtype=torch.int32, device=weight.device)
    _lib.check("lk_mmvq_subdots", _lib.load().lk_mmvq_subdots(
        wtype, weight.data_ptr(), q8_1_row.data_ptr(), dots.data_ptr(), sums.data_ptr(), k, n, _stream()))
    return dots, sums


# ------------------------------------------------------------------------------------ prefill
MMQ_QUANTIZER = {_lib.TYPE_Q4_K: "launch_mmq_quantize_q8_1_DS4", _lib.TYPE_Q5_K: "launch_mmq_quantize_q8_1_DS4",
                 _lib.TYPE_Q6_K: "launch_mmq_quantize_q8_1_D4",
                 _lib.TYPE_Q8_0: "launch_mmq_quantize_q8_1_D4",
                 # the 32-value formats as the reference's table pairs them (quantized/mmq.rs:274-285);
                 # IQ4_NL and MXFP4 are expert-only there and take the scale-only layout
                 _lib.TYPE_Q4_0: "launch_mmq_quantize_q8_1_DS4", _lib.TYPE_Q4_1: "launch_mmq_quantize_q8_1_DS4",
                 _lib.TYPE_Q5_0: "launch_mmq_quantize_q8_1_D4", _lib.TYPE_Q5_1: "launch_mmq_quantize_q8_1_DS4",
                 _lib.TYPE_IQ4_NL: "launch_mmq_quantize_q8_1_D4", _lib.TYPE_MXFP4: "launch_mmq_quantize_q8_1_D4",
                 _lib.TYPE_Q3_K: "launch_mmq_quantize_q8_1_D4", _lib.TYPE_IQ4_XS: "launch_mmq_quantize_q8_1_D4",
                 _lib.TYPE_IQ3_XXS: "launch_mmq_quantize_q8_1_D4", _lib.TYPE_IQ3_S: "launch_mmq_quantize_q8_1_D4",
                 _lib.TYPE_IQ2_S: "launch_mmq_quantize_q8_1_D4", _lib.TYPE_Q2_0: "launch_mmq_quantize_q8_1_D4",
                 _lib.TYPE_Q2_K: "launch_mmq_quantize_q8_1_D2S6"}
MMQ_LAUNCHER = {_lib.TYPE_Q4_K: "launch_mmq_gguf_q4_k", _lib.TYPE_Q5_K: "launch_mmq_gguf_q5_k",
                _lib.TYPE_Q6_K: "launch_mmq_gguf_q6_k",
                _lib.TYPE_Q8_0: "launch_mmq_gguf_q8_0",
                _lib.TYPE_Q4_0: "launch_mmq_gguf_q4_0", _lib.TYPE_Q4_1: "launch_mmq_gguf_q4_1",
                _lib.TYPE_Q5_0: "launch_mmq_gguf_q5_0", _lib.TYPE_Q5_1: "launch_mmq_gguf_q5_1",
                _lib.TYPE_Q3_K: "launch_mmq_gguf_q3_k", _lib.TYPE_Q2_K: "launch_mmq_gguf_q2_k"}
MMQ_DEVICE_INFO = dict(cc=0x1000950, nsm=256, smpbo=160 * 1024, warp_size=64)


def dense_q4k_rows(weight: torch.Tensor, x: torch.Tensor, n: int, q5: bool = False) -> torch.Tensor:
    """``[rows, k]`` f32 x Q4_K (``q5``: Q5_K) weight ``[n, k]`` -> ``[rows, n]`` f32 on the matrix unit, rows
    quantized to plain Q8_1 first (dense_q4k_imma_m8_matmul, src/inference/moe_cuda/dense/imma.rs:82-135)."""
    rows, k = x.shape
    if k % 256:
        raise ValueError("dense_q4k_rows: k must be a multiple of 256")
    q = quantize_q8_1_rows(x, k_padded=k)
    out = torch.empty((rows, n), dtype=torch.float32, device=x.device)
    # the status-returning form of loken_dense_q4k_imma_m8_plain: a launch it declines must not
    # come back as an untouched buffer
    fn = _lib.load().lk_dense_q5k_rows if q5 else _lib.load().lk_dense_q4k_rows
    _lib.check("lk_dense_q5k_rows" if q5 else "lk_dense_q4k_rows",
               fn(weight.data_ptr(), q.data_ptr(), out.data_ptr(), rows, n, k, _stream()))
    return out


def dense_q4k_rows_multi(weights, x: torch.Tensor, sizes_n, q5: bool = False, q8_1: torch.Tensor | None = None):
    """Up to three Q4_K (``q5``: Q5_K) weights ``[n_i, k]`` over the same ``[rows, k]`` f32 rows in one
    launch on the matrix unit (q + k + v); a list of ``[rows, n_i]`` f32 outputs. ``q8_1``: the rows
    already quantized (then ``x`` only gives the shape)."""
    import ctypes as C
    rows, k = x.shape
    if k % 256:
        raise ValueError("dense_q4k_rows_multi: k must be a multiple of 256")
    q = quantize_q8_1_rows(x, k_padded=k) if q8_1 is None else q8_1
    outs = [torch.empty((rows, n), dtype=torch.float32, device=x.device) for n in sizes_n]
    count = len(weights)
    wp = (C.c_void_p * count)(*[w.data_ptr() for w in weights])
    op = (C.c_void_p * count)(*[o.data_ptr() for o in outs])
    ns = (C.c_int * count)(*[int(n) for n in sizes_n])
    _lib.check("lk_dense_q4k_rows_multi",
               _lib.load().lk_dense_q4k_rows_multi(wp, op, ns, count, q.data_ptr(), rows, k, 1 if q5 else 0, _stream()))
    return outs


def mmq_workspace_bytes(rows: int, k: int) -> int:
    """The reference's sizing (kernel_matmul/mmq.rs:38-41): 144 bytes per 128 padded values per
    row, plus 128 records of slack."""
    k_padded = pad_to(pad_to(k, 512), 128)
    return rows * (k_padded // 128) * 144 + 128 * 144


def mmq_quantize(wtype: int, x: torch.Tensor, gather: torch.Tensor | None = None,
                 rows: int | None = None) -> torch.Tensor:
    """Rows of ``x`` ``[_, k]`` (f32 or f16) into the tile kernels' workspace; row ``i`` of the
    result is row ``gather[i]`` of ``x`` when a gather is given (MmqRouting::quantize)."""
    k = x.shape[1]
    rows = (gather.numel() if gather is not None else x.shape[0]) if rows is None else rows
    k_padded = pad_to(pad_to(k, 512), 128)
    ws = torch.empty(mmq_workspace_bytes(rows, k), dtype=torch.uint8, device=x.device)
    fn = getattr(_lib.load(), MMQ_QUANTIZER[wtype])
    fn(x.data_ptr(), gather.data_ptr() if gather is not None else None, ws.data_ptr(),
       1 if x.dtype == torch.float16 else 0, k, x.stride(0), 0, 0, k_padded, rows, 1, 1, _stream())
    return ws


MMQ_FIXUP_BYTES = 256 * 128 * 128 * 4   # FIXUP_BYTES of MmqWorkspace (kernel_matmul/mmq.rs:42)
_mmq_fixup = {}


def mmq_fixup(device) -> torch.Tensor:
    """The card's ``tmp_fixup`` buffer of MmqWorkspace (kernel_matmul/mmq.rs:42-60), made on first use and kept:
    the tiled launchers hold the partial products of a cut K there (calls that share it must not overlap,
    as with the reference's workspace)."""
    key = torch.device(device)
    if key not in _mmq_fixup:
        _mmq_fixup[key] = torch.empty(MMQ_FIXUP_BYTES, dtype=torch.uint8, device=key)
    return _mmq_fixup[key]


def mmq_forward(wtype: int, weight: torch.Tensor, x: torch.Tensor, n: int, fixup: bool = True) -> torch.Tensor:
    """``[rows, k]`` x weight ``[n, k]`` -> ``[rows, n]`` f32 through the tiled kernels, the two
    launches of QKernelMatMul::mmq_forward (kernel_matmul/mmq.rs:103-136). ``fixup`` false passes no
    ``tmp_fixup``: the launcher then never cuts K."""
    rows, k = x.shape
    ws = mmq_quantize(wtype, x)
    out = torch.empty((rows, n), dtype=torch.float32, device=x.device)
    fn = getattr(_lib.load(), MMQ_LAUNCHER[wtype])
    i = MMQ_DEVICE_INFO
    fix = mmq_fixup(x.device).data_ptr() if fixup else None
    launched = fn(fix, weight.data_ptr(), ws.data_ptr(), out.data_ptr(), k, n, rows, k // BLOCK_LEN[wtype], n,
                  i["cc"], i["nsm"], i["smpbo"], i["warp_size"], _stream())
    if launched == 0:
        raise _lib.LokenError(MMQ_LAUNCHER[wtype], _lib.LK_ERR_ARG)
    return out


def dense_q4k_rows_actmul(gate: torch.Tensor, up: torch.Tensor, x: torch.Tensor, n: int, use_gelu: bool,
                          q5: bool = False) -> torch.Tensor:
    """``act(gate . x) * (up . x)`` for ``[rows, k]`` f32 x two Q4_K (``q5``: Q5_K) weights ``[n, k]`` in one launch
    on the matrix unit (dense_q4k_imma_m8_act_mul, src/inference/moe_cuda/dense/imma.rs:320-400)."""
    rows, k = x.shape
    if k % 256:
        raise ValueError("dense_q4k_rows_actmul: k must be a multiple of 256")
    q = quantize_q8_1_rows(x, k_padded=k)
    out = torch.empty((rows, n), dtype=torch.float32, device=x.device)
    fn = _lib.load().lk_dense_q5k_rows_actmul if q5 else _lib.load().lk_dense_q4k_rows_actmul
    _lib.check("lk_dense_q5k_rows_actmul" if q5 else "lk_dense_q4k_rows_actmul",
               fn(gate.data_ptr(), up.data_ptr(), q.data_ptr(), out.data_ptr(), rows, n, k, 1 if use_gelu else 0, _stream()))
    return out


def dense_q4k_rows_actmul_q8_1(gate: torch.Tensor, up: torch.Tensor, x: torch.Tensor, n: int, use_gelu: bool,
                               q5: bool = False) -> torch.Tensor:
    """dense_q4k_rows_actmul with the result as Q8_1 rows ``[rows, n / 32, 36]`` (what the down projection
    reads): at most 16 rows, k 2048 or 4096, n a multiple of 32."""
    rows, k = x.shape
    q = quantize_q8_1_rows(x, k_padded=k)
    out = torch.empty((rows, n // 32, 36), dtype=torch.uint8, device=x.device)
    _lib.check("lk_dense_q4k_rows_actmul_q8_1",
               _lib.load().lk_dense_q4k_rows_actmul_q8_1(gate.data_ptr(), up.data_ptr(), q.data_ptr(), out.data_ptr(), rows, n,
                                                         k, 1 if use_gelu else 0, 1 if q5 else 0, _stream()))
    return out


def mmvq_exact(wtype: int, weight: torch.Tensor, q8_k: torch.Tensor, n: int) -> torch.Tensor:
    """Q4_K / Q6_K weight ``[n, k]`` x Q8_K rows ``[rows, k / 256, 292]`` uint8 -> ``[rows, n]`` f32 with the
    reference's exact fold (dot_exact, src/tensor/quant_cpu/format/q4_k.rs:117-156, q6_k.rs:121-163): the bits
    of the CPU path."""
    rows, nb, _ = q8_k.shape
    out = torch.empty((rows, n), dtype=torch.float32, device=q8_k.device)
    _lib.check("lk_mmvq_exact", _lib.load().lk_mmvq_exact(wtype, weight.data_ptr(), q8_k.data_ptr(), out.data_ptr(),
                                                          nb * 256, n, rows, _stream()))
    return out


def dense_q6k_rows(weight: torch.Tensor, x: torch.Tensor, n: int) -> torch.Tensor:
    """``[rows, k]`` f32 x Q6_K weight ``[n, k]`` -> ``[rows, n]`` f32 on the matrix unit, rows
    quantized to plain Q8_1 first."""
    rows, k = x.shape
    if k % 256:
        raise ValueError("dense_q6k_rows: k must be a multiple of 256")
    q = quantize_q8_1_rows(x, k_padded=k)
    out = torch.empty((rows, n), dtype=torch.float32, device=x.device)
    _lib.check("lk_dense_q6k_rows",
               _lib.load().lk_dense_q6k_rows(weight.data_ptr(), q.data_ptr(), out.data_ptr(), rows, n, k, _stream()))
    return out

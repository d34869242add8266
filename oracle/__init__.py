"""ctypes binding of the CPU oracle (``libloken_oracle.so``). TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package, and only as the checker; the shipped ``loken_amd`` package never does.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libloken_oracle.so"

Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
IQ4_NL, MXFP4 = 20, 39
Q2_K, Q3_K = 10, 11
IQ4_XS = 23
IQ2_XXS, IQ3_XXS, IQ3_S, IQ2_S, Q2_0 = 16, 18, 21, 22, 42   # the codebook expert formats
CODEBOOK = (IQ2_XXS, IQ3_XXS, IQ3_S, IQ2_S, Q2_0)
Q8_0, Q8_1, Q4_K, Q5_K, Q6_K, Q8_K = 8, 9, 12, 13, 14, 15
BLOCK_LEN = {IQ2_XXS: 256, IQ3_XXS: 256, IQ3_S: 256, IQ2_S: 256, Q2_0: 64, IQ4_XS: 256, Q2_K: 256, Q3_K: 256, IQ4_NL: 32, MXFP4: 32, Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: 32, Q8_1: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256, Q8_K: 256}
BLOCK_BYTES = {IQ2_XXS: 66, IQ3_XXS: 98, IQ3_S: 110, IQ2_S: 82, Q2_0: 18, IQ4_XS: 136, Q2_K: 84, Q3_K: 110, IQ4_NL: 18, MXFP4: 17, Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: 34, Q8_1: 36, Q4_K: 144, Q5_K: 176, Q6_K: 210, Q8_K: 292}


def build(force: bool = False) -> Path:
    """Compile the oracle with the Makefile beside it (gcc only)."""
    if force:
        subprocess.run(["make", "-C", str(_HERE), "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", str(_HERE)], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        _lib = C.CDLL(str(_LIB_PATH))
        _declare(_lib)
    return _lib


_sz, _i, _vp = C.c_size_t, C.c_int, C.c_void_p


def _declare(l: C.CDLL) -> None:
    l.lko_f16_to_f32.restype = C.c_float
    l.lko_f16_to_f32.argtypes = [C.c_uint16]
    l.lko_f32_to_f16.restype = C.c_uint16
    l.lko_f32_to_f16.argtypes = [C.c_float]
    l.lko_unpack_scales_mins.argtypes = [_vp, _vp, _vp]
    l.lko_pack_scales_mins.argtypes = [_vp, _vp, _vp]
    l.lko_dequantize.argtypes = [_i, _vp, _sz, _vp]
    for name in ("lko_quantize_q8_0", "lko_quantize_q8_1", "lko_quantize_q8_k"):
        getattr(l, name).argtypes = [_vp, _sz, _vp]
        getattr(l, name).restype = None
    l.oa_matmul.argtypes = [_i, _sz, _sz, _sz, _vp, _vp, _sz, _vp]
    l.oa_matmul_fast.argtypes = [_i, _sz, _sz, _sz, _vp, _vp, _sz, _vp, _i]
    l.oa_matmul_exact.argtypes = [_i, _sz, _sz, _sz, _vp, _vp, _vp]
    l.lko_dot_q4k_q8k.argtypes = [_i, _vp, _vp, _sz]
    l.lko_dot_q4k_q8k.restype = C.c_float
    l.lko_dot_q4k_q8k_many.argtypes = [_vp, _vp, _sz, _sz, _vp]
    l.lko_dot_q4k_q8k_many.restype = None
    for fn in (l.oa_matmul_multi, l.oa_matmul_grouped):
        fn.argtypes = [_i, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp]
        fn.restype = _i
    l.ob_subdots.argtypes = [_i, _sz, _sz, _vp, _vp, _vp, _vp]
    l.lko_cb_run.argtypes = [_i, _vp, _i, _vp, _vp]
    l.lko_cb_table.argtypes = [_i, _vp]
    l.lko_cb_table.restype = _vp
    l.ob_matmul_q8_1.argtypes = [_i, _sz, _sz, _sz, _vp, _sz, _vp, _vp]
    l.ob_matmul.argtypes = [_i, _sz, _sz, _sz, _vp, _vp, _vp]
    l.ob_matmul_f64.argtypes = [_i, _sz, _sz, _sz, _vp, _vp, _vp]
    l.lko_topk_softmax.argtypes = [_vp, _sz, _sz, _sz, _i, _vp, _vp]
    l.lko_topk_softmax.restype = None
    l.lko_topk_sigmoid.argtypes = [_vp, _vp, _sz, _sz, _sz, _i, C.c_float, _vp, _vp]
    l.lko_topk_sigmoid.restype = None
    l.lko_group_by_expert.argtypes = [_vp, _sz, _vp, _vp]
    l.lko_group_by_expert.restype = None
    l.lko_moe_forward.argtypes = [_i, _i, _i, _sz, _sz, _sz, _sz, _sz] + [_vp] * 8
    l.lko_cpu_has_avx2.restype = _i
    l.lko_pool_start.argtypes = [_i]
    l.lko_repack_q4k_x8.argtypes = [_vp, _sz, _sz, _vp]
    l.lko_repack_q4k_x8.restype = None
    l.oa_matmul_q4k_x8.argtypes = [_sz, _sz, _sz, _vp, _vp, _vp]
    l.oa_matmul_q4k_x8_tiled.argtypes = [_sz, _sz, _sz, _vp, _vp, _vp]
    l.lko_repack_q6k_x8.argtypes = [_vp, _sz, _sz, _vp]
    l.lko_repack_q6k_x8.restype = None
    l.oa_matmul_q6k_x8_tiled.argtypes = [_sz, _sz, _sz, _vp, _vp, _vp]
    l.lko_gemv_group_q6k_x8_scalar.argtypes = [_vp, _vp, _sz, _vp]
    l.lko_gemv_group_q6k_x8_scalar.restype = None
    l.lko_moe_forward_pool.argtypes = [_i, _i, _i, _sz, _sz, _sz, _sz, _sz] + [_vp] * 7
    l.lko_inv_rms_wide.restype = C.c_float
    l.lko_inv_rms_wide.argtypes = [_vp, _sz, C.c_float]
    l.lko_norm_rows.restype = None
    l.lko_norm_rows.argtypes = [_i, _vp, _vp, _vp, _vp, _vp, _vp, C.c_float, C.c_float, _sz, _sz]
    l.lko_split_act_mul.restype = None
    l.lko_split_act_mul.argtypes = [_vp, _vp, _sz, _sz, _i]


def _p(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8).reshape(-1)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def f16_to_f32(h: int) -> float:
    return float(lib().lko_f16_to_f32(int(h)))


def f32_to_f16(f: float) -> int:
    return int(lib().lko_f32_to_f16(float(f)))


def unpack_scales_mins(packed12) -> tuple[np.ndarray, np.ndarray]:
    p = _u8(packed12)
    sc, mn = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
    lib().lko_unpack_scales_mins(_p(p), _p(sc), _p(mn))
    return sc, mn


def pack_scales_mins(scales, mins) -> np.ndarray:
    sc, mn = _u8(scales), _u8(mins)
    out = np.zeros(12, np.uint8)
    lib().lko_pack_scales_mins(_p(sc), _p(mn), _p(out))
    return out


def dequantize(dtype: int, blocks) -> np.ndarray:
    b = _u8(blocks)
    n_blocks = b.size // BLOCK_BYTES[dtype]
    out = np.empty(n_blocks * BLOCK_LEN[dtype], np.float32)
    rc = lib().lko_dequantize(dtype, _p(b), n_blocks, _p(out))
    if rc:
        raise ValueError(f"dequantize: dtype {dtype} not handled")
    return out


def _quantize(fn: str, dtype: int, x) -> np.ndarray:
    x = _f32(x).reshape(-1)
    assert x.size % BLOCK_LEN[dtype] == 0
    out = np.zeros(x.size // BLOCK_LEN[dtype] * BLOCK_BYTES[dtype], np.uint8)
    getattr(lib(), fn)(_p(x), x.size, _p(out))
    return out


def quantize_q8_0(x) -> np.ndarray:
    return _quantize("lko_quantize_q8_0", Q8_0, x)


def quantize_q8_1(x) -> np.ndarray:
    return _quantize("lko_quantize_q8_1", Q8_1, x)


def quantize_q8_k(x) -> np.ndarray:
    return _quantize("lko_quantize_q8_k", Q8_K, x)


class OracleError(ValueError):
    pass


_ERR = {-1: "k is not a multiple of the block size", -2: "rhs byte length is wrong",
        -3: "dtype not handled", -4: "an lhs entry has the wrong length", -5: "an outs entry has the wrong length"}


def _check(rc: int) -> None:
    if rc:
        raise OracleError(_ERR.get(rc, f"oracle error {rc}"))


def oa_matmul(dtype: int, lhs, rhs, n: int, *, fast_threads: int = 0, exact: bool = False) -> np.ndarray:
    lhs = _f32(lhs)
    m, k = lhs.shape
    rhs = _u8(rhs)
    dst = np.empty((m, n), np.float32)
    if exact:
        _check(lib().oa_matmul_exact(dtype, m, k, n, _p(lhs), _p(rhs), _p(dst)))
    elif fast_threads > 0:
        _check(lib().oa_matmul_fast(dtype, m, k, n, _p(lhs), _p(rhs), rhs.size, _p(dst), fast_threads))
    else:
        _check(lib().oa_matmul(dtype, m, k, n, _p(lhs), _p(rhs), rhs.size, _p(dst)))
    return dst


def _per_expert(fn, dtype: int, k: int, n: int, rhs_list, lhs_list, out_shapes):
    import ctypes as C
    ne = len(rhs_list)
    rhs = [_u8(r) for r in rhs_list]
    lhs = [_f32(x).reshape(-1) for x in lhs_list]
    outs = [np.empty(int(np.prod(s)), np.float32) for s in out_shapes]
    ptrs = lambda arrs: (C.c_void_p * max(ne, 1))(*[a.ctypes.data for a in arrs])
    sizes = lambda arrs: (C.c_size_t * max(ne, 1))(*[a.size for a in arrs])
    _check(fn(dtype, k, n, ne, ptrs(rhs), sizes(rhs), ptrs(lhs), sizes(lhs), ptrs(outs), sizes(outs)))
    return [o.reshape(s) for o, s in zip(outs, out_shapes)]


def oa_matmul_multi(dtype: int, k: int, n: int, rhs_list, lhs_list, out_lens=None):
    """matmul_bytes_multi: expert e's one row against its own weight -> a list of ``[n]`` outputs."""
    shapes = [(n,)] * len(rhs_list) if out_lens is None else [(l,) for l in out_lens]
    return _per_expert(lib().oa_matmul_multi, dtype, k, n, rhs_list, lhs_list, shapes)


def oa_matmul_grouped(dtype: int, k: int, n: int, rhs_list, lhs_list, out_shapes=None):
    """matmul_bytes_grouped: expert e's rows ``[rows_e, k]`` against its own weight -> ``[rows_e, n]`` each."""
    if out_shapes is None:
        out_shapes = [(np.asarray(x).size // k, n) for x in lhs_list]
    return _per_expert(lib().oa_matmul_grouped, dtype, k, n, rhs_list, lhs_list, out_shapes)


def dot_q4k_q8k(w_row, x_row, wide: bool = False) -> float:
    """One Q4_K row against one f32 row quantized to Q8_K, through the 256-bit or the 512-bit kernel."""
    w = _u8(w_row)
    x = _f32(x_row).reshape(-1)
    nb = x.size // 256
    act = np.empty(nb * 292, np.uint8)
    lib().lko_quantize_q8_k(_p(x), x.size, _p(act))
    return float(lib().lko_dot_q4k_q8k(1 if wide else 0, _p(w), _p(act), nb))


def dot_q4k_q8k_many(w_row, x_rows) -> np.ndarray:
    """One Q4_K row against several f32 rows (each quantized to Q8_K) in passes of four."""
    import ctypes as C
    w = _u8(w_row)
    x = _f32(x_rows)
    rows, k = x.shape
    nb = k // 256
    acts = [np.empty(nb * 292, np.uint8) for _ in range(rows)]
    for r in range(rows):
        lib().lko_quantize_q8_k(_p(np.ascontiguousarray(x[r])), k, _p(acts[r]))
    ptrs = (C.c_void_p * max(rows, 1))(*[a.ctypes.data for a in acts])
    out = np.empty(rows, np.float32)
    lib().lko_dot_q4k_q8k_many(_p(w), ptrs, rows, nb, _p(out))
    return out


def repack_q4k_x8(rhs, n: int, k: int) -> np.ndarray:
    """Q4_K rows `[n, k/256]` (n a multiple of 8) -> the eight-row group blocks the served CPU path reads."""
    rhs = _u8(rhs)
    nb = k // 256
    out = np.empty((n // 8) * nb * 1152, np.uint8)
    lib().lko_repack_q4k_x8(_p(rhs), n, nb, _p(out))
    return out


def oa_matmul_q4k_x8(lhs, x8: np.ndarray, n: int) -> np.ndarray:
    """The served Q4_K CPU path: Q8_K activations against repacked weights on the persistent pool."""
    lhs = _f32(lhs)
    m, k = lhs.shape
    dst = np.empty((m, n), np.float32)
    _check(lib().oa_matmul_q4k_x8(m, k, n, _p(lhs), _p(x8), _p(dst)))
    return dst


def oa_matmul_q4k_x8_tiled(lhs, x8: np.ndarray, n: int) -> np.ndarray:
    """The served Q4_K prefill path: one pool chunk per eight columns, rows in tiles of eight."""
    lhs = _f32(lhs)
    m, k = lhs.shape
    dst = np.empty((m, n), np.float32)
    _check(lib().oa_matmul_q4k_x8_tiled(m, k, n, _p(lhs), _p(x8), _p(dst)))
    return dst


def repack_q6k_x8(rhs, n: int, k: int) -> np.ndarray:
    """Q6_K rows `[n, k/256]` (n a multiple of 8) -> eight-row group blocks of 1680 bytes."""
    rhs = _u8(rhs)
    nb = k // 256
    out = np.empty((n // 8) * nb * 1680, np.uint8)
    lib().lko_repack_q6k_x8(_p(rhs), n, nb, _p(out))
    return out


def oa_matmul_q6k_x8_tiled(lhs, x8: np.ndarray, n: int) -> np.ndarray:
    """The served Q6_K prefill path over repacked weights."""
    lhs = _f32(lhs)
    m, k = lhs.shape
    dst = np.empty((m, n), np.float32)
    _check(lib().oa_matmul_q6k_x8_tiled(m, k, n, _p(lhs), _p(x8), _p(dst)))
    return dst


def gemv_group_q6k_x8_scalar(x8: np.ndarray, group: int, nb: int, act_q8k: np.ndarray) -> np.ndarray:
    """Scalar group dot of group `group` against one Q8_K row (`nb` blocks of 292 bytes)."""
    x8 = _u8(x8)
    act_q8k = _u8(act_q8k)
    out = np.empty(8, np.float32)
    grp = np.ascontiguousarray(x8.reshape(-1)[group * nb * 1680:(group + 1) * nb * 1680])
    lib().lko_gemv_group_q6k_x8_scalar(_p(grp), _p(act_q8k), nb, _p(out))
    return out


def moe_forward_pool(family: int, dt_gu: int, dt_down: int, x, gate, up, down, ids, weights,
                     n_experts: int, ffn: int) -> np.ndarray:
    """`moe_forward` with the tokens spread over the worker pool."""
    x = _f32(x)
    tokens, hidden = x.shape
    ids = np.ascontiguousarray(ids, np.int32)
    weights = _f32(weights)
    gate, up, down = _u8(gate), _u8(up), _u8(down)
    out = np.empty((tokens, hidden), np.float32)
    _check(lib().lko_moe_forward_pool(family, dt_gu, dt_down, tokens, hidden, ffn, n_experts, ids.shape[1],
                                      _p(x), _p(gate), _p(up), _p(down), _p(ids), _p(weights), _p(out)))
    return out


def pool_start(threads: int = 0) -> int:
    return lib().lko_pool_start(threads)


def cpu_counts() -> tuple[int, int]:
    """(physical cores, logical CPUs) this process may run on."""
    return lib().lko_physical_cores(), lib().lko_logical_cpus()


def ob_matmul(dtype: int, lhs, rhs, n: int) -> np.ndarray:
    lhs = _f32(lhs)
    m, k = lhs.shape
    rhs = _u8(rhs)
    dst = np.empty((m, n), np.float32)
    _check(lib().ob_matmul(dtype, m, k, n, _p(lhs), _p(rhs), _p(dst)))
    return dst


def ob_matmul_q8_1(dtype: int, act_q8_1, m: int, k: int, rhs, n: int, stride_blocks: int | None = None) -> np.ndarray:
    act = _u8(act_q8_1)
    rhs = _u8(rhs)
    dst = np.empty((m, n), np.float32)
    _check(lib().ob_matmul_q8_1(dtype, m, k, n, _p(act), stride_blocks or k // 32, _p(rhs), _p(dst)))
    return dst


def ob_matmul_f64(dtype: int, lhs, rhs, n: int) -> np.ndarray:
    lhs = _f32(lhs)
    m, k = lhs.shape
    rhs = _u8(rhs)
    dst = np.empty((m, n), np.float64)
    _check(lib().ob_matmul_f64(dtype, m, k, n, _p(lhs), _p(rhs), _p(dst)))
    return dst


def ob_subdots(dtype: int, k: int, n: int, rhs, act_q8_1) -> tuple[np.ndarray, np.ndarray]:
    """(dots[n, k/32 or k/16], sums[k/32]) of weight rows against one Q8_1 activation row."""
    rhs, act = _u8(rhs), _u8(act_q8_1)
    per = 16 if dtype in (Q6_K, Q2_K, Q3_K) or dtype in CODEBOOK else 32
    dots = np.empty((n, k // per), np.int32)
    sums = np.empty(k // 32, np.int32)
    _check(lib().ob_subdots(dtype, k, n, _p(rhs), _p(act), _p(dots), _p(sums)))
    return dots, sums


def codebook_run(dtype: int, block, run: int) -> tuple[np.ndarray, np.ndarray]:
    """(32 signed integer weights, the scales of the two halves) of run `run` of one block."""
    block = _u8(block)
    v = np.empty(32, np.int8)
    s = np.empty(2, np.float32)
    _check(lib().lko_cb_run(dtype, _p(block), run, _p(v), _p(s)))
    return v, s


def codebook_table(dtype: int) -> bytes:
    """The expanded grid of a codebook format, little-endian entries."""
    n = C.c_size_t(0)
    ptr = lib().lko_cb_table(dtype, C.byref(n))
    return C.string_at(ptr, n.value)


def topk_softmax(logits, topk: int, renorm: bool = True) -> tuple[np.ndarray, np.ndarray]:
    logits = _f32(logits)
    t, e = logits.shape
    ids = np.empty((t, topk), np.int32)
    w = np.empty((t, topk), np.float32)
    lib().lko_topk_softmax(_p(logits), t, e, topk, int(renorm), _p(ids), _p(w))
    return ids, w


def group_by_expert(ids) -> tuple[np.ndarray, np.ndarray]:
    ids = np.ascontiguousarray(ids, np.int32).reshape(-1)
    slots = np.empty(ids.size, np.int32)
    experts = np.empty(ids.size, np.int32)
    lib().lko_group_by_expert(_p(ids), ids.size, _p(slots), _p(experts))
    return slots, experts


def moe_forward(family: int, dt_gu: int, dt_down: int, x, gate, up, down, ids, weights,
                n_experts: int, ffn: int, want_h: bool = False):
    x = _f32(x)
    tokens, hidden = x.shape
    ids = np.ascontiguousarray(ids, np.int32)
    topk = ids.shape[1]
    weights = _f32(weights)
    gate, up, down = _u8(gate), _u8(up), _u8(down)
    out = np.empty((tokens, hidden), np.float32)
    h = np.empty((tokens * topk, ffn), np.float32) if want_h else None
    _check(lib().lko_moe_forward(family, dt_gu, dt_down, tokens, hidden, ffn, n_experts, topk,
                                 _p(x), _p(gate), _p(up), _p(down), _p(ids), _p(weights),
                                 _p(h) if want_h else None, _p(out)))
    return (out, h) if want_h else out


def inv_rms_wide(row, eps: float) -> float:
    row = _f32(row).reshape(-1)
    return float(lib().lko_inv_rms_wide(_p(row), row.size, eps))


def norm_rows(mode: int, x, w, *, w_first=None, residual=None, eps: float = 1e-6, eps_first: float = 1e-6):
    """mode 0 -> out; mode 1 (add then norm) and 2 (norm, add, norm) -> (mid, out)."""
    x = _f32(x)
    rows, cols = x.shape
    w = _f32(w)
    w_first = _f32(w_first) if w_first is not None else None
    residual = _f32(residual) if residual is not None else None
    out = np.empty_like(x)
    mid = np.empty_like(x) if mode else None
    lib().lko_norm_rows(mode, _p(x), _p(w_first) if w_first is not None else None,
                        _p(residual) if residual is not None else None, _p(w), _p(mid) if mode else None, _p(out),
                        eps_first, eps, cols, rows)
    return (mid, out) if mode else out


def split_act_mul(gu, act: int = 0) -> np.ndarray:
    gu = _f32(gu)
    rows, two_n = gu.shape
    out = np.empty((rows, two_n // 2), np.float32)
    lib().lko_split_act_mul(_p(gu), _p(out), two_n // 2, rows, act)
    return out


def topk_sigmoid(logits, topk: int, bias=None, renorm: bool = True, scale: float = 1.0):
    logits = _f32(logits)
    t, e = logits.shape
    bias = _f32(bias) if bias is not None else None
    ids = np.empty((t, topk), np.int32)
    w = np.empty((t, topk), np.float32)
    lib().lko_topk_sigmoid(_p(logits), _p(bias) if bias is not None else None, t, e, topk, int(renorm), scale,
                           _p(ids), _p(w))
    return ids, w

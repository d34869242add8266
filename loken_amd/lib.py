"""Loads ``libloken_gfx950.so`` and declares the C ABI of ``include/loken_gfx950.h``.

There is no fallback: a missing library raises, it is never replaced by another code path.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libloken_gfx950.so"

LK_OK, LK_ERR_ARG, LK_ERR_TYPE, LK_ERR_LAUNCH, LK_ERR_NOMEM, LK_ERR_SIZE, LK_NOT_TAKEN = 0, 1, 2, 3, 4, 5, 6
_ERR_NAMES = {1: "LK_ERR_ARG", 2: "LK_ERR_TYPE", 3: "LK_ERR_LAUNCH", 4: "LK_ERR_NOMEM", 5: "LK_ERR_SIZE", 6: "LK_NOT_TAKEN"}
STATIC_SCRATCH_BYTES = 8 << 20

TYPE_F32, TYPE_F16, TYPE_BF16 = 0, 1, 30
TYPE_Q4_0, TYPE_Q4_1, TYPE_Q5_0, TYPE_Q5_1 = 2, 3, 6, 7
TYPE_IQ4_NL, TYPE_MXFP4 = 20, 39
TYPE_Q2_K, TYPE_Q3_K = 10, 11
TYPE_IQ4_XS = 23
TYPE_IQ2_XXS, TYPE_IQ3_XXS, TYPE_IQ3_S, TYPE_IQ2_S, TYPE_Q2_0 = 16, 18, 21, 22, 42
TYPE_Q8_0, TYPE_Q8_1, TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K = 8, 9, 12, 13, 14


class LokenError(RuntimeError):
    def __init__(self, fn: str, code: int):
        super().__init__(f"{fn} failed: {_ERR_NAMES.get(code, code)}")
        self.code = code


_vp, _i, _i64, _f = C.c_void_p, C.c_int, C.c_int64, C.c_float
_cp, _u64 = C.c_char_p, C.c_uint64

# name -> (restype, argtypes); mirrors include/loken_gfx950.h declaration by declaration
SIGNATURES = {
    "lk_device_info": (_i, [_vp, _vp, _vp, _vp]),
    "lk_quantize_q8_1": (_i, [_vp, _i, _vp, _i, _i, _i, _vp]),
    "lk_mmvq": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _i, _vp]),
    "lk_mmvq_multi": (_i, [_i, _i, _vp, _vp, _vp, _i, _i, _vp, _i, _i, _i, _vp, _vp]),
    "lk_mmvq_fused": (_i, [_i, _i, _vp, _vp, _i, _vp, _i, _i, _vp, _i, _i, _vp, _vp]),
    "lk_mmvq_pair_act": (_i, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "lk_mmvq_grouped": (_i, [_i, _vp, _i, _vp, _vp, _i, _i, _vp]),
    "lk_mmvq_subdots": (_i, [_i, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "launch_mmq_quantize_q8_1_D4": (None, [_vp, _vp, _vp, _i] + [_i64] * 8 + [_vp]),
    "launch_mmq_quantize_q8_1_DS4": (None, [_vp, _vp, _vp, _i] + [_i64] * 8 + [_vp]),
    "launch_mmq_quantize_q8_1_D2S6": (None, [_vp, _vp, _vp, _i] + [_i64] * 8 + [_vp]),
    "launch_mmq_gguf_q4_k": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q5_k": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q6_k": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q8_0": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q4_0": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q4_1": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q5_0": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q5_1": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q3_k": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
    "launch_mmq_gguf_q2_k": (_i, [_vp, _vp, _vp, _vp] + [_i64] * 5 + [_i, _i, _i64, _i, _vp]),
}
_MOE_MMQ = (_i, [_vp, _vp, _i64, _vp, _vp, _vp, _vp] + [_i64] * 6 + [_i, _i64, _i64, _i, _i, _i64, _i, _vp])
SIGNATURES.update({
    "launch_mmq_moe_gguf_q4_k": _MOE_MMQ,
    "launch_mmq_moe_gguf_q5_k": _MOE_MMQ,
    "launch_mmq_moe_gguf_q6_k": _MOE_MMQ,
    "launch_mmq_moe_gguf_q8_0": _MOE_MMQ,
    "launch_mmq_moe_gguf_q4_0": _MOE_MMQ,
    "launch_mmq_moe_gguf_q4_1": _MOE_MMQ,
    "launch_mmq_moe_gguf_q5_0": _MOE_MMQ,
    "launch_mmq_moe_gguf_q5_1": _MOE_MMQ,
    "launch_mmq_moe_gguf_iq4_nl": _MOE_MMQ,
    "launch_mmq_moe_gguf_mxfp4": _MOE_MMQ,
    "launch_mmq_moe_gguf_q3_k": _MOE_MMQ,
    "launch_mmq_moe_gguf_q2_k": _MOE_MMQ,
    "launch_mmq_moe_gguf_iq4_xs": _MOE_MMQ,
    "launch_mmq_moe_gguf_iq3_xxs": _MOE_MMQ,
    "launch_mmq_moe_gguf_iq3_s": _MOE_MMQ,
    "launch_mmq_moe_gguf_iq2_s": _MOE_MMQ,
    "launch_mmq_moe_gguf_q2_0": _MOE_MMQ,
    "loken_moe_mmq_plan": (None, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "loken_moe_mmq_route": (None, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "loken_moe_mmq_silu_mul": (None, [_vp, _vp, _i64, _i, _vp]),
    "loken_moe_mmq_swiglu_oai": (None, [_vp, _vp, _i64, _i, _vp, _i, _vp, _vp, _f, _f, _vp]),
    "loken_moe_gemm_gguf": (_i, [_vp] * 6 + [_i] * 6 + [_vp]),
    "loken_moe_gemm_gguf_gate_up_silu_mul": (_i, [_vp] * 6 + [_i] * 6 + [_vp]),
    "loken_moe_gemm_gguf_gate_up_swiglu_oai": (_i, [_vp] * 8 + [_i] * 6 + [_f, _f, _vp]),
    "loken_moe_gemm_gguf_gate_up_swiglu_limited": (_i, [_vp] * 6 + [_i] * 6 + [_f, _vp]),
    "loken_moe_gemm_gguf_gate_up_gelu_mul_concat": (_i, [_vp] * 5 + [_i] * 6 + [_vp]),
    "loken_moe_gemm_gguf_gate_up_silu_mul_live": (_i, [_vp] * 6 + [_i] * 6 + [_vp, _vp]),
    "loken_moe_gemm_gguf_down_pairs_live": (_i, [_vp] * 6 + [_i] * 6 + [_vp, _vp]),
    "loken_moe_gemm_gguf_gate_up_silu_mul_two": (_i, [_vp] * 5 + [_i] + [_vp] * 4 + [_i] * 6 + [_vp]),
    "loken_moe_gemm_gguf_down_reduce_two": (_i, [_vp] * 3 + [_i] + [_vp] * 4 + [_i] * 6 + [_vp, _vp, _vp]),
    "loken_moe_gemm_gguf_down_pairs_two": (_i, [_vp] * 3 + [_i] + [_vp] * 5 + [_i] * 6 + [_vp]),
    "loken_moe_gemm_gguf_down_reduce": (_i, [_vp] * 6 + [_i] * 6 + [_vp, _vp, _vp]),
    "loken_moe_gemm_gguf_down_reduce_static": (_i, [_vp] * 6 + [_i] * 6 + [_vp, _vp, _vp]),
    "loken_moe_sum_topk": (None, [_vp, _vp, _i, _i, _i, _vp]),
    "loken_stream_scratch_release": (None, []),
    "lk_rmsnorm_q8_1": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _vp]),
    "lk_add_rmsnorm_q8_1": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _vp]),
    "lk_post_norm_add_norm_q8_1": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _i, _i, _vp]),
    "lk_split_act_mul_q8_1": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "lk_mmvq_pair_act_q8_1": (_i, [_i, _vp, _vp, _vp, _i, _i, _vp, _i, _i, _i, _i, _i, _vp]),
    "lkh_qkernel_matmul_new": (_vp, [_i, _i, _i, _vp, _i]),
    "lkh_qkernel_matmul_free": (None, [_vp]),
    "lkh_qkernel_matmul_forward": (_i, [_vp, _vp, _i, _i, _vp, _vp, _i]),
    "lkh_qkernel_matmul_last_path": (_i, [_vp]),
    "lkh_matvec_rows": (_i, [_i, _i]),
    "lkh_quantized_activation_bytes": (C.c_size_t, [_i, _i]),
    "lkh_qkernel_matmul_quantize_for_matvec": (_i, [_vp, _vp, _i, _i, _vp, _vp, _i]),
    "lkh_qkernel_matmul_forward_quantized": (_i, [_vp, _vp, _i, _i, _vp, _vp, _i]),
    "lkh_qkernel_matmul_forward_quantized_pair": (_i, [_vp, _vp, _vp, _vp, _vp, _vp]),
    "lkh_release_workspaces": (None, []),
    "lkh_gguf_open": (_vp, [_cp, _vp, _i]),
    "lkh_gguf_over": (_vp, [_vp, _u64, _vp, _i]),
    "lkh_gguf_close": (None, [_vp]),
    "lkh_gguf_layout": (_i, [_vp] * 6),
    "lkh_gguf_find_tensor": (_i, [_vp, _cp]),
    "lkh_gguf_tensor": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp]),
    "lkh_gguf_tensor_data": (_vp, [_vp, _i]),
    "lkh_gguf_find_key": (_i, [_vp, _cp]),
    "lkh_gguf_kv": (_i, [_vp, _i, _vp, _vp, _vp, _vp]),
    "lkh_gguf_kv_u64": (_i, [_vp, _i, _vp]),
    "lkh_gguf_kv_i64": (_i, [_vp, _i, _vp]),
    "lkh_gguf_kv_f64": (_i, [_vp, _i, _vp]),
    "lkh_gguf_kv_bool": (_i, [_vp, _i, _vp]),
    "lkh_gguf_kv_str": (_i, [_vp, _i, _vp, _vp]),
    "lkh_gguf_kv_item_u64": (_i, [_vp, _i, _u64, _vp]),
    "lkh_gguf_kv_item_i64": (_i, [_vp, _i, _u64, _vp]),
    "lkh_gguf_kv_item_f64": (_i, [_vp, _i, _u64, _vp]),
    "lkh_gguf_kv_item_str": (_i, [_vp, _i, _u64, _vp, _vp]),
    "lkh_gguf_facts": (_i, [_vp] * 6),
    "lkh_gguf_upload": (_vp, [_vp, _i, _i, _vp, _vp]),
    "lkh_gguf_free_blob": (None, [_vp]),
    "lkh_gguf_linear": (_vp, [_vp, _cp, _i, _vp, _vp, _vp, _i]),
    "loken_gate_topk_softmax": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "loken_topk_sigmoid_post": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _vp]),
    "loken_stable_sort_u32": (None, [_vp, _vp, _vp, _i, _vp]),
    "loken_argsort_small_u32": (None, [_vp, _vp, _vp, _i, _vp]),
    "loken_topk_softmax": (None, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "loken_dense_q4k_imma_m8_plain": (None, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "lk_dense_q4k_rows": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "loken_dense_q4k_imma_m8_actmul": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "lk_dense_q4k_rows_actmul": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "lk_dense_q4k_rows_multi": (_i, [_vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp]),
    "lk_mmvq_exact": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "lk_dense_q4k_rows_actmul_q8_1": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "loken_dense_q5k_imma_m8_plain": (None, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "lk_dense_q5k_rows": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "loken_dense_q5k_imma_m8_actmul": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "lk_dense_q5k_rows_actmul": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "q4k_mmvq_imma": (None, [_vp, _vp, _vp, _i, _i, _vp]),
    "lk_dense_q6k_rows": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "lk_moe_q4k_rows_grouped": (_i, [_vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, C.c_int64, _i, _i, _i, _vp]),
    "loken_moe_q4k_imma_m8_gate_up": (None, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "lk_moe_q4k_rows_gate_up": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "loken_moe_q4k_imma_m8_down": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "lk_tune_refresh": (None, []),
    "loken_moe_gemm_gguf_prefill": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "loken_rms_quantize_q8_1": (None, [_vp, _vp, _vp, _i, _f, _vp]),
    "loken_rms_quantize_q8_1_bf16": (None, [_vp, _vp, _vp, _i, _f, _vp]),
    "loken_moe_mmq_fold": (None, [_vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _vp]),
})

_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m loken_amd.build` (hipcc, gfx950)")
        lib = C.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(fn: str, code: int) -> None:
    if code != LK_OK:
        raise LokenError(fn, code)

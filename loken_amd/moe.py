"""Host side of the MoE expert block, mirroring loken's ``MmqRouting``
(src/inference/moe_cuda/mmq_experts.rs:108-736): group the routed pairs by expert, run gate and
up as one expert-batched launch, apply the GLU, run down scattered back to slot order, fold each
token's slots in slot order. torch holds the buffers; every computation is a C-ABI call.
"""
from __future__ import annotations

import math

import torch

from . import lib as _lib
from .ops import MMQ_DEVICE_INFO, _stream, mmq_quantize
from .synth import BLOCK_BYTES, BLOCK_LEN

MMQ_MOE_LAUNCHER = {_lib.TYPE_Q4_K: "launch_mmq_moe_gguf_q4_k", _lib.TYPE_Q5_K: "launch_mmq_moe_gguf_q5_k",
                    _lib.TYPE_Q6_K: "launch_mmq_moe_gguf_q6_k",
                    _lib.TYPE_Q8_0: "launch_mmq_moe_gguf_q8_0",
                    _lib.TYPE_Q4_0: "launch_mmq_moe_gguf_q4_0", _lib.TYPE_Q4_1: "launch_mmq_moe_gguf_q4_1",
                    _lib.TYPE_Q5_0: "launch_mmq_moe_gguf_q5_0", _lib.TYPE_Q5_1: "launch_mmq_moe_gguf_q5_1",
                    # the formats only mixtures store (quantized/mmq.rs:326-334)
                    _lib.TYPE_IQ4_NL: "launch_mmq_moe_gguf_iq4_nl", _lib.TYPE_MXFP4: "launch_mmq_moe_gguf_mxfp4",
                    _lib.TYPE_IQ4_XS: "launch_mmq_moe_gguf_iq4_xs",
                    # the codebook formats (quantized/mmq.rs:335-343)
                    _lib.TYPE_IQ3_XXS: "launch_mmq_moe_gguf_iq3_xxs", _lib.TYPE_IQ3_S: "launch_mmq_moe_gguf_iq3_s",
                    _lib.TYPE_IQ2_S: "launch_mmq_moe_gguf_iq2_s", _lib.TYPE_Q2_0: "launch_mmq_moe_gguf_q2_0",
                    _lib.TYPE_Q3_K: "launch_mmq_moe_gguf_q3_k", _lib.TYPE_Q2_K: "launch_mmq_moe_gguf_q2_k"}
MMQ_X_MIN, GRID_Y_MAX = 8, 65535


def moe_mmq_serves(wtype: int, k: int) -> bool:
    """mmq_experts.rs:90-92; the tile kernels here walk 256 values per step."""
    return wtype in MMQ_MOE_LAUNCHER and k % 256 == 0


class MmqRouting:
    """The routing in the form the expert-batched launches read it."""

    def __init__(self, tokens: int, topk: int, n_experts: int, device):
        rows = tokens * topk
        self.tokens, self.topk, self.experts = tokens, topk, n_experts
        self.bounds = torch.zeros(n_experts + 1, dtype=torch.int32, device=device)
        self.slots = torch.zeros(rows, dtype=torch.int32, device=device)
        self.src_rows = torch.zeros(rows, dtype=torch.int32, device=device)
        self.choices = None
        self.mmq_x = 0
        self.path = "auto"   # "tiled" / "rows" pin the launch family (measurement and tests)

    @classmethod
    def new(cls, slots: torch.Tensor, experts: torch.Tensor, topk: int, n_experts: int) -> "MmqRouting":
        """From the stably sorted routing (mmq_experts.rs:157-176)."""
        rows = slots.numel()
        if rows % topk:
            raise ValueError(f"moe mmq: {rows} routed rows is not a multiple of topk={topk}")
        plan = cls(rows // topk, topk, n_experts, slots.device)
        _lib.load().loken_moe_mmq_plan(experts.data_ptr(), slots.data_ptr(), rows, topk, n_experts,
                                       plan.bounds.data_ptr(), plan.slots.data_ptr(),
                                       plan.src_rows.data_ptr(), _stream())
        return plan

    @classmethod
    def from_choices(cls, choices: torch.Tensor, n_experts: int) -> "MmqRouting":
        """From the router's choices ``[tokens, topk]`` (mmq_experts.rs:183-206)."""
        tokens, topk = choices.shape
        choices = choices.to(torch.int32).contiguous()
        plan = cls(tokens, topk, n_experts, choices.device)
        counts = torch.zeros(n_experts, dtype=torch.int32, device=choices.device)
        _lib.load().loken_moe_mmq_route(choices.data_ptr(), tokens * topk, topk, n_experts, counts.data_ptr(),
                                        plan.bounds.data_ptr(), plan.slots.data_ptr(),
                                        plan.src_rows.data_ptr(), _stream())
        plan.choices = choices
        return plan

    def with_tile_width(self, mmq_x: int) -> "MmqRouting":
        self.mmq_x = mmq_x
        return self

    def with_path(self, path: str) -> "MmqRouting":
        if path not in ("auto", "tiled", "rows"):
            raise ValueError(f"moe mmq: unknown path {path!r}")
        self.path = path
        return self

    @property
    def rows(self) -> int:
        return self.tokens * self.topk

    def longest_run_expected(self) -> int:
        """mmq_experts.rs:215-227: mean + sqrt(2 ln experts) deviations of a binomial count."""
        experts = float(max(self.experts, 1))
        p = min(self.topk / experts, 1.0)
        mean = self.tokens * p
        dev = math.sqrt(mean * (1.0 - p))
        longest = mean + dev * math.sqrt(2.0 * math.log(experts)) if experts > 1 else mean
        return max(1, min(int(math.ceil(longest)), max(self.tokens, 1)))

    def _matmul(self, wtype: int, stack: torch.Tensor, second: torch.Tensor | None, second_offset: int,
                n: int, k: int, y: torch.Tensor, dst: torch.Tensor, stride: int, ids_dst: torch.Tensor | None):
        if not moe_mmq_serves(wtype, k):
            raise ValueError(f"moe mmq: no expert-batched kernel for type {wtype} at k={k}")
        blocks_per_row = k // BLOCK_LEN[wtype]
        expert_bytes = n * blocks_per_row * BLOCK_BYTES[wtype]
        longest = self.longest_run_expected()
        i = MMQ_DEVICE_INFO
        launched = getattr(_lib.load(), MMQ_MOE_LAUNCHER[wtype])(
            stack.data_ptr(), second.data_ptr() if second is not None else None, second_offset, y.data_ptr(),
            dst.data_ptr(), self.bounds.data_ptr(), ids_dst.data_ptr() if ids_dst is not None else None,
            expert_bytes, k, n, self.rows, blocks_per_row, stride, self.experts,
            min(longest, GRID_Y_MAX * MMQ_X_MIN), longest, self.mmq_x, i["cc"], i["smpbo"], i["warp_size"], _stream())
        if launched == 0:
            raise _lib.LokenError(MMQ_MOE_LAUNCHER[wtype], _lib.LK_ERR_ARG)

    # Rows an expert is expected to own up to which the matrix-unit rows launch (weights straight from
    # HBM into the operand, a wave per 16-row tile, a pass per 8, 16 or 48 rows) beats the tiled one
    # (weights expanded into LDS per 32 tokens). Measured on MI355X at 128 experts of 2048 -> 768 -> 2048,
    # top-8: 64 tokens 112 us against 173, 128 tokens 121 against 170, 256 tokens 159 against 183, 512
    # tokens 228 against 271, 1024 tokens 394 against 408, 1536 tokens 537 against 463 (the expected
    # longest run is 17 at 128 tokens, 29 at 256, 88 at 1024, 126 at 1536).
    ROWS_LAUNCH_MAX_RUN = 90

    def takes_rows_launch(self, wtype: int, k: int) -> bool:
        return (self.path != "tiled" and wtype == _lib.TYPE_Q4_K and k % 256 == 0
                and (self.path == "rows" or self.longest_run_expected() <= self.ROWS_LAUNCH_MAX_RUN))

    def _rows_launch(self, weights: torch.Tensor, second: torch.Tensor | None, q: torch.Tensor, src, dst_map,
                     out: torch.Tensor, n: int, k: int):
        expert_bytes = n * (k // 256) * 144
        _lib.check("lk_moe_q4k_rows_grouped", _lib.load().lk_moe_q4k_rows_grouped(
            weights.data_ptr(), second.data_ptr() if second is not None else None, 0, q.data_ptr(), q.shape[1],
            self.bounds.data_ptr(), src.data_ptr() if src is not None else None,
            dst_map.data_ptr() if dst_map is not None else None, out.data_ptr(), out.shape[1], self.experts,
            expert_bytes, n, k, self.longest_run_expected(), _stream()))

    def gate_up_silu(self, wtype: int, xs: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, width: int) -> torch.Tensor:
        """``silu(gate . x) * (up . x)`` for every routed row, in sorted order: ``[rows, width]``
        (mmq_experts.rs:300-435). ``gate`` / ``up`` are stacks of ``[experts, width, k]`` blocks."""
        tokens, k = xs.shape
        if tokens != self.tokens:
            raise ValueError(f"moe mmq: {tokens} tokens against a plan of {self.tokens}")
        if self.takes_rows_launch(wtype, k):
            # one Q8_1 row per token; a sorted row reads its token's; gate, up and the activation in one launch
            from . import ops
            q = ops.quantize_q8_1_rows(xs.to(torch.float32).contiguous(), k_padded=k)
            out = torch.empty((self.rows, width), dtype=torch.float32, device=xs.device)
            self._rows_launch(gate, up, q, self.src_rows, None, out, width, k)
            return out
        y = mmq_quantize(wtype, xs.to(torch.float32).contiguous(), gather=self.src_rows)
        gu = torch.empty((self.rows, 2 * width), dtype=torch.float32, device=xs.device)
        self._matmul(wtype, gate, up, width, width, k, y, gu, 2 * width, None)
        out = torch.empty((self.rows, width), dtype=torch.float32, device=xs.device)
        _lib.load().loken_moe_mmq_silu_mul(gu.data_ptr(), out.data_ptr(), self.rows, width, _stream())
        return out

    def down_fold(self, wtype: int, hs: torch.Tensor, down: torch.Tensor, hidden: int, topk_weights: torch.Tensor,
                  residual: torch.Tensor | None = None) -> torch.Tensor:
        """Down projection of the sorted rows ``hs`` ``[rows, k]``, each scaled by its router
        weight and folded into its token in slot order: ``[tokens, hidden]`` (mmq_experts.rs:440-557)."""
        rows, k = hs.shape
        if rows != self.rows:
            raise ValueError(f"moe mmq: {rows} rows against a plan of {self.rows}")
        pairs = torch.empty((rows, hidden), dtype=torch.float32, device=hs.device)
        if self.takes_rows_launch(wtype, k):
            from . import ops
            q = ops.quantize_q8_1_rows(hs.contiguous(), k_padded=k)
            self._rows_launch(down, None, q, None, self.slots, pairs, hidden, k)
        else:
            y = mmq_quantize(wtype, hs.contiguous())
            self._matmul(wtype, down, None, 0, hidden, k, y, pairs, hidden, self.slots)
        out = (residual.reshape(self.tokens, hidden).to(torch.float32).clone() if residual is not None
               else torch.zeros((self.tokens, hidden), dtype=torch.float32, device=hs.device))
        w = topk_weights.to(torch.float32).contiguous()
        if w.numel() != rows:
            raise ValueError(f"moe mmq: {w.numel()} router weights for {rows} rows")
        _lib.load().loken_moe_mmq_fold(pairs.data_ptr(), w.data_ptr(), None, None, out.data_ptr(), self.tokens,
                                       self.topk, hidden, _stream())
        return out


# ------------------------------------------------------------------------------------ decode
# loken's wire ids for the MoE decode launchers (EXPERT_QUANT_CODES, cuda/moe/gguf.cuh:55-71)
EXPERT_QUANT_CODES = {_lib.TYPE_Q8_0: 0, _lib.TYPE_Q4_K: 1, _lib.TYPE_Q2_K: 2, _lib.TYPE_Q3_K: 3, _lib.TYPE_Q5_K: 4,
                      _lib.TYPE_Q6_K: 5, _lib.TYPE_Q5_0: 6, _lib.TYPE_MXFP4: 7, _lib.TYPE_Q5_1: 8, _lib.TYPE_IQ4_NL: 9,
                      _lib.TYPE_IQ4_XS: 10, _lib.TYPE_IQ3_XXS: 11, _lib.TYPE_IQ3_S: 12, _lib.TYPE_IQ2_S: 13, _lib.TYPE_Q2_0: 14,
                      _lib.TYPE_IQ2_XXS: 15}


class ExpertRouting:
    """The routing grouped by expert: a stable sort of the flattened (token, choice) slots by
    expert id (ExpertRouting::group, src/inference/generic_transformer/moe_weights.rs:27-54,102-116)."""

    def __init__(self, choices: torch.Tensor):
        flat = choices.reshape(-1).to(torch.int64)
        order = torch.sort(flat, stable=True).indices
        self.sorted_token_ids = order.to(torch.int32).contiguous()
        self.expert_ids = flat[order].to(torch.int32).contiguous()
        self.tokens, self.topk = choices.shape


def moe_gemm_gguf_gate_up_silu_mul(wtype: int, x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
                                   routing: ExpertRouting, n_experts: int, ffn: int) -> torch.Tensor:
    """``[tokens, k]`` -> ``[tokens * topk, ffn]`` in SLOT order (src/inference/moe_cuda/gemm.rs:285-302)."""
    tokens, k = x.shape
    pairs = tokens * routing.topk
    out = torch.empty((pairs, ffn), dtype=torch.float32, device=x.device)
    _lib.check("loken_moe_gemm_gguf_gate_up_silu_mul", _lib.load().loken_moe_gemm_gguf_gate_up_silu_mul(
        x.data_ptr(), gate.data_ptr(), up.data_ptr(), routing.sorted_token_ids.data_ptr(),
        routing.expert_ids.data_ptr(), out.data_ptr(), n_experts, routing.topk, pairs, ffn, k,
        EXPERT_QUANT_CODES[wtype], _stream()))
    return out


def moe_gemm_gguf_gate_up_swiglu_oai(wtype: int, x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
                                     routing: ExpertRouting, n_experts: int, n: int, alpha: float, limit: float,
                                     gate_bias: torch.Tensor | None = None,
                                     up_bias: torch.Tensor | None = None) -> torch.Tensor:
    """gpt-oss's clamped SwiGLU with per-expert biases in the gated launch
    (src/inference/moe_cuda/gemm.rs:596-651)."""
    k = x.shape[1]
    pairs = routing.tokens * routing.topk
    out = torch.empty((pairs, n), dtype=torch.float32, device=x.device)
    _lib.check("loken_moe_gemm_gguf_gate_up_swiglu_oai", _lib.load().loken_moe_gemm_gguf_gate_up_swiglu_oai(
        x.data_ptr(), gate.data_ptr(), up.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        gate_bias.data_ptr() if gate_bias is not None else None, up_bias.data_ptr() if up_bias is not None else None,
        out.data_ptr(), n_experts, routing.topk, pairs, n, k, EXPERT_QUANT_CODES[wtype], alpha, limit, _stream()))
    return out


def moe_gemm_gguf_gate_up_swiglu_limited(wtype: int, x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
                                         routing: ExpertRouting, n_experts: int, n: int, limit: float) -> torch.Tensor:
    """The bounded SwiGLU (src/inference/moe_cuda/gemm.rs:656-704)."""
    k = x.shape[1]
    pairs = routing.tokens * routing.topk
    out = torch.empty((pairs, n), dtype=torch.float32, device=x.device)
    _lib.check("loken_moe_gemm_gguf_gate_up_swiglu_limited", _lib.load().loken_moe_gemm_gguf_gate_up_swiglu_limited(
        x.data_ptr(), gate.data_ptr(), up.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        out.data_ptr(), n_experts, routing.topk, pairs, n, k, EXPERT_QUANT_CODES[wtype], limit, _stream()))
    return out


def moe_gemm_gguf_gate_up_gelu_mul_concat(wtype: int, x: torch.Tensor, gate_up: torch.Tensor, routing: ExpertRouting,
                                          n_experts: int, n: int) -> torch.Tensor:
    """gelu(gate) * up over one ``[experts, 2 n, k]`` tensor, an expert's gate rows then its up rows
    (src/inference/moe_cuda/gemm.rs:706-747)."""
    k = x.shape[1]
    pairs = routing.tokens * routing.topk
    out = torch.empty((pairs, n), dtype=torch.float32, device=x.device)
    _lib.check("loken_moe_gemm_gguf_gate_up_gelu_mul_concat", _lib.load().loken_moe_gemm_gguf_gate_up_gelu_mul_concat(
        x.data_ptr(), gate_up.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        out.data_ptr(), n_experts, routing.topk, pairs, n, k, EXPERT_QUANT_CODES[wtype], _stream()))
    return out


def moe_gemm_gguf_gate_up_silu_mul_live(wtype: int, x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
                                        routing: ExpertRouting, n_experts: int, n: int, live: torch.Tensor,
                                        out: torch.Tensor | None = None) -> torch.Tensor:
    """The gated launch over the first ``live[0]`` routed pairs (a uint32 on the card); the other
    pairs' rows of ``out`` keep what they held (src/inference/moe_cuda/gemm.rs:424-474)."""
    k = x.shape[1]
    pairs = routing.tokens * routing.topk
    if out is None:
        out = torch.zeros((pairs, n), dtype=torch.float32, device=x.device)
    _lib.check("loken_moe_gemm_gguf_gate_up_silu_mul_live", _lib.load().loken_moe_gemm_gguf_gate_up_silu_mul_live(
        x.data_ptr(), gate.data_ptr(), up.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        out.data_ptr(), n_experts, routing.topk, pairs, n, k, EXPERT_QUANT_CODES[wtype], live.data_ptr(), _stream()))
    return out


def moe_gemm_gguf_down_pairs_live(wtype: int, h: torch.Tensor, down: torch.Tensor, routing: ExpertRouting,
                                  topk_weights: torch.Tensor, n_experts: int, hidden: int,
                                  live: torch.Tensor) -> torch.Tensor:
    """Each of the first ``live[0]`` routed pairs' down rows at its weight, ``[pairs, hidden]`` in slot
    order, zero rows for the rest (src/inference/moe_cuda/gemm.rs:550-590)."""
    pairs, k = h.shape
    out = torch.empty((pairs, hidden), dtype=torch.float32, device=h.device)
    _lib.check("loken_moe_gemm_gguf_down_pairs_live", _lib.load().loken_moe_gemm_gguf_down_pairs_live(
        h.data_ptr(), down.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        topk_weights.data_ptr(), out.data_ptr(), n_experts, routing.topk, pairs, hidden, k, EXPERT_QUANT_CODES[wtype],
        live.data_ptr(), _stream()))
    return out


def moe_gemm_gguf_gate_up_silu_mul_over(wtype: int, x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
                                        more_gate: torch.Tensor, more_up: torch.Tensor, more_from: int,
                                        routing: ExpertRouting, n_experts: int, n: int,
                                        more_at: torch.Tensor | None = None) -> torch.Tensor:
    """The gated launch with the experts from ``more_from`` on in a second pair of tensors; ``more_at``
    (two int64 addresses on the card) names them at run time instead
    (src/inference/moe_cuda/gemm.rs:319-419)."""
    k = x.shape[1]
    pairs = routing.tokens * routing.topk
    out = torch.empty((pairs, n), dtype=torch.float32, device=x.device)
    _lib.check("loken_moe_gemm_gguf_gate_up_silu_mul_two", _lib.load().loken_moe_gemm_gguf_gate_up_silu_mul_two(
        x.data_ptr(), gate.data_ptr(), up.data_ptr(), more_gate.data_ptr(), more_up.data_ptr(), more_from,
        more_at.data_ptr() if more_at is not None else None, routing.sorted_token_ids.data_ptr(),
        routing.expert_ids.data_ptr(), out.data_ptr(), n_experts, routing.topk, pairs, n, k, EXPERT_QUANT_CODES[wtype],
        _stream()))
    return out


def moe_gemm_gguf_down_reduce_over(wtype: int, h: torch.Tensor, down: torch.Tensor, more_down: torch.Tensor,
                                   more_from: int, routing: ExpertRouting, topk_weights: torch.Tensor, n_experts: int,
                                   hidden: int, down_bias: torch.Tensor | None = None) -> torch.Tensor:
    """Down + fold with the experts from ``more_from`` on in a second tensor
    (src/inference/moe_cuda/gemm.rs:778-...)."""
    pairs, k = h.shape
    out = torch.zeros((pairs // routing.topk, hidden), dtype=torch.float32, device=h.device)
    _lib.check("loken_moe_gemm_gguf_down_reduce_two", _lib.load().loken_moe_gemm_gguf_down_reduce_two(
        h.data_ptr(), down.data_ptr(), more_down.data_ptr(), more_from, routing.sorted_token_ids.data_ptr(),
        routing.expert_ids.data_ptr(), topk_weights.data_ptr(), out.data_ptr(), n_experts, routing.topk, pairs, hidden, k,
        EXPERT_QUANT_CODES[wtype], down_bias.data_ptr() if down_bias is not None else None, None, _stream()))
    return out


def moe_gemm_gguf_down_pairs_over(wtype: int, h: torch.Tensor, down: torch.Tensor, more_down: torch.Tensor,
                                  more_from: int, routing: ExpertRouting, topk_weights: torch.Tensor, n_experts: int,
                                  hidden: int, more_at: torch.Tensor | None = None) -> torch.Tensor:
    """The same up to the pairs' weighted rows, ``[pairs, hidden]`` (src/inference/moe_cuda/gemm.rs:479-545)."""
    pairs, k = h.shape
    out = torch.empty((pairs, hidden), dtype=torch.float32, device=h.device)
    _lib.check("loken_moe_gemm_gguf_down_pairs_two", _lib.load().loken_moe_gemm_gguf_down_pairs_two(
        h.data_ptr(), down.data_ptr(), more_down.data_ptr(), more_from,
        more_at.data_ptr() if more_at is not None else None, routing.sorted_token_ids.data_ptr(),
        routing.expert_ids.data_ptr(), topk_weights.data_ptr(), out.data_ptr(), n_experts, routing.topk, pairs, hidden, k,
        EXPERT_QUANT_CODES[wtype], _stream()))
    return out


def moe_gemm_gguf_down_reduce(wtype: int, h: torch.Tensor, down: torch.Tensor, routing: ExpertRouting,
                              topk_weights: torch.Tensor, n_experts: int, hidden: int,
                              residual: torch.Tensor | None = None, down_bias: torch.Tensor | None = None,
                              add_after: torch.Tensor | None = None) -> torch.Tensor:
    """``[tokens * topk, k]`` in slot order -> ``[tokens, hidden]`` (src/inference/moe_cuda/mod.rs:437-441)."""
    pairs, k = h.shape
    tokens = pairs // routing.topk
    if residual is not None:
        out = residual.to(torch.float32).clone()
    elif add_after is not None:   # the sum is written, not added to what `out` holds
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=h.device)
    else:
        out = torch.zeros((tokens, hidden), dtype=torch.float32, device=h.device)
    w = topk_weights.to(torch.float32).contiguous()
    _lib.check("loken_moe_gemm_gguf_down_reduce", _lib.load().loken_moe_gemm_gguf_down_reduce(
        h.data_ptr(), down.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        w.data_ptr(), out.data_ptr(), n_experts, routing.topk, pairs, hidden, k, EXPERT_QUANT_CODES[wtype],
        down_bias.data_ptr() if down_bias is not None else None,
        add_after.data_ptr() if add_after is not None else None, _stream()))
    return out


def moe_gemm_gguf(wtype: int, x: torch.Tensor, weights: torch.Tensor, routing: ExpertRouting, n_experts: int, n: int,
                  topk_weights: torch.Tensor | None = None) -> torch.Tensor:
    """One routed product per pair, rows in slot order (src/inference/moe_cuda/gemm.rs:18-...)."""
    k = x.shape[1]
    pairs = routing.tokens * routing.topk
    out = torch.empty((pairs, n), dtype=torch.float32, device=x.device)
    _lib.check("loken_moe_gemm_gguf", _lib.load().loken_moe_gemm_gguf(
        x.data_ptr(), weights.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        topk_weights.data_ptr() if topk_weights is not None else None, out.data_ptr(), n_experts, routing.topk,
        pairs, n, k, EXPERT_QUANT_CODES[wtype], _stream()))
    return out


def moe_gemm_gguf_prefill(wtype: int, x: torch.Tensor, weights: torch.Tensor, routing: ExpertRouting, n_experts: int,
                          n: int, topk_weights: torch.Tensor | None = None) -> torch.Tensor:
    """The same product from f16 / bf16 activation rows: what moe_gemm_gguf calls for a prefill on a card
    with matrix instructions (src/inference/moe_cuda/gemm.rs:221-258)."""
    k = x.shape[1]
    pairs = routing.tokens * routing.topk
    out = torch.empty((pairs, n), dtype=torch.float32, device=x.device)
    input_dtype = {torch.float16: 0, torch.bfloat16: 1}[x.dtype]
    _lib.check("loken_moe_gemm_gguf_prefill", _lib.load().loken_moe_gemm_gguf_prefill(
        x.data_ptr(), weights.data_ptr(), routing.sorted_token_ids.data_ptr(), routing.expert_ids.data_ptr(),
        topk_weights.data_ptr() if topk_weights is not None else None, out.data_ptr(), n_experts, routing.topk,
        pairs, n, k, input_dtype, EXPERT_QUANT_CODES[wtype], _stream()))
    return out


def topk_softmax(logits: torch.Tensor, topk: int, renorm: bool = True):
    """Router: ``[tokens, experts]`` f32 logits -> (weights f32 ``[tokens, topk]``, choices int32
    ``[tokens, topk]``), probabilities descending, ties to the lower expert id (topk_softmax,
    src/inference/moe_cuda_cpu/mod.rs:2098-2113)."""
    tokens, experts = logits.shape
    if experts > 512 or topk > 64 or topk > experts:
        raise ValueError("topk_softmax: at most 512 experts and 64 choices")
    logits = logits.to(torch.float32).contiguous()
    weights = torch.empty((tokens, topk), dtype=torch.float32, device=logits.device)
    ids = torch.empty((tokens, topk), dtype=torch.int32, device=logits.device)
    _lib.load().loken_topk_softmax(logits.data_ptr(), weights.data_ptr(), ids.data_ptr(), tokens, experts, topk,
                                   int(renorm), _stream())
    return weights, ids


def _router_out(tokens: int, topk: int, device):
    return (torch.empty((tokens, topk), dtype=torch.float32, device=device),
            torch.empty((tokens, topk), dtype=torch.int32, device=device))


def gate_topk_softmax(x: torch.Tensor, gate_w: torch.Tensor, topk: int, renorm: bool = True):
    """Gate mat-vec + softmax + top-k in one launch: ``x [tokens, hidden]`` f32, ``gate_w [experts,
    hidden]`` f32 -> (weights, choices) as ``topk_softmax`` (gate_topk_softmax,
    src/inference/moe_cuda/dense/gate.rs:20-75)."""
    tokens, hidden = x.shape
    experts = gate_w.shape[0]
    if hidden > 8192 or experts > 512 or topk > 64 or topk > experts or gate_w.shape[1] != hidden:
        raise ValueError("gate_topk_softmax: hidden <= 8192, at most 512 experts and 64 choices")
    weights, ids = _router_out(tokens, topk, x.device)
    _lib.load().loken_gate_topk_softmax(x.data_ptr(), gate_w.data_ptr(), weights.data_ptr(), ids.data_ptr(), hidden,
                                        tokens, experts, topk, int(renorm), _stream())
    return weights, ids


def topk_sigmoid_post(logits: torch.Tensor, topk: int, bias: torch.Tensor | None = None, renorm: bool = True,
                      scale: float = 1.0):
    """Sigmoid router: chosen on probability + bias, weighted by the probability alone
    (topk_sigmoid_post, src/inference/moe_cuda/dense/gate.rs:100-160)."""
    tokens, experts = logits.shape
    if experts > 512 or topk > 64 or topk > experts:
        raise ValueError("topk_sigmoid_post: at most 512 experts and 64 choices")
    weights, ids = _router_out(tokens, topk, logits.device)
    _lib.load().loken_topk_sigmoid_post(logits.data_ptr(), bias.data_ptr() if bias is not None else None,
                                        weights.data_ptr(), ids.data_ptr(), tokens, experts, topk, int(renorm), scale,
                                        _stream())
    return weights, ids


def stable_sort_u32(keys: torch.Tensor, small: bool = False):
    """-> (sorted keys, the index each came from), equal keys in their original order
    (loken_stable_sort_u32 / loken_argsort_small_u32, src/inference/moe_cuda/routing.rs:200-242)."""
    n = keys.numel()
    if small and n > 256:
        raise ValueError("argsort_small: at most 256 keys")
    out, order = torch.empty_like(keys), torch.empty_like(keys)
    fn = _lib.load().loken_argsort_small_u32 if small else _lib.load().loken_stable_sort_u32
    fn(keys.data_ptr(), out.data_ptr(), order.data_ptr(), n, _stream())
    return out, order


def moe_mmq_pays(rows: int, experts: int, wtype: int | None = None) -> bool:
    """Routed rows from which the expert-batched launches beat the per-pair kernels. The reference
    breaks even at one routed row per expert (mmq_experts.rs:72-86); on MI355X, with this
    library's kernels, the mat-vec per routed pair stays ahead of the tiled matmul up to three rows
    per expert (Qwen3-30B-A3B shapes: 117 us against 162 us at 32 tokens, 176 against 168 at 48), and
    of the matrix-unit rows launch that Q4_K stacks take at short runs up to 1.625 (per block inside
    a step's graph, 16 tokens: 51 us against 74; 24: 81 against 83; 32: 92 against 88; 48: 139
    against 106)."""
    if wtype == _lib.TYPE_Q4_K:
        return 8 * rows >= 13 * max(experts, 1)
    return rows >= 3 * max(experts, 1)


def moe_forward(wtype_gu: int, wtype_down: int, x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
                down: torch.Tensor, choices: torch.Tensor, topk_weights: torch.Tensor, n_experts: int,
                ffn: int, return_rows: bool = False):
    """The expert block of one layer, path chosen as the reference's layer code chooses it
    (src/inference/generic_transformer/moe_weights.rs:2118-2152): the expert-batched tiled
    matmuls when there is at least a routed row per expert, else one mat-vec per routed pair.
    `return_rows`: also the gated rows the second product read, in slot order (token * topk + choice)."""
    tokens, hidden = x.shape
    topk = choices.shape[1]
    if (moe_mmq_pays(tokens * topk, n_experts, wtype_gu if wtype_gu == wtype_down else None)
            and moe_mmq_serves(wtype_gu, hidden) and moe_mmq_serves(wtype_down, ffn)):
        plan = MmqRouting.from_choices(choices, n_experts)
        h = plan.gate_up_silu(wtype_gu, x, gate, up, ffn)
        out = plan.down_fold(wtype_down, h, down, hidden, topk_weights.reshape(-1))
        if not return_rows:
            return out
        rows = torch.empty_like(h)
        rows[plan.slots.long()] = h   # sorted order -> slot order
        return out, rows
    routing = ExpertRouting(choices)
    h = moe_gemm_gguf_gate_up_silu_mul(wtype_gu, x.contiguous(), gate, up, routing, n_experts, ffn)
    out = moe_gemm_gguf_down_reduce(wtype_down, h, down, routing, topk_weights.reshape(-1), n_experts, hidden)
    return (out, h) if return_rows else out


def moe_q4k_imma_m8_gate_up(x: torch.Tensor, gate_up: torch.Tensor, sorted_token_ids: torch.Tensor,
                            expert_of_pair: torch.Tensor, n_experts: int, topk: int, n: int) -> torch.Tensor:
    """``gelu(gate . x) * (up . x)`` per routed pair over Q8_1 rows quantized here, one expert id
    per pair, ``[tokens * topk, n]`` in slot order, zero where a pair's expert is out of range
    (moe_q4k_imma_m8_gate_up, src/inference/moe_cuda/dense/imma.rs:140-190)."""
    from . import ops
    tokens, k = x.shape
    pairs = tokens * topk
    q = ops.quantize_q8_1_rows(x, k_padded=k)
    out = torch.zeros((pairs, n), dtype=torch.float32, device=x.device)
    _lib.check("lk_moe_q4k_rows_gate_up", _lib.load().lk_moe_q4k_rows_gate_up(
        gate_up.data_ptr(), q.data_ptr(), sorted_token_ids.data_ptr(), expert_of_pair.data_ptr(), out.data_ptr(),
        n_experts, topk, pairs, n, k, _stream()))
    return out


def moe_q4k_imma_m8_down_reduce(h: torch.Tensor, down: torch.Tensor, sorted_token_ids: torch.Tensor,
                                expert_of_pair: torch.Tensor, topk_weights: torch.Tensor, n_experts: int, topk: int,
                                hidden: int) -> torch.Tensor:
    """Down over one Q8_1 row per routed pair (quantized here, at the pair's slot), weighted and
    folded into ``[tokens, hidden]`` (moe_q4k_imma_m8_down_reduce, src/inference/moe_cuda/dense/imma.rs:
    200-300)."""
    from . import ops
    pairs, k = h.shape
    q = ops.quantize_q8_1_rows(h, k_padded=k)
    out = torch.zeros((pairs // topk, hidden), dtype=torch.float32, device=h.device)
    _lib.check("loken_moe_q4k_imma_m8_down", _lib.load().loken_moe_q4k_imma_m8_down(
        down.data_ptr(), q.data_ptr(), sorted_token_ids.data_ptr(), expert_of_pair.data_ptr(),
        topk_weights.data_ptr(), out.data_ptr(), n_experts, topk, pairs, hidden, k, _stream()))
    return out

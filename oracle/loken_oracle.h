/*
 * CPU oracle for the GGUF block-quantized matmul path. TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of loken's CPU quantized-matmul path (Rust, under
 * src/tensor/quant_cpu and src/inference/moe_cuda_cpu of the reference). Nothing in the
 * shipped library links, loads or calls this file: only the test-suite, the smoke check and
 * the CPU-baseline leg of the benchmark do, and there only as the checker.
 *
 * Two families of entry points:
 *   oa_*  "as served": K-quant weights against Q8_K activations (256 values, f32 scale,
 *         bsums), Q8_0 weights against Q8_0 activations. This is what loken's CPU backend
 *         runs (format/q4_k.rs:62-88, q6_k.rs:51-82, q8_0.rs:83-97, drivers.rs:2108-2142).
 *   ob_*  "same codes": the activation is quantized by loken's BlockQ8_1::quantize
 *         (format/q8_1.rs:46-61), the integer sub-block dots are the inner `dot` of
 *         q4_k.rs:138-153 / q6_k.rs:137-160 / q8_0.rs:88-95 taken per Q8_1 block, and the f32
 *         combine is the one a Q8_1-activation kernel performs (cuda/moe/gguf.cuh:664-685,
 *         782-816, 486-495). The GPU kernels are compared bit-for-bit on the integers and to
 *         1e-3 relative / 1e-4 absolute on the f32 outputs against this family.
 *
 * Pinned by (see tests/test_oracle_*.py): ggml's own QUANT/DEQUANT records for q4_K, q6_K,
 * q8_0, q8_K (scripts/oracle/vectors.txt) and ggml-written blocks with their decoded rows
 * (tests/vectors/ggml_encode.json) for layouts, f16 conversion and dequantizers; exhaustive
 * pack/unpack round-trip for the 6-bit scales; closed forms for the three activation
 * quantizers; numpy int64 brute force for every integer sum; an f64 dot over dequantized
 * values and the reduction to a plain int8 GEMV for the f32 combines; decomposition into
 * single-matrix calls for the MoE routines; a textbook softmax/top-k for the router; for the
 * served Q4_K path of cpu_baseline.c (eight-row repack, group dot, persistent pool:
 * tests/test_oracle_served_cpu_path.py) the reference's index map byte by byte, the exact integer
 * combination of the scalar definition on crafted inputs, the reference's own vector-vs-scalar
 * bound on random ones, and the same bits whatever the pool size. No function is parity unpinned.
 */
#ifndef LOKEN_ORACLE_H
#define LOKEN_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids, src/tensor/quantized/dtype.rs:66-96 */
enum { LKO_Q4_0 = 2, LKO_Q4_1 = 3, LKO_Q5_0 = 6, LKO_Q5_1 = 7, LKO_Q8_0 = 8, LKO_Q8_1 = 9, LKO_Q2_K = 10, LKO_Q3_K = 11,
       LKO_Q4_K = 12, LKO_Q5_K = 13,
       LKO_Q6_K = 14, LKO_Q8_K = 15, LKO_IQ4_NL = 20, LKO_IQ4_XS = 23, LKO_MXFP4 = 39 };

#define LKO_QK_K 256
#define LKO_Q4K_BYTES 144
#define LKO_Q5K_BYTES 176
#define LKO_Q6K_BYTES 210
#define LKO_Q80_BYTES 34
#define LKO_Q81_BYTES 36
#define LKO_Q8K_BYTES 292

/* ---- scalar helpers ---- */
float    lko_f16_to_f32(uint16_t h);
uint16_t lko_f32_to_f16(float f);            /* IEEE round-to-nearest-even, as the `half` crate */
int      lko_block_len(int dtype);           /* values per block, 0 if not handled */
int      lko_block_bytes(int dtype);         /* bytes per block, 0 if not handled */

/* blocks.rs:145-158 / 167-179 */
void lko_unpack_scales_mins(const uint8_t packed[12], uint8_t scales[8], uint8_t mins[8]);
void lko_pack_scales_mins(const uint8_t scales[8], const uint8_t mins[8], uint8_t packed[12]);

/* ---- dequantizers (pin the layouts) ---- */
int lko_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out);

/* ---- activation quantizers ---- */
void lko_quantize_q8_0(const float* x, size_t n, uint8_t* out);   /* q8_0.rs:51-67 */
void lko_quantize_q8_1(const float* x, size_t n, uint8_t* out);   /* q8_1.rs:46-61 */
void lko_quantize_q8_k(const float* x, size_t n, uint8_t* out);   /* q8_k.rs:96-119 */

/* ---- O-A: the served CPU path ---- */
/* dst[m,n] = lhs[m,k] (f32) x rhs[n, k/blk] blocks. Returns 0, or a negative code with the
 * reference's error conditions (drivers.rs:2122-2139): -1 k not a multiple of the block,
 * -2 rhs byte length wrong, -3 dtype not handled. */
int oa_matmul(int dtype, size_t m, size_t k, size_t n, const float* lhs,
              const uint8_t* rhs, size_t rhs_bytes, float* dst);
/* matmul_bytes_multi (drivers.rs:2144-2316): expert e's one row lhs[e] [k] x rhs[e] [n, k/blk] ->
 * outs[e] [n]; bit for bit one oa_matmul((1,k,n)) per expert. Further codes: -4 an lhs entry is not
 * k floats, -5 an outs entry is not n floats. ne == 0 is a no-op. */
int oa_matmul_multi(int dtype, size_t k, size_t n, size_t ne, const uint8_t* const* rhs, const size_t* rhs_bytes,
                    const float* const* lhs, const size_t* lhs_len, float* const* outs, const size_t* outs_len);
/* matmul_bytes_grouped (drivers.rs:2318-2425): expert e's lhs_len[e] / k rows x rhs[e] -> outs[e]
 * [rows, n]; bit for bit one GEMV per (expert, row). -4: an lhs entry is not whole rows of k; -5: an
 * outs entry is not rows x n. */
int oa_matmul_grouped(int dtype, size_t k, size_t n, size_t ne, const uint8_t* const* rhs, const size_t* rhs_bytes,
                      const float* const* lhs, const size_t* lhs_len, float* const* outs, const size_t* outs_len);
/* The exact-fold variant, dot_exact (q4_k.rs:117-131, q6_k.rs:121-134): integer block sums,
 * `combine`, shares added in block order from -0.0. K-quants only. */
int oa_matmul_exact(int dtype, size_t m, size_t k, size_t n, const float* lhs,
                    const uint8_t* rhs, float* dst);

/* ---- O-B: same-codes path ---- */
/* Integer sub-block dots of one weight row set against ONE Q8_1 activation row.
 *   Q4_K: dots[n][k/32] = sum_32 nibble*q8 ; sums[k/32] = sum_32 q8 (weight independent)
 *   Q6_K: dots[n][k/16] = sum_16 (code-32)*q8
 *   Q8_0: dots[n][k/32] = sum_32 q*q8
 * `act_q8_1` is k/32 Q8_1 blocks. `sums` may be NULL. */
int ob_subdots(int dtype, size_t k, size_t n, const uint8_t* rhs, const uint8_t* act_q8_1,
               int32_t* dots, int32_t* sums);
/* dst[m,n] from Q8_1 activation rows (m rows of k/32 blocks, row stride `act_stride_blocks`). */
int ob_matmul_q8_1(int dtype, size_t m, size_t k, size_t n, const uint8_t* act_q8_1,
                   size_t act_stride_blocks, const uint8_t* rhs, float* dst);
/* Same, quantizing lhs[m,k] f32 first with lko_quantize_q8_1. */
int ob_matmul(int dtype, size_t m, size_t k, size_t n, const float* lhs,
              const uint8_t* rhs, float* dst);
/* f64 evaluation of the same-codes product: sum over dequantized weight x dequantized Q8_1. */
int ob_matmul_f64(int dtype, size_t m, size_t k, size_t n, const float* lhs,
                  const uint8_t* rhs, double* dst);

/* ---- router and MoE ---- */
/* softmax -> top-k by value descending (ties: lower index first) -> optional renormalize.
 * moe_cuda_cpu/mod.rs:2098-2113. ids[t,topk], weights[t,topk]. */
void lko_topk_softmax(const float* logits, size_t tokens, size_t n_experts, size_t topk,
                      int renorm, int32_t* ids, float* weights);
/* Sigmoid router (cuda/moe/gate_topk.cu:140-200, 329-364): p = 1 / (1 + exp(-logit)); top-k on
 * p + bias (bias nullable; ties: lower index first); weights = p of the chosen, divided by
 * max(sum, 2^-14) if renorm, times scale. */
void lko_topk_sigmoid(const float* logits, const float* bias, size_t tokens, size_t n_experts, size_t topk,
                      int renorm, float scale, int32_t* ids, float* weights);
/* Stable sort of the flattened (token, choice) slots by expert id:
 * sorted_slots[i], sorted_experts[i] (generic_transformer/moe_weights.rs:27-54,102-116). */
void lko_group_by_expert(const int32_t* ids, size_t pairs, int32_t* sorted_slots,
                         int32_t* sorted_experts);
/* Whole expert block, host semantics of fused_gate_up_silu_cpu + fused_down_reduce_cpu
 * (moe_cuda_cpu/mod.rs:459-605, 1478-1660): x[tokens,hidden] -> out[tokens,hidden].
 * gate/up: [experts, ffn, hidden/blk], down: [experts, hidden, ffn/blk]; `family` 0 = O-A
 * activations (Q8_K / Q8_0), 1 = O-B (Q8_1). SiLU is u*(g/(1+exp(-g))); the fold adds
 * tw[slot]*dot into the token row in expert-run order. `h_sorted` (pairs x ffn, sorted order)
 * may be NULL. */
int lko_moe_forward(int family, int dtype_gate_up, int dtype_down, size_t tokens, size_t hidden,
                    size_t ffn, size_t n_experts, size_t topk, const float* x,
                    const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                    const int32_t* ids, const float* weights, float* h_sorted, float* out);

/* ---- decode-step producers that end in a Q8_1 row (src/inference/cuda/mmvq_gguf.cu:789-999) ---- */
/* 1 / sqrt(mean of squares + eps) as the wide norm kernels accumulate it (:811-829): lane t of 256
 * folds the squares of values t, t + 256, ... with a fused multiply-add, the 256 partial sums fold
 * as a stride-halving tree. The reciprocal square root is 1 / sqrtf, both correctly rounded (the
 * reference's rsqrtf approximation has no portable bits). */
float lko_inv_rms_wide(const float* row, size_t cols, float eps);
/* mode 0: out = (x * rms) * w (:805-837). mode 1: mid = x + residual, out = rmsnorm(mid, w)
 * (:839-877). mode 2: mid = (x * rms_first) * w_first + residual, each product rounded before it
 * is added; out = rmsnorm(mid, w) (:879-936). rows x cols; unused pointers may be NULL. */
void lko_norm_rows(int mode, const float* x, const float* w_first, const float* residual, const float* w,
                   float* mid, float* out, float eps_first, float eps, size_t cols, size_t rows);
/* out[r, i] = act(gu[r, i]) * gu[r, n + i]; act 0 = g / (1 + exp(-g)), 1 = tanh-GELU (:971-999). */
void lko_split_act_mul(const float* gu, float* out, size_t n, size_t rows, int act);

/* ---- timed CPU baseline (cpu_baseline.c): O-A semantics, AVX2 kernels, worker pool ---- */
int lko_cpu_has_avx2(void);
int lko_cpu_has_avx512(void);   /* f, bw, vl, dq and vnni */
/* The vector dots of one Q4_K row (nb super-blocks) against Q8_K rows, for the tests: the 256-bit
 * kernel (wide = 0; avx/superblock.rs:327-350) or its 512-bit VNNI twin (wide = 1;
 * avx512/superblock.rs:20-90), and the several-rows-per-pass form (avx/superblock.rs:425-490), each of
 * whose outputs carries the bits of the one-row kernel. Call only where lko_cpu_has_avx2 /
 * lko_cpu_has_avx512 say so. */
float lko_dot_q4k_q8k(int wide, const uint8_t* w, const uint8_t* y, size_t nb);
void lko_dot_q4k_q8k_many(const uint8_t* w, const uint8_t* const* ys, size_t rows, size_t nb, float* out);
/* The worker pool both drivers run on: persistent, one worker per physical core of the affinity
 * mask unless `threads` says otherwise (gemv_pool.rs:186-203). Returns the threads in use. */
int lko_pool_start(int threads);
int lko_physical_cores(void);
int lko_logical_cpus(void);
/* BlockQ4Kx8::repack (repack_q4k.rs:44-68): n rows (a multiple of 8) of nb Q4_K blocks into
 * n / 8 * nb group blocks of 1152 bytes; `out` holds that many. */
void lko_repack_q4k_x8(const uint8_t* rhs, size_t n, size_t nb, uint8_t* out);
/* The served Q4_K path over the repacked weights (matmul_q4k_plain_pre, drivers.rs:61-95). */
int oa_matmul_q4k_x8(size_t m, size_t k, size_t n, const float* lhs, const uint8_t* x8, float* dst);
/* The served prefill forms over repacked weights (matmul_q4k_repacked_tiled / matmul_q6k_repacked_tiled,
 * src/tensor/quant_cpu/drivers.rs:231-406): one pool chunk per group of eight columns, rows in tiles of
 * eight; and the Q6_K repack (repack_q6k.rs:41-64) with its scalar group dot (:96-123). Same returns. */
int oa_matmul_q4k_x8_tiled(size_t m, size_t k, size_t n, const float* lhs, const uint8_t* x8, float* dst);
void lko_repack_q6k_x8(const uint8_t* rhs, size_t n, size_t nb, uint8_t* out);
int oa_matmul_q6k_x8_tiled(size_t m, size_t k, size_t n, const float* lhs, const uint8_t* x8, float* dst);
void lko_gemv_group_q6k_x8_scalar(const uint8_t* grp, const uint8_t* y, size_t nb, float out[8]);
/* lko_moe_forward over chunks of tokens on the pool (the timed CPU figure beside the card's block). */
int lko_moe_forward_pool(int family, int dt_gu, int dt_down, size_t tokens, size_t hidden, size_t ffn, size_t n_experts,
                         size_t topk, const float* x, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                         const int32_t* ids, const float* weights, float* out);
int oa_matmul_fast(int dtype, size_t m, size_t k, size_t n, const float* lhs,
                   const uint8_t* rhs, size_t rhs_bytes, float* dst, int threads);

#ifdef __cplusplus
}
#endif
#endif

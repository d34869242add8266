/*
 * loken_gfx950: C ABI of the MI355X (gfx950) GGUF block-quantized matmul library.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream (`void*` holding a
 * hipStream_t, NULL = the default stream), launches asynchronously on that stream and returns.
 * Nothing here synchronizes, and nothing allocates unless a comment says so. Buffers are owned by the caller.
 * Weight blobs are raw GGUF blocks, row-major `[n rows][k / block_len blocks]`.
 *
 * Each declaration cites the reference interface (loken, paths relative to its root) it
 * stands in for. Two groups:
 *   * names and signatures kept verbatim where loken links a launcher statically
 *     (launch_mmq_*, loken_moe_*): src/tensor/quantized/mmq.rs, src/inference/moe_cuda/ (*.rs);
 *   * lk_* launchers where loken fetches a kernel BY NAME from a run-time-compiled module and
 *     launches it with a (32, nwarps) block (src/tensor/cuda/quant.rs:3581-3684): a wave64
 *     kernel cannot honour that block contract, so the launch geometry moves behind the ABI.
 *
 * Status: `int` launchers return LK_OK (0) or a positive LK_ERR_* code and never abort; the
 * launch_mmq_* family keeps loken's convention of returning the tile width launched, 0 when
 * nothing ran.
 */
#ifndef LOKEN_GFX950_H
#define LOKEN_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (src/tensor/quantized/dtype.rs:66-96) */
#define LK_TYPE_F32 0
#define LK_TYPE_F16 1
#define LK_TYPE_Q4_0 2
#define LK_TYPE_Q4_1 3
#define LK_TYPE_Q5_0 6
#define LK_TYPE_Q5_1 7
#define LK_TYPE_Q8_0 8
#define LK_TYPE_Q8_1 9
#define LK_TYPE_Q2_K 10
#define LK_TYPE_Q3_K 11
#define LK_TYPE_Q4_K 12
#define LK_TYPE_Q5_K 13
#define LK_TYPE_Q6_K 14
#define LK_TYPE_IQ2_XXS 16
#define LK_TYPE_IQ3_XXS 18
#define LK_TYPE_IQ4_NL 20
#define LK_TYPE_IQ3_S 21
#define LK_TYPE_IQ2_S 22
#define LK_TYPE_IQ4_XS 23
#define LK_TYPE_BF16 30
#define LK_TYPE_MXFP4 39
#define LK_TYPE_Q2_0 42

#define LK_OK 0
#define LK_ERR_ARG 1        /* a size, stride or pointer the kernels cannot take */
#define LK_ERR_TYPE 2       /* weight / activation / output type not served */
#define LK_ERR_LAUNCH 3     /* the HIP runtime refused the launch */
#define LK_ERR_NOMEM 4      /* scratch could not be reserved (MoE decode launchers only) */
#define LK_ERR_SIZE 5       /* the call needs more than the fixed scratch of an entry point that allocates nothing */
#define LK_NOT_TAKEN 6      /* host mirror only: forward would serve this call another way (the reference's None) */

/* Bytes of the per-device fixed scratch array behind loken_moe_gemm_gguf_down_reduce_static. */
#define LK_STATIC_SCRATCH_BYTES (8u << 20)

/* Row padding of a quantized activation, in values (MATRIX_ROW_PADDING,
 * src/tensor/quantized/mod.rs:29-35). */
#define LK_ROW_PADDING 512

/* Library / device facts: {abi version, CU count, LDS bytes per workgroup, wave size}. */
int lk_device_info(int* abi_version, int* compute_units, int* lds_bytes, int* wave_size);

/* ---------------------------------------------------------------------------------------
 * Decode path: Q8_1 row quantizer + mat-vec.
 * ------------------------------------------------------------------------------------- */

/* Rows of `x` (`x_type` LK_TYPE_F32 / F16 / BF16, `rows` x `kx`, contiguous) into Q8_1 blocks of
 * 32: `vy` receives rows * (kx_padded / 32) blocks of 36 bytes {f16 d, f16 s, 32 x i8}; values
 * past kx quantize as zero blocks. d = amax/127, codes = round_half_away(x * (1/d)),
 * s = f16(sum(codes) * d): loken's BlockQ8_1::quantize (src/tensor/quant_cpu/format/q8_1.rs:46-61).
 * Replaces kernel `mmvq_gguf_quantize_q8_1_{f32,f16,bf16}` and its launcher
 * quantize_q8_1_rows_t (src/inference/cuda/mmvq_gguf.cu:766-775; src/tensor/cuda/quant.rs:112-151).
 * kx_padded must be a multiple of 32 (loken passes a multiple of 512). */
int lk_quantize_q8_1(const void* x, int x_type, void* vy, int kx, int kx_padded, int rows,
                     void* stream);

/* dst[j, row] = weight row `row` . activation row j, j < batch (1..8).
 *   wtype          LK_TYPE_Q4_K | LK_TYPE_Q5_K | LK_TYPE_Q6_K | LK_TYPE_Q8_0, and (this launcher and
 *                  lk_mmvq_subdots only) the 32-value nibble formats LK_TYPE_Q4_0 | Q4_1 | Q5_0 | Q5_1 | IQ4_NL | MXFP4, Q2_K | Q3_K | IQ4_XS
 *                  and the codebook formats IQ2_XXS | IQ3_XXS | IQ3_S | IQ2_S | Q2_0 (lk_mmvq_subdots: two integers per run
 *                  of 32 values, its halves)
 *   vx             nrows_x rows of ncols_x / block_len blocks (Q4_K / Q5_K 16-byte aligned, Q2_K / IQ4_XS
 *                  4-byte, MXFP4 any address, every other format 2-byte; else LK_ERR_ARG)
 *   vy_q8_1        batch rows of Q8_1 blocks, `stride_col_y` blocks apart (k_padded / 32)
 *   dst            `dst_type` LK_TYPE_F32 | F16 | BF16, rows `stride_col_dst` elements apart
 *   bias           nullable f32[nrows_x], added in the store
 *   decode_order   non-zero: every row of a batch sums exactly as a batch-1 launch would
 * Replaces kernels `mmvq_gguf_{tag}_{f32,f16,bf16}_plain[_do|_smallk|_bias]_cuda{1..8}` and
 * launch_mmvq / mmvq_geometry (src/inference/cuda/mmvq_gguf.cu:153-281,338-510;
 * src/tensor/cuda/quant.rs:3581-3684). Lanes never reduce across launches, so a row's sum
 * does not depend on batch: decode_order is honoured by construction. */
int lk_mmvq(int wtype, const void* vx, const void* vy_q8_1, void* dst, int dst_type,
            int ncols_x, int nrows_x, int batch, int stride_col_y, int stride_col_dst,
            const float* bias, int decode_order, void* stream);

/* Up to 4 weight matrices of one format and one k over the SAME activation rows in one launch:
 * matrix i has nrows_x[i] rows and writes dst[i] (bias[i] nullable, `bias` itself nullable).
 * The pointer arrays are host arrays. Every row carries the bits lk_mmvq gives it alone.
 * Generalizes the two-matrix launch `mmvq_gguf_{tag}_f32_plain_dual_cuda1` / mmvq_f32_dual
 * (src/inference/cuda/mmvq_gguf.cu:515-545; src/tensor/cuda/quant.rs:3369-3413), which attention
 * uses for q and k; three matrices serve q, k, v of a layer at once. */
int lk_mmvq_multi(int wtype, int count, const void* const* vx, const void* vy_q8_1, void* const* dst,
                  int dst_type, int ncols_x, const int* nrows_x, int batch, int stride_col_y,
                  int stride_col_dst, const float* const* bias, void* stream);

/* lk_mmvq_multi straight from f32 activation rows (`batch` rows, `stride_x` floats apart, 16-byte
 * aligned, stride a multiple of 4): every workgroup quantizes the rows to Q8_1 in LDS while it
 * stages them, with the steps of lk_quantize_q8_1, so the outputs carry the bits of the
 * two-launch path and the quantize launch disappears. This is what QKernelMatMul::forward does
 * for a decode row (quantize, then mat-vec: src/tensor/quantized/kernel_matmul.rs:1474-1487,
 * 658-691) folded into one launch, in the spirit of the reference's fused Q8_1 producers
 * (src/inference/cuda/mmvq_gguf.cu:760-1000; src/tensor/cuda/prequant.rs). */
int lk_mmvq_fused(int wtype, int count, const void* const* vx, const float* x, int stride_x,
                  void* const* dst, int dst_type, int ncols_x, const int* nrows_x, int batch,
                  int stride_col_dst, const float* const* bias, void* stream);

/* dst[j, row] = act(gate row . x_j) * (up row . x_j), act 0 = SiLU g/(1+exp(-g)), 1 = tanh-GELU;
 * gate and up have the same shape; batch 1..4; dst f32 or bf16. Replaces kernels
 * `mmvq_gguf_pair_{g}_{u}_silu*_cuda1` and `mmvq_gguf_q4_k_{f32,bf16}_fused_{silu,gelu}_cuda1`
 * with fast_mmvq::try_fused (src/inference/cuda/mmvq_gguf.cu:588-758;
 * src/tensor/quantized/fast_mmvq.rs:97-282). */
int lk_mmvq_pair_act(int wtype, const void* gate, const void* up, const void* vy_q8_1, void* dst,
                     int dst_type, int ncols_x, int nrows_x, int batch, int stride_col_y,
                     int stride_col_dst, int act, void* stream);

/* Decode-step producers that end in the activation a mat-vec reads: the f32 row is written as
 * before and the same row leaves as Q8_1 blocks (`vy`: rows * cols / 32 blocks of 36 bytes, byte
 * for byte what lk_quantize_q8_1 makes of the f32 row), so the mat-vec that follows needs no
 * quantizer launch. rows x cols f32, contiguous; cols a multiple of 512 (the quantized row has no
 * padding), one workgroup per row. Sum of squares as the reference's wide kernels fold it (lane t
 * of 256 over t, t + 256, ..., then a stride-halving tree); rms = 1 / sqrt(mean + eps), correctly
 * rounded, where the reference takes the card's rsqrtf approximation.
 * Replace kernels `rmsnorm_wide_q8_1_f32`, `add_rmsnorm_dual_wide_q8_1_f32` and
 * `post_norm_add_norm_wide_q8_1_f32` (src/inference/cuda/mmvq_gguf.cu:805-936) with their launch
 * sites rms_norm_f32 (src/tensor/cuda/gemm.rs:561-590) and fused_post_norm_add_norm /
 * fused_add_rmsnorm_dual (src/inference/kernel/fused/buffers/conv.rs:990-1110). */
int lk_rmsnorm_q8_1(const float* x, const float* weight, float* out, void* vy, float eps, int cols, int rows,
                    void* stream);
/* The reference's own single-row launchers in front of a mat-vec, names and arguments kept
 * (cuda/moe/rms_qmatmul.cu:152-169 f32 row, :221-238 bf16 row; declared src/inference/moe_cuda/mod.rs:
 * 117-119, 468-471; called from src/inference/moe_cuda/norm.rs:154, 206): y = Q8_1(rmsnorm(x, w_norm)),
 * hidden a multiple of 32, no f32 copy. The blocks are lk_rmsnorm_q8_1's (wide-kernel order of the
 * sum of squares, correctly rounded 1 / sqrt, lk_quantize_q8_1's block rule). Void: nothing is
 * launched on a bad argument. */
void loken_rms_quantize_q8_1(const float* x, const float* w_norm, void* y_q8_1, int hidden, float rms_eps,
                             void* stream);
void loken_rms_quantize_q8_1_bf16(const void* x, const float* w_norm, void* y_q8_1, int hidden, float rms_eps,
                                  void* stream);
/* sum_out = x + residual; norm_out = rmsnorm(sum_out, weight), also as Q8_1. */
int lk_add_rmsnorm_q8_1(const float* x, const float* residual, const float* weight, float* sum_out,
                        float* norm_out, void* vy, float eps, int cols, int rows, void* stream);
/* x_out = rmsnorm(a, w_post) + residual (each product rounded before it is added);
 * norm_out = rmsnorm(x_out, w_ffn), also as Q8_1. */
int lk_post_norm_add_norm_q8_1(const float* a, const float* w_post, const float* residual, const float* w_ffn,
                               float* x_out, float* norm_out, void* vy, float eps_post, float eps_ffn, int cols,
                               int rows, void* stream);
/* out[r, i] = act(gu[r, i]) * gu[r, n + i] for rows of 2 n values (gate then up), also as Q8_1;
 * act 0 = SiLU g / (1 + exp(-g)), 1 = tanh-GELU; n a multiple of 32. Replaces kernels
 * `split_silu_mul_q8_1_f32` / `split_gelu_mul_q8_1_f32` (src/inference/cuda/mmvq_gguf.cu:971-999;
 * launched from src/inference/kernel/fused/buffers/conv.rs:735,834), which take one row. */
int lk_split_act_mul_q8_1(const float* gu, float* out, void* vy, int n, int rows, int act, void* stream);

/* The gate/up pair launch that hands its result on as Q8_1: dst = Q8_1(act(gate . x) * (up . x)),
 * blocks of 32 consecutive output rows, written with lk_quantize_q8_1's rule, so the down
 * projection of a decode layer reads it without a quantizer launch in between (the fused
 * neighbours of the mat-vec: pair kernels src/inference/cuda/mmvq_gguf.cu:588-758 followed by
 * quantize_q8_1_rows, src/tensor/cuda/quant.rs:112-151, in one launch). `act`: the activation
 * rows, f32 (act_is_f32 != 0, stride_act floats apart, quantized to Q8_1 in the kernel) or Q8_1
 * (stride_act blocks apart). dst: batch rows of nrows_x / 32 blocks, stride_dst_blocks apart.
 * nrows_x a multiple of 32; batch 1..4; act_fn 0 = SiLU, 1 = tanh-GELU. */
int lk_mmvq_pair_act_q8_1(int wtype, const void* gate, const void* up, const void* act, int act_is_f32,
                          int stride_act, void* dst_q8_1, int stride_dst_blocks, int ncols_x, int nrows_x,
                          int batch, int act_fn, void* stream);
/* `groups` weights of one shape [nrows_x, ncols_x], each over its OWN Q8_1 row: weight g lives at
 * device address table[g] (a device array), reads the blocks from g * ncols_x/32 of vy_q8_1 and
 * writes dst from g * nrows_x. ncols_x must be a multiple of 512. Replaces kernel
 * `mmvq_gguf_{tag}_f32_plain_grouped_cuda1` / mmvq_f32_grouped
 * (src/inference/cuda/mmvq_gguf.cu:547-565; src/tensor/cuda/quant.rs:3418-3466). */
int lk_mmvq_grouped(int wtype, const uint64_t* table, int groups, const void* vy_q8_1, float* dst,
                    int ncols_x, int nrows_x, void* stream);

/* Parity probe: the exact integer sub-block dot products the mat-vec kernels form, for ONE
 * activation row. dots: Q4_K int32[nrows_x][ncols_x/32] (sum over 32 of nibble*q8),
 * Q6_K int32[nrows_x][ncols_x/16] (sum over 16 of (code-32)*q8), Q8_0 int32[nrows_x][ncols_x/32].
 * sums (nullable): int32[ncols_x/32], sum over 32 of q8. Same device functions as lk_mmvq.
 * No counterpart in the reference: it exists so a test can compare integers bit for bit with
 * the inner sums of BlockQ4K::dot_scalar and friends (format/q4_k.rs:62-88, q6_k.rs:51-82,
 * q8_0.rs:83-97). */
int lk_mmvq_subdots(int wtype, const void* vx, const void* vy_q8_1, int32_t* dots, int32_t* sums,
                    int ncols_x, int nrows_x, void* stream);

/* The exact mode: Q4_K / Q6_K weight rows x `batch` Q8_K activation rows (292-byte blocks {f32 d, 256 x i8,
 * 16 x i16 sums}, batch rows of ncols_x / 256 blocks, 4-byte aligned) -> dst[batch][nrows_x] f32 with the
 * reference's cross-device contract (ExactDot, src/tensor/quant_cpu/format/blocks.rs:80-96; dot_exact,
 * format/q4_k.rs:117-156, q6_k.rs:121-163): exact integer sums per super-block, then a fixed f32 fold,
 * total += d8 * (d * f32(scaled) - dmin * f32(offset)) from -0.0 in block order, one rounding per
 * operation. The result carries the bits of the CPU's dot_exact. A parity path, not a fast one. */
int lk_mmvq_exact(int wtype, const void* vx, const void* vy_q8_k, float* dst, int ncols_x, int nrows_x, int batch,
                  void* stream);

/* ---------------------------------------------------------------------------------------
 * Prefill path: tiled quantized matmul on int8 MFMA. Names, argument lists and return
 * conventions are loken's (src/tensor/quantized/mmq.rs:64-116 quantizers, :132-147 and
 * cuda/mmq_gguf/mmq_launch.cuh:192-206 tile kernels), so `mmq_forward`
 * (src/tensor/quantized/kernel_matmul/mmq.rs:21-159) links against them unchanged.
 * ------------------------------------------------------------------------------------- */

/* Activation rows -> the workspace the tile kernels read. `x` is f32, or f16 when type_x == 1;
 * row r of the result is row ids[r] of x (ids nullable); ne00 = values per row, s01/s02/s03 =
 * element strides of row / channel / sample, ne0 = padded row length (multiple of 512),
 * ne1 = rows, ne2 * ne3 = channels. `vy` needs ne1 * (ne0/128) * 144 bytes per channel, the
 * size loken allocates. D4 (scale only: Q6_K, Q8_0), DS4 (scale and sum: Q4_K) and D2S6 (Q2_K: in
 * the reference a scale per 64 values and sums per 16) write the same records here: a scale and a
 * sum per 32 values, the Q2_K tile forming its sums per 16 from the codes.
 * Replaces launch_mmq_quantize_q8_1_{D4,DS4,D2S6} of cuda/mmq_gguf/mmq_quantize.cu:67-166; codes
 * follow BlockQ8_1::quantize (1/d rule), not that file's 127/amax rule, so that tiled and
 * mat-vec products see the same integers. */
void launch_mmq_quantize_q8_1_D4(const void* x, const int32_t* ids, void* vy, int type_x,
                                 int64_t ne00, int64_t s01, int64_t s02, int64_t s03, int64_t ne0,
                                 int64_t ne1, int64_t ne2, int64_t ne3, void* stream);
void launch_mmq_quantize_q8_1_DS4(const void* x, const int32_t* ids, void* vy, int type_x,
                                  int64_t ne00, int64_t s01, int64_t s02, int64_t s03, int64_t ne0,
                                  int64_t ne1, int64_t ne2, int64_t ne3, void* stream);
void launch_mmq_quantize_q8_1_D2S6(const void* x, const int32_t* ids, void* vy, int type_x,
                                   int64_t ne00, int64_t s01, int64_t s02, int64_t s03, int64_t ne0,
                                   int64_t ne1, int64_t ne2, int64_t ne3, void* stream);

/* dst[col, row] (f32, rows `stride_col_dst` floats apart) = weight row `row` . token `col`.
 *   x = weights [nrows_x][stride_row_x blocks], y = workspace of ncols_y rows, ncols_x = k.
 * Returns the token-tile width launched (32, 64 or 128), 0 when nothing ran (bad sizes, or k
 * not a multiple of 256). cc, nsm, smpbo, warp_size are accepted and unused: one device family.
 * tmp_fixup: null, or the 16 MiB buffer the reference's workspace keeps for its stream-k partial
 * tiles (FIXUP_BYTES = 256 * 128 * 128 * 4, src/tensor/quantized/kernel_matmul/mmq.rs:42; 16-byte
 * aligned, contents irrelevant on entry, overwritten). With it, a product whose tiles would leave
 * most of the chip idle is launched with K cut into ranges of blocks: each workgroup writes its
 * partial tile there and a second launch adds the ranges in ascending order into dst (same integers,
 * a fixed order of f32 sums: the result does not depend on scheduling; it differs from the null
 * call's in the last bits). Used only when every partial product fits the 16 MiB, nrows_x and
 * stride_col_dst are multiples of 4 and dst is 16-byte aligned. Calls sharing one buffer must not
 * overlap on the card (the reference holds its workspace mutex across quantize and matmul,
 * kernel_matmul/mmq.rs:43-86). Both launches are capturable.
 * Replaces launch_mmq_gguf_{q4_k,q5_k,q6_k,q8_0} (cuda/mmq_gguf/mmq_launch.cuh:61-206). */
int launch_mmq_gguf_q4_k(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);
int launch_mmq_gguf_q5_k(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);
int launch_mmq_gguf_q6_k(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);
/* Q8_0 rows are 32-value blocks (stride_row_x = k / 32); k must still be a multiple of 256. */
int launch_mmq_gguf_q8_0(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);

/* The 32-value nibble formats on the Q8_0 tile (stride_row_x = k / 32 blocks; weights 2-byte aligned):
 * codes expanded to int8 less the format's bias on the way into the tile, Q4_1 / Q5_1 with the
 * block minimum as + m * (d8 * sum of the token's codes).
 * Replaces launch_mmq_gguf_{q4_0,q4_1,q5_0,q5_1} (src/tensor/quantized/mmq.rs:274-279). */
int launch_mmq_gguf_q4_0(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);
int launch_mmq_gguf_q4_1(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);
int launch_mmq_gguf_q5_0(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);
int launch_mmq_gguf_q5_1(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);

/* Q3_K (110-byte super-blocks, stride_row_x = k / 256; weights 2-byte aligned) on the Q6_K tile shape:
 * codes -4..3, one six-bit scale less 32 per 16 values.
 * Replaces launch_mmq_gguf_q3_k (src/tensor/quantized/mmq.rs:281). */
int launch_mmq_gguf_q3_k(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);

/* Q2_K (84-byte super-blocks, weights 4-byte aligned): unsigned two-bit codes, a four-bit scale and a
 * four-bit minimum per 16 values, the minimum against the token's sums per 16 codes.
 * Replaces launch_mmq_gguf_q2_k (src/tensor/quantized/mmq.rs:280). */
int launch_mmq_gguf_q2_k(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,
                         int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                         int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                         void* stream);

/* ---------------------------------------------------------------------------------------
 * MoE prefill: expert-batched tiled matmul and the steps around it. Names and argument lists are
 * loken's (src/tensor/quantized/mmq.rs:151-173; src/inference/moe_cuda/mmq_experts.rs:42-56),
 * called as MmqRouting::{from_choices, gate_up_over, down_fold_over} call them (:183-557).
 * ------------------------------------------------------------------------------------- */

/* For each expert e < n_experts: slab `x + e * stride_expert_x` (bytes) of nrows_x rows against
 * the workspace rows [expert_bounds[e], expert_bounds[e+1]) of `y` (ncols_y rows in all, sorted
 * by expert); workspace row c is written to destination row ids_dst[c] (or c when ids_dst is
 * null), rows `stride_col_dst` floats apart. A second stack `x_second` of the same shape is
 * multiplied in the same launch, its results `dst_second` floats after the first's in each row.
 * ncols_max sizes the grid's column-tile axis (longer runs are still covered), ncols_hint or a
 * non-zero mmq_x picks the tile width. Returns the tile width launched, 0 when nothing ran.
 * Replaces launch_mmq_moe_gguf_* (cuda/mmq_gguf/mmq_launch.cuh:212-319). */
int launch_mmq_moe_gguf_q4_k(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_q5_k(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_q6_k(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_q8_0(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);

/* The same launch for the 32-value nibble formats, and for the two that only mixtures store and that
 * have no dense entry point (IQ4_NL: the 16 levels as int8 codes; MXFP4: its levels, E8M0 scale, 17-byte
 * blocks at any byte address). Replaces launch_mmq_moe_gguf_{q4_0,q4_1,q5_0,q5_1} and the expert-only
 * launch_mmq_moe_gguf_{iq4_nl,mxfp4} (src/tensor/quantized/mmq.rs:274-279, 326-334). */
int launch_mmq_moe_gguf_q4_0(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_q4_1(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_q5_0(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_q5_1(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_iq4_nl(const void* x, const void* x_second, int64_t dst_second, const void* y,
                               void* dst, const int* expert_bounds, const int* ids_dst,
                               int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                               int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                               int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                               int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_mxfp4(const void* x, const void* x_second, int64_t dst_second, const void* y,
                              void* dst, const int* expert_bounds, const int* ids_dst,
                              int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                              int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                              int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                              int64_t smpbo, int warp_size, void* stream);

/* Q3_K, and IQ4_XS (expert-only in the reference: eight runs of IQ4_NL levels under six-bit scales
 * less 32; weights 4-byte aligned). Replaces launch_mmq_moe_gguf_{q3_k,iq4_xs}
 * (src/tensor/quantized/mmq.rs:281, 329). */
int launch_mmq_moe_gguf_q3_k(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_iq4_xs(const void* x, const void* x_second, int64_t dst_second, const void* y,
                               void* dst, const int* expert_bounds, const int* ids_dst,
                               int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                               int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                               int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                               int64_t smpbo, int warp_size, void* stream);

/* The codebook formats only mixtures store: IQ3_XXS (98-byte blocks), IQ3_S (110), IQ2_S (82), all of 256
 * values, and Q2_0 (18 bytes, 64 values, stride_row_x in those blocks); weights 2-byte aligned. Replaces
 * launch_mmq_moe_gguf_{iq3_xxs,iq3_s,iq2_s,q2_0} (src/tensor/quantized/mmq.rs:335-343; kernels
 * cuda/mmq_gguf/mmq_instance_iq3_xxs.cu and siblings, dequantizers cuda/moe/gguf_iq.cuh:126-196). */
int launch_mmq_moe_gguf_iq3_xxs(const void* x, const void* x_second, int64_t dst_second, const void* y,
        void* dst, const int* expert_bounds, const int* ids_dst, int64_t stride_expert_x, int64_t ncols_x,
        int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst, int n_experts,
        int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc, int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_iq3_s(const void* x, const void* x_second, int64_t dst_second, const void* y,
        void* dst, const int* expert_bounds, const int* ids_dst, int64_t stride_expert_x, int64_t ncols_x,
        int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst, int n_experts,
        int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc, int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_iq2_s(const void* x, const void* x_second, int64_t dst_second, const void* y,
        void* dst, const int* expert_bounds, const int* ids_dst, int64_t stride_expert_x, int64_t ncols_x,
        int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst, int n_experts,
        int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc, int64_t smpbo, int warp_size, void* stream);
int launch_mmq_moe_gguf_q2_0(const void* x, const void* x_second, int64_t dst_second, const void* y,
        void* dst, const int* expert_bounds, const int* ids_dst, int64_t stride_expert_x, int64_t ncols_x,
        int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst, int n_experts,
        int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc, int64_t smpbo, int warp_size, void* stream);

/* Replaces launch_mmq_moe_gguf_q2_k (src/tensor/quantized/mmq.rs:280). */
int launch_mmq_moe_gguf_q2_k(const void* x, const void* x_second, int64_t dst_second, const void* y,
                             void* dst, const int* expert_bounds, const int* ids_dst,
                             int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x,
                             int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst,
                             int n_experts, int64_t ncols_max, int64_t ncols_hint, int mmq_x, int cc,
                             int64_t smpbo, int warp_size, void* stream);

/* From a routing already sorted by expert: bounds[e] = first sorted row of expert >= e
 * (n_experts + 1 entries), slots_out = slots, src_rows[i] = slots[i] / topk.
 * cuda/moe/moe_mmq.cu:30-55,180-188. */
void loken_moe_mmq_plan(const int32_t* experts, const int32_t* slots, int n, int topk, int n_experts,
                        int32_t* bounds, int32_t* slots_out, int32_t* src_rows, void* stream);
/* From the router's choices [n = tokens * topk]: groups the pairs by expert on the device.
 * `counts` is n_experts ints of scratch. Rows of one expert come in ascending pair order (the
 * reference leaves that order unspecified). cuda/moe/moe_mmq.cu:57-99,190-198. */
void loken_moe_mmq_route(const int32_t* choices, int n, int topk, int n_experts, int32_t* counts,
                         int32_t* bounds, int32_t* slots, int32_t* src_rows, void* stream);
/* out[r, c] = silu(gu[r, c]) * gu[r, width + c] over gu [rows, 2 * width]. moe_mmq.cu:101-114. */
void loken_moe_mmq_silu_mul(const float* gu, float* out, int64_t rows, int width, void* stream);
/* gpt-oss gate: x = min(g + gb, limit), u' = clamp(u + ub, -limit, limit),
 * out = x * sigmoid(alpha x) * (1 + u'); biases [n_experts, width], nullable. moe_mmq.cu:131-153. */
void loken_moe_mmq_swiglu_oai(const float* gu, float* out, int64_t rows, int width,
                              const int32_t* bounds, int n_experts, const float* gate_bias,
                              const float* up_bias, float alpha, float limit, void* stream);
/* out[t, c] += sum over k ascending of weights[p] * (pairs[p, c] + down_bias[choices[p], c]),
 * p = t * topk + k; bias and choices nullable together. moe_mmq.cu:155-176. */
void loken_moe_mmq_fold(const float* pairs, const float* weights, const int32_t* choices,
                        const float* down_bias, float* out, int64_t tokens, int topk, int cols,
                        void* stream);

/* ---------------------------------------------------------------------------------------
 * MoE decode: one mat-vec per routed pair (few rows per expert). Names, argument lists and row
 * conventions are loken's (src/inference/moe_cuda/mod.rs:235-262, 415-442, 473-483;
 * cuda/moe/moe_gguf.cu:476-511, 755-860, 1049-1061). sorted_token_ids[i] is the flattened
 * (token * topk + choice) slot of routed pair i, expert_ids[i] its expert; size_m = pairs,
 * size_n = output rows per expert, size_k = reduction length; quant_type is loken's wire id
 * (0 = Q8_0, 1 = Q4_K, 2 = Q2_K, 3 = Q3_K, 4 = Q5_K, 5 = Q6_K, 6 = Q5_0, 7 = MXFP4, 8 = Q5_1, 9 = IQ4_NL,
 * 10 = IQ4_XS, 11 = IQ3_XXS, 12 = IQ3_S, 13 = IQ2_S, 14 = Q2_0, 15 = IQ2_XXS: src/inference/moe_cuda/gemm.rs:23-39).
 * Weights are stacks [num_experts][size_n][size_k / block].
 * These launchers quantize the f32 activation themselves into a per-(device, stream)
 * grow-only scratch (the one allocation in this library; growing is refused with
 * LK_ERR_NOMEM while the stream is being captured). Return 0 or an LK_ERR_* code.
 * ------------------------------------------------------------------------------------- */

/* out[slot, :] = expert(slot) . x[row], times topk_weights[slot] when given; with weights the
 * activation row is `slot` (inputs [size_m, k]), without it is slot / topk (inputs [size_m/topk, k]). */
int loken_moe_gemm_gguf(const float* inputs, const void* weights, const int32_t* sorted_token_ids,
                        const int32_t* expert_ids, const float* topk_weights, void* outputs,
                        int num_experts, int topk, int size_m, int size_n, int size_k, int quant_type,
                        void* stream);
/* The prefill form (declared src/inference/moe_cuda/mod.rs:478-483; called from moe_gemm_gguf when
 * the card has matrix instructions, src/inference/moe_cuda/gemm.rs:221-258; AMD body
 * cuda/moe/moe_wmma_amd.cu:311-339): activation rows at the model's own width, input_dtype 0 = f16,
 * 1 = bf16 (anything else: LK_ERR_TYPE); the other arguments, the row conventions and the status as
 * loken_moe_gemm_gguf. Rows are quantized to Q8_1 from that width and served by the same kernels, so
 * results carry the decode path's integers (the reference multiplies dequantized weights on bf16
 * fragments instead: both approximate the f32 product). */
int loken_moe_gemm_gguf_prefill(const void* input, const uint8_t* weights, const int32_t* sorted_token_ids,
                                const int32_t* expert_ids, const float* topk_weights, void* output,
                                int num_experts, int topk, int size_m, int size_n, int size_k, int input_dtype,
                                int gguf_dtype, void* stream);
/* out[slot, :] = silu(gate_e . x[slot / topk]) * (up_e . x[slot / topk]); inputs [size_m/topk, k]. */
int loken_moe_gemm_gguf_gate_up_silu_mul(const float* inputs, const void* gate_weights,
                                         const void* up_weights, const int32_t* sorted_token_ids,
                                         const int32_t* expert_ids, float* outputs, int num_experts,
                                         int topk, int size_m, int size_n, int size_k, int quant_type,
                                         void* stream);
/* The same launch with the other gated activations of the reference's expert kernels
 * (cuda/moe/moe_gguf.cu:960-1003, 1101-1118; 1146-1184, 1196-...; 1243-1289, 1301-...;
 * src/inference/moe_cuda/gemm.rs:596-747), g = gate_e . x, u = up_e . x:
 *   swiglu_oai      g += gate_bias[e], u += up_bias[e] ([num_experts, size_n] f32, nullable);
 *                   x = min(g, limit); out = x * sigmoid(alpha x) * (1 + clamp(u, -limit, limit))
 *   swiglu_limited  g = min(g, limit), u = clamp(u, -limit, limit); out = silu(g) * u
 *   gelu_mul_concat one tensor [num_experts, 2 size_n, k] per layer, an expert's gate rows then its
 *                   up rows; out = gelu_tanh(g) * u */
int loken_moe_gemm_gguf_gate_up_swiglu_oai(const float* inputs, const void* gate_weights,
                                           const void* up_weights, const int32_t* sorted_token_ids,
                                           const int32_t* expert_ids, const float* gate_bias,
                                           const float* up_bias, float* outputs, int num_experts, int topk,
                                           int size_m, int size_n, int size_k, int quant_type, float alpha,
                                           float limit, void* stream);
int loken_moe_gemm_gguf_gate_up_swiglu_limited(const float* inputs, const void* gate_weights,
                                               const void* up_weights, const int32_t* sorted_token_ids,
                                               const int32_t* expert_ids, float* outputs, int num_experts,
                                               int topk, int size_m, int size_n, int size_k, int quant_type,
                                               float limit, void* stream);
int loken_moe_gemm_gguf_gate_up_gelu_mul_concat(const float* inputs, const void* gate_up_weights,
                                                const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                                float* outputs, int num_experts, int topk, int size_m,
                                                int size_n, int size_k, int quant_type, void* stream);
/* loken_moe_gemm_gguf_gate_up_silu_mul over the first `*live` routed pairs, the count read on the
 * card when the kernel runs (a captured step whose routing changes between replays); the rows of
 * the other pairs are not written (cuda/moe/moe_gguf.cu:1063-1075; moe_cuda/gemm.rs:424-474). */
int loken_moe_gemm_gguf_gate_up_silu_mul_live(const float* inputs, const void* gate_weights,
                                              const void* up_weights, const int32_t* sorted_token_ids,
                                              const int32_t* expert_ids, float* outputs, int num_experts,
                                              int topk, int size_m, int size_n, int size_k, int quant_type,
                                              const unsigned int* live, void* stream);
/* The down launch up to the pairs' rows: pair_rows[slot, :] = topk_weights[slot] * (down_e . inputs[slot])
 * for the first `*live` routed pairs, zero rows for the others; the caller sums a token's topk rows
 * (cuda/moe/moe_gguf.cu:838-852; moe_cuda/gemm.rs:550-590). */
int loken_moe_gemm_gguf_down_pairs_live(const float* inputs, const void* weights,
                                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                        const float* topk_weights, float* pair_rows, int num_experts,
                                        int topk, int size_m, int size_n, int size_k, int quant_type,
                                        const unsigned int* live, void* stream);
/* A layer's experts over two tensors: the slots from `alt_from` on are slot (expert - alt_from) of
 * the `alt_*` tensor (same format and row count per expert). `alt_at`, when not NULL, is an array
 * of two addresses ON THE CARD read when the kernel runs and used in place of alt_gate / alt_up
 * (for the down launch: [0] in place of alt_weights). Otherwise as the launch each is named after
 * (cuda/moe/moe_gguf.cu:239-257, 824-836, 868-880, 1078-1091; moe_cuda/gemm.rs:319-419, 479-545, 778-...). */
int loken_moe_gemm_gguf_gate_up_silu_mul_two(const float* inputs, const void* gate_weights,
                                             const void* up_weights, const void* alt_gate,
                                             const void* alt_up, int alt_from, const void* const* alt_at,
                                             const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                             float* outputs, int num_experts, int topk, int size_m,
                                             int size_n, int size_k, int quant_type, void* stream);
int loken_moe_gemm_gguf_down_reduce_two(const float* inputs, const void* weights, const void* alt_weights,
                                        int alt_from, const int32_t* sorted_token_ids,
                                        const int32_t* expert_ids, const float* topk_weights, float* outputs,
                                        int num_experts, int topk, int size_m, int size_n, int size_k,
                                        int quant_type, const float* down_bias, const float* add_after,
                                        void* stream);
int loken_moe_gemm_gguf_down_pairs_two(const float* inputs, const void* weights, const void* alt_weights,
                                       int alt_from, const void* const* alt_at,
                                       const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                       const float* topk_weights, float* pair_rows, int num_experts,
                                       int topk, int size_m, int size_n, int size_k, int quant_type,
                                       void* stream);
/* outputs[t, :] (+)= sum over k ascending of topk_weights[p] * (down_e(p) . inputs[p] + down_bias[e(p)]),
 * p = t * topk + k; inputs [size_m, k] in slot order. Without add_after `outputs` [size_m/topk,
 * size_n] must be pre-filled (zeros or the residual) and is accumulated into; with it the result
 * is written as fold + add_after. down_bias [num_experts, size_n] nullable. Q4_K / Q5_K / Q6_K rows of
 * 512, 768 or 1024 values with at most 512 routed pairs and topk <= 8 run as one launch that needs no
 * scratch (same bits as the mat-vec launch + fold every other call takes). */
int loken_moe_gemm_gguf_down_reduce(const float* inputs, const void* weights,
                                    const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                    const float* topk_weights, float* outputs, int num_experts, int topk,
                                    int size_m, int size_n, int size_k, int gguf_dtype,
                                    const float* down_bias, const float* add_after, void* stream);
/* loken_moe_gemm_gguf_down_reduce for callers that cannot allocate device memory (code recording a
 * HIP graph, serving loops and harnesses that forbid it): same arguments, same kernels, same
 * result, but the pairs' rows (and the Q8_1 rows of the formats that read them) live in a fixed
 * array of LK_STATIC_SCRATCH_BYTES that every GPU's copy of the library holds from load until the
 * process ends. No hipMalloc, hipFree or other allocating call is made. A call that needs more,
 * size_m * size_n * 4 bytes plus, for the formats that read Q8_1 rows,
 * size_m * pad512(size_k) / 32 * 36 bytes rounded up to 256, returns LK_ERR_SIZE and launches
 * nothing. Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
 * streams, or two host threads) race; calls on one stream are ordered and safe. The array keeps the
 * last call's contents and nothing is cleared: like the allocating entry point, the call relies on
 * sorted_token_ids naming every slot once (every named slot's row is written, zeros for a pair whose
 * expert is out of range). The first call on a device asks the runtime for the array's address there:
 * make it before a capture begins; later calls may be recorded into a graph (kernels only, no memset
 * node). No counterpart in the reference. */
int loken_moe_gemm_gguf_down_reduce_static(const float* inputs, const void* weights,
                                           const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                           const float* topk_weights, float* outputs, int num_experts,
                                           int topk, int size_m, int size_n, int size_k, int gguf_dtype,
                                           const float* down_bias, const float* add_after, void* stream);
/* outputs[t, c] += sum over k ascending of pairs[(t * topk + k), c] (cuda/moe/moe_gguf.cu:745-752). */
void loken_moe_sum_topk(const float* pairs, float* outputs, int tokens, int topk, int cols, void* stream);
/* Q4_K weight [size_n rows, size_k] x plain Q8_1 rows [size_m, size_k / 32 blocks] -> output
 * [size_m, size_n] f32 on the int8 matrix unit, 32 activation rows per pass and no weight staging
 * in LDS: the path for row counts between the mat-vec kernels and the tiled matmul. Replaces
 * loken_dense_q4k_imma_m8_plain (declared src/inference/moe_cuda/mod.rs:456-458, called from
 * dense_q4k_imma_m8_matmul, src/inference/moe_cuda/dense/imma.rs:82-135). size_k a multiple of
 * 256; weights 16-byte aligned; nothing is launched on a bad argument (void, as the reference's). */
void loken_dense_q4k_imma_m8_plain(const void* w, const void* q8_1, float* output, int size_m, int size_n,
                                   int size_k, void* stream);
/* The same launch with a status: LK_ERR_ARG (and nothing launched) for rows too long for the kernel's
 * scale tables in LDS (beyond roughly 36 thousand values) or a misaligned buffer, where the void
 * form above can only stay silent. What the host mirror calls, so that such a call goes on to the
 * tiled matmul instead of returning an untouched buffer. */
int lk_dense_q4k_rows(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                      void* stream);
/* Gate and up over the same plain Q8_1 rows in one launch: output[m, n] = act(gate[n] . x[m]) *
 * (up[n] . x[m]), act = SiLU (use_gelu == 0) or the tanh-form GELU. Replaces
 * loken_dense_q4k_imma_m8_actmul (declared src/inference/moe_cuda/mod.rs:452-455; launcher
 * cuda/moe/dense_q4k_imma_m8.cu:272-286; called from dense_q4k_imma_m8_gate_up_actmul,
 * src/inference/moe_cuda/dense/imma.rs:320-400). Same limits as the plain form. */
void loken_dense_q4k_imma_m8_actmul(const void* gate, const void* up, const void* q8_1, float* output,
                                    int size_m, int size_n, int size_k, int use_gelu, void* stream);
/* The same launch with a status, as lk_dense_q4k_rows is to the plain form. */
int lk_dense_q4k_rows_actmul(const void* gate, const void* up, const void* q8_1, float* output, int size_m,
                             int size_n, int size_k, int use_gelu, void* stream);
/* Up to three Q4_K (q5 != 0: Q5_K) matrices over the same plain Q8_1 rows (q + k + v of a decode step) in
 * one launch: outputs[i] is [size_m, sizes_n[i]] f32. The reference issues one
 * loken_dense_q4k_imma_m8_plain per matrix (dense_q4k_imma_m8_matmul, src/inference/moe_cuda/dense/
 * imma.rs:82-135); results equal those launches' bit for bit. `weights`, `outputs` and `sizes_n`
 * are host arrays of `count` (1..3) entries. */
int lk_dense_q4k_rows_multi(const void* const* weights, float* const* outputs, const int* sizes_n, int count,
                            const void* q8_1, int size_m, int size_k, int q5, void* stream);
/* Gate and up in one launch with the result handed on as Q8_1 rows: q8_1_out [size_m][size_n / 32 blocks]
 * = lk_quantize_q8_1(act(gate . x) * (up . x)) byte for byte, which the layer's down projection reads
 * with no f32 round trip and no quantizer launch in between. size_n a multiple of 32; up to 16 rows also
 * size_k 2048 or 4096 (anything else: LK_ERR_ARG; take lk_dense_q4k_rows_actmul and the quantizer). q5 != 0:
 * Q5_K weights. No counterpart in the reference, whose dense_q4k_imma_m8_act_mul writes f32
 * (src/inference/moe_cuda/dense/imma.rs:320-400); the mat-vec sibling is lk_mmvq_pair_act_q8_1. */
int lk_dense_q4k_rows_actmul_q8_1(const void* gate, const void* up, const void* q8_1, void* q8_1_out, int size_m,
                                  int size_n, int size_k, int use_gelu, int q5, void* stream);
/* The Q5_K siblings of the four launches above (block_q5_K = block_q4_K plus a plane of fifth bits):
 * loken_dense_q5k_imma_m8_plain / _actmul, declared src/inference/moe_cuda/mod.rs:459-466 and picked
 * by weight dtype at src/inference/moe_cuda/dense/imma.rs:113-116 and 362-365. */
void loken_dense_q5k_imma_m8_plain(const void* w, const void* q8_1, float* output, int size_m, int size_n,
                                   int size_k, void* stream);
int lk_dense_q5k_rows(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                      void* stream);
void loken_dense_q5k_imma_m8_actmul(const void* gate, const void* up, const void* q8_1, float* output,
                                    int size_m, int size_n, int size_k, int use_gelu, void* stream);
int lk_dense_q5k_rows_actmul(const void* gate, const void* up, const void* q8_1, float* output, int size_m,
                             int size_n, int size_k, int use_gelu, void* stream);
/* Expert-batched Q4_K rows on the matrix unit, for routings that give an expert a handful of rows:
 * expert e's matrix (weights + e * expert_bytes, size_n rows of size_k) against the sorted rows
 * [bounds[e], bounds[e + 1]) of the routing, 8, 16 or 32 of them per pass over the weights (rows_hint,
 * the run length expected per expert, picks the width; any count is served). Sorted row i reads the
 * plain Q8_1 row src_rows[i] (or i) of q8_1 (stride_blocks blocks apart) and writes row dst_rows[i]
 * (or i) of output (ldd floats apart). With weights_second (same layout) the result is
 * act(w . x) * (w2 . x), act 0 SiLU / 1 tanh-form GELU, else w . x. The reference reaches these
 * loads through launch_mmq_moe_gguf_q4_k (src/tensor/quantized/mmq.rs:274-286; MmqRouting,
 * src/inference/moe_cuda/mmq_experts.rs:300-557) or one mat-vec per routed pair; it has no launcher of
 * this shape. The host mirror of MmqRouting uses it while an expert's run stays short. */
int lk_moe_q4k_rows_grouped(const void* weights, const void* weights_second, int act, const void* q8_1,
                            int stride_blocks, const int32_t* bounds, const int32_t* src_rows,
                            const int32_t* dst_rows, float* output, int ldd, int n_experts,
                            int64_t expert_bytes, int size_n, int size_k, int rows_hint, void* stream);
/* Q6_K weight [size_n rows, size_k] x plain Q8_1 rows [size_m, size_k / 32 blocks] -> output
 * [size_m, size_n] f32 on the int8 matrix unit: the Q6_K member of the family above. The reference
 * has no launcher of this shape (its Q6_K rows go one at a time through vec_dot_q6_K_q8_1,
 * cuda/moe/gguf.cuh:782-816); the host mirror of QKernelMatMul::forward uses it between the mat-vec
 * kernels and the tiled matmul. LK_ERR_ARG, and nothing launched, for rows too long for the kernel's
 * scale table in LDS. */
int lk_dense_q6k_rows(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                      void* stream);
/* Q4_K weight [nrows_x, ncols_x] x ONE plain Q8_1 row -> dst [nrows_x] f32. Name and arguments of the
 * reference's batch-1 matrix-unit mat-vec (cuda/q4k_mmvq_imma.cu:149-175; AMD twin cuda/moe/imma_amd.cu:476;
 * declared src/inference/quantized_cuda/mod.rs:29-40, call site quantize.rs:50-60, switched off there);
 * served by the Q4_K mat-vec launch. ncols_x a multiple of 256; nothing is launched otherwise. */
void q4k_mmvq_imma(const void* vx, const void* vy, void* dst, int ncols_x, int nrows_x, void* stream);
/* Q4_K expert rows for a handful of routed pairs per expert, over Q8_1 rows the caller quantized.
 * gate_up: gate_up_weights [num_experts, 2 size_n, size_k] (an expert's gate rows, then its up
 * rows); q8_1 one row per token [size_m / topk, size_k / 32 blocks]; expert_ids one expert PER PAIR;
 * output[sorted_token_ids[pair], :] = gelu_tanh(gate . x) * (up . x). Replaces
 * loken_moe_q4k_imma_m8_gate_up (declared src/inference/moe_cuda/mod.rs:444-447; launcher
 * cuda/moe/moe_q4k_imma_m8.cu:312-335; caller src/inference/moe_cuda/dense/imma.rs:140-190). A pair
 * whose expert is out of range leaves its row untouched, as there. */
void loken_moe_q4k_imma_m8_gate_up(const void* gate_up_weights, const void* q8_1,
                                   const int32_t* sorted_token_ids, const int32_t* expert_ids, float* output,
                                   int num_experts, int topk, int size_m, int size_n, int size_k, void* stream);
/* The same launch with a status. */
int lk_moe_q4k_rows_gate_up(const void* gate_up_weights, const void* q8_1, const int32_t* sorted_token_ids,
                            const int32_t* expert_ids, float* output, int num_experts, int topk, int size_m,
                            int size_n, int size_k, void* stream);
/* down: weights [num_experts, hidden, size_k]; q8_1 one row per routed pair at the pair's slot
 * [size_m, size_k / 32 blocks]; each pair's row is scaled by topk_weights[slot] and the rows of a
 * token are added into output [size_m / topk, hidden] in slot order (output is accumulated into, as
 * loken_moe_sum_topk does). Replaces loken_moe_q4k_imma_m8_down (declared
 * src/inference/moe_cuda/mod.rs:448-451; launcher cuda/moe/moe_q4k_imma_m8_down.cu:238-276). Returns 0,
 * or non-zero when the pair rows' scratch cannot be had (the reference returns 1 there). */
int loken_moe_q4k_imma_m8_down(const void* weights, const void* q8_1, const int32_t* sorted_token_ids,
                               const int32_t* expert_ids, const float* topk_weights, float* output,
                               int num_experts, int topk, int size_m, int hidden, int size_k, void* stream);
/* The router step in front of the expert block: softmax over each row of logits [n_rows,
 * n_experts], the n_expert_used largest probabilities in descending order (ties to the lower
 * expert id) into weights / ids [n_rows, n_expert_used], divided by their sum when with_norm != 0.
 * Name and arguments of the reference's launcher (cuda/moe/gate_topk.cu:405-451; topk_softmax,
 * src/inference/moe_cuda_cpu/mod.rs:2098-2113). Up to 512 experts, up to 64 used; nothing is
 * launched outside that (the caller falls back). */
void loken_topk_softmax(const float* logits, float* weights, uint32_t* ids, int n_rows, int n_experts,
                        int n_expert_used, int with_norm, void* stream);
/* Gate mat-vec + softmax + top-k of each token in one launch: logits = gate_w [n_experts, hidden]
 * f32 . x [n_rows, hidden] f32, then the selection of loken_topk_softmax. A token has a workgroup
 * of 16 waves whose lanes walk each weight row together, so a logit is a 64-lane f32 sum (the
 * reference's is one lane's serial sum: same value up to summation order). Name and arguments of
 * the reference's launcher (cuda/moe/gate_topk.cu:366-403; called from
 * src/inference/moe_cuda/dense/gate.rs:51). hidden up to 8192, up to 512 experts (the reference:
 * 32/64/128/256); nothing is launched outside that (the caller falls back). */
void loken_gate_topk_softmax(const float* x_in, const float* gate_w, float* weights_out, uint32_t* ids_out,
                             int hidden, int n_rows, int n_experts, int n_expert_used, int with_norm, void* stream);
/* Sigmoid router over logits [n_rows, n_experts]: p = 1 / (1 + exp(-logit)); the n_expert_used
 * experts with the largest p + bias[expert] (bias nullable; ties to the lower id), weights = the
 * unbiased p, divided by max(their sum, 2^-14) when with_norm != 0, then times `scale`. Name and
 * arguments of the reference's launcher (cuda/moe/gate_topk.cu:140-200, 479-512; called from
 * src/inference/moe_cuda/dense/gate.rs:133). exp is the accurate one (the reference's is the fast
 * intrinsic). */
void loken_topk_sigmoid_post(const float* logits_in, const float* bias, float* weights_out, uint32_t* ids_out,
                             int n_rows, int n_experts, int n_expert_used, int with_norm, float scale, void* stream);
/* Stable ascending sort of n u32 keys by rank: sorted[r] = the key, order[r] = the index it came
 * from; equal keys keep their order. Groups the routing's (token, choice) pairs by expert on the
 * device (cuda/moe/gate_topk.cu:515-548; called from src/inference/moe_cuda/routing.rs:223). */
void loken_stable_sort_u32(const uint32_t* keys, uint32_t* sorted, uint32_t* order, int n, void* stream);
/* The decode-size form (cuda/moe/gate_topk.cu:453-477; src/inference/moe_cuda/dense/gate.rs:185):
 * same result for m keys; the reference serves m <= 32, this m <= 256, nothing is launched above. */
void loken_argsort_small_u32(const uint32_t* in, uint32_t* sorted_out, uint32_t* index_out, int m, void* stream);
/* Frees the current device's MoE decode scratch (cuda/moe/moe_gguf.cu:104-118). Synchronizes. */
void loken_stream_scratch_release(void);

/* Makes every LK_TUNE_* / LK_MMQ_* environment override (launch shapes and path choices of
 * measurement runs and A/B tests; none changes what a result means) be read again. The launchers
 * read each once and keep it; a process that changes its environment while it runs calls this.
 * No counterpart in the reference. */
void lk_tune_refresh(void);

#ifdef __cplusplus
}
#endif
#endif

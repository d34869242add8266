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
 *     (launch_mmq_*, loken_moe_*): src/tensor/quantized/mmq.rs, src/inference/moe_cuda/*.rs;
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
#define LK_TYPE_Q8_0 8
#define LK_TYPE_Q8_1 9
#define LK_TYPE_Q4_K 12
#define LK_TYPE_Q6_K 14
#define LK_TYPE_BF16 30

#define LK_OK 0
#define LK_ERR_ARG 1        /* a size, stride or pointer the kernels cannot take */
#define LK_ERR_TYPE 2       /* weight / activation / output type not served */
#define LK_ERR_LAUNCH 3     /* the HIP runtime refused the launch */
#define LK_ERR_NOMEM 4      /* scratch could not be reserved (MoE decode launchers only) */

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
 *   wtype          LK_TYPE_Q4_K | LK_TYPE_Q6_K | LK_TYPE_Q8_0
 *   vx             nrows_x rows of ncols_x / block_len blocks
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

/* Parity probe: the exact integer sub-block dot products the mat-vec kernels form, for ONE
 * activation row. dots: Q4_K int32[nrows_x][ncols_x/32] (sum over 32 of nibble*q8),
 * Q6_K int32[nrows_x][ncols_x/16] (sum over 16 of (code-32)*q8), Q8_0 int32[nrows_x][ncols_x/32].
 * sums (nullable): int32[ncols_x/32], sum over 32 of q8. Same device functions as lk_mmvq.
 * No counterpart in the reference: it exists so a test can compare integers bit for bit with
 * the inner sums of BlockQ4K::dot_scalar and friends (format/q4_k.rs:62-88, q6_k.rs:51-82,
 * q8_0.rs:83-97). */
int lk_mmvq_subdots(int wtype, const void* vx, const void* vy_q8_1, int32_t* dots, int32_t* sums,
                    int ncols_x, int nrows_x, void* stream);

#ifdef __cplusplus
}
#endif
#endif

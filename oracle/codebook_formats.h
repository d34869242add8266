/* CPU oracle, test infrastructure only: the codebook expert formats (codebook_formats.c). */
#ifndef LKO_CODEBOOK_FORMATS_H
#define LKO_CODEBOOK_FORMATS_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (src/tensor/quantized/dtype.rs:83-89) */
enum { LKO_IQ2_XXS = 16, LKO_IQ3_XXS = 18, LKO_IQ3_S = 21, LKO_IQ2_S = 22, LKO_Q2_0 = 42 };

int lko_cb_is(int dtype);
int lko_cb_block_len(int dtype);
int lko_cb_block_bytes(int dtype);
/* Run `run` (thirty-two values) of one block: the signed integer weights and the scale of each half. */
int lko_cb_run(int dtype, const uint8_t* blk, int run, int8_t v[32], float s[2]);
int lko_cb_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out);
int lko_cb_dequantize_f64(int dtype, const uint8_t* blocks, size_t n_blocks, double* out);
void lko_cb_half_dots(int dtype, const uint8_t* blk, int run, const int8_t* acts, int32_t out[2]);
float lko_cb_dot(int dtype, const uint8_t* w, const uint8_t* y, size_t nb);
/* The expanded grid of a format (u32 or u64 entries) and its size in bytes. */
const void* lko_cb_table(int dtype, size_t* bytes);

#ifdef __cplusplus
}
#endif
#endif

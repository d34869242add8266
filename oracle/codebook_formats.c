/* CPU oracle, test infrastructure only: the codebook formats the reference's expert kernels serve
 * beside the K-quants (wire ids 11..15, src/inference/moe_cuda/gemm.rs:23-39): IQ3_XXS, IQ3_S,
 * IQ2_S, Q2_0, IQ2_XXS. Each is stated as runs of thirty-two integer weights under a scale per half
 * run (the two halves share it everywhere but in IQ2_S), which is how loken's readers state them
 * (Runs::run_values / run_scale, src/tensor/quant_cpu/format/iq_read.rs:27-33):
 *
 *   IQ3_XXS  98 B  {d, codes[64], tail[8] u32}: iq3_xxs.rs:27-55, 186-213
 *   IQ3_S   110 B  {d, qs[64], qh[8], signs[32], scales[4]}: iq3_s.rs:38-70
 *   IQ2_S    82 B  {d, qs[32] + signs[32], qh[8], scales[8]}: iq2_s.rs:33-57
 *   IQ2_XXS  66 B  {d, qs[32] u16}: iq2_xxs.rs:32-56
 *   Q2_0     18 B  {d, qs[16]}, 64 values, (code - 1) * d: q2_0.rs:33-42
 *
 * The activation side of all five is runs of thirty-two codes quantized as Q8_1 quantizes (BlockQ8K32,
 * q8_k32.rs:44-57; BlockQ8_64, q8_64.rs:47-63), so the served CPU dot and the card's dot
 * (cuda/moe/gguf_iq.cuh:309-418) read the same codes and differ in the order of three float products. */
#include "codebook_formats.h"

#include <string.h>

#include "codebook_tables.h"
#include "loken_oracle.h"

static uint32_t g_iq3xxs[256], g_iq3s[512];
static uint64_t g_iq2xxs[256], g_iq2s[1024];
static int g_ready;

static void expand_tables(void) {
    static const uint8_t l2[3] = {8, 25, 43};
    static const uint8_t l3xxs[8] = {4, 12, 20, 28, 36, 44, 52, 62};
    if (g_ready) return;
    for (int i = 0; i < 256; ++i) {
        uint64_t v = 0;
        for (int b = 0; b < 8; ++b) v |= (uint64_t)l2[(LKO_IQ2XXS_PACKED[i] >> (2 * b)) & 3] << (8 * b);
        g_iq2xxs[i] = v;
    }
    for (int i = 0; i < 1024; ++i) {
        uint64_t v = 0;
        for (int b = 0; b < 8; ++b) v |= (uint64_t)l2[(LKO_IQ2S_PACKED[i] >> (2 * b)) & 3] << (8 * b);
        g_iq2s[i] = v;
    }
    for (int i = 0; i < 256; ++i) {
        uint32_t v = 0;
        for (int b = 0; b < 4; ++b) v |= (uint32_t)l3xxs[(LKO_IQ3XXS_PACKED[i] >> (3 * b)) & 7] << (8 * b);
        g_iq3xxs[i] = v;
    }
    for (int i = 0; i < 512; ++i) {
        uint32_t v = 0;
        for (int b = 0; b < 4; ++b) v |= (uint32_t)(2 * ((LKO_IQ3S_PACKED[i] >> (3 * b)) & 7) + 1) << (8 * b);
        g_iq3s[i] = v;
    }
    g_ready = 1;
}

const void* lko_cb_table(int dtype, size_t* bytes) {
    expand_tables();
    switch (dtype) {
        case LKO_IQ2_XXS: *bytes = sizeof g_iq2xxs; return g_iq2xxs;
        case LKO_IQ2_S: *bytes = sizeof g_iq2s; return g_iq2s;
        case LKO_IQ3_XXS: *bytes = sizeof g_iq3xxs; return g_iq3xxs;
        case LKO_IQ3_S: *bytes = sizeof g_iq3s; return g_iq3s;
        default: *bytes = 0; return NULL;
    }
}

int lko_cb_is(int dtype) {
    return dtype == LKO_IQ2_XXS || dtype == LKO_IQ2_S || dtype == LKO_IQ3_XXS || dtype == LKO_IQ3_S || dtype == LKO_Q2_0;
}
int lko_cb_block_len(int dtype) { return dtype == LKO_Q2_0 ? 64 : lko_cb_is(dtype) ? 256 : 0; }
int lko_cb_block_bytes(int dtype) {
    switch (dtype) {
        case LKO_IQ2_XXS: return 66;
        case LKO_IQ2_S: return 82;
        case LKO_IQ3_XXS: return 98;
        case LKO_IQ3_S: return 110;
        case LKO_Q2_0: return 18;
        default: return 0;
    }
}

/* The 7-bit sign patterns of IQ2_XXS / IQ3_XXS: the eighth sign makes the count of negations even
 * (KSIGNS_IQ2XS, iq2_xxs.rs:584-594, is this rule tabulated). */
static inline uint8_t signs_of7(uint32_t s7) {
    s7 &= 127;
    return (uint8_t)(s7 | ((uint32_t)(__builtin_popcount(s7) & 1) << 7));
}
static inline uint32_t rd32(const uint8_t* p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
static inline float rd_d(const uint8_t* p) { return lko_f16_to_f32((uint16_t)(p[0] | (p[1] << 8))); }
static inline void put8(int8_t* v, uint64_t grid, int count, uint8_t signs) {
    for (int j = 0; j < count; ++j) {
        const int8_t mag = (int8_t)((grid >> (8 * j)) & 0xFF);
        v[j] = ((signs >> j) & 1) ? (int8_t)-mag : mag;
    }
}

int lko_cb_run(int dtype, const uint8_t* blk, int run, int8_t v[32], float s[2]) {
    expand_tables();
    const float d = rd_d(blk);
    switch (dtype) {
        case LKO_IQ3_XXS: {
            const uint8_t* codes = blk + 2 + 8 * run;
            const uint32_t word = rd32(blk + 2 + 64 + 4 * run);
            s[0] = s[1] = d * (0.5f + (float)(word >> 28)) * 0.5f;
            for (int l = 0; l < 4; ++l) {
                const uint8_t sg = signs_of7(word >> (7 * l));
                put8(v + 8 * l, g_iq3xxs[codes[2 * l]], 4, sg);
                put8(v + 8 * l + 4, g_iq3xxs[codes[2 * l + 1]], 4, (uint8_t)(sg >> 4));
            }
            return 0;
        }
        case LKO_IQ3_S: {
            const uint8_t* q = blk + 2 + 8 * run;
            const uint32_t qh = blk[2 + 64 + run];
            const uint8_t* signs = blk + 2 + 64 + 8 + 4 * run;
            const uint8_t sc = blk[2 + 64 + 8 + 32 + run / 2];
            const int scale = (run % 2 == 0) ? (sc & 0x0F) : (sc >> 4);
            s[0] = s[1] = d * (float)(1 + 2 * scale);
            for (int l = 0; l < 4; ++l) {
                const uint32_t i1 = q[2 * l] | ((qh << (8 - 2 * l)) & 256), i2 = q[2 * l + 1] | ((qh << (7 - 2 * l)) & 256);
                put8(v + 8 * l, g_iq3s[i1], 4, signs[l]);
                put8(v + 8 * l + 4, g_iq3s[i2], 4, (uint8_t)(signs[l] >> 4));
            }
            return 0;
        }
        case LKO_IQ2_S: {
            const uint8_t* qs = blk + 2;
            const uint8_t* signs = qs + 32;
            const uint32_t qh = blk[2 + 64 + run];
            const uint8_t sc = blk[2 + 64 + 8 + run];
            s[0] = d * (0.5f + (float)(sc & 0x0F)) * 0.25f;
            s[1] = d * (0.5f + (float)(sc >> 4)) * 0.25f;
            for (int l = 0; l < 4; ++l) {
                const uint32_t code = qs[4 * run + l] | ((qh << (8 - 2 * l)) & 0x300);
                put8(v + 8 * l, g_iq2s[code], 8, signs[4 * run + l]);
            }
            return 0;
        }
        case LKO_IQ2_XXS: {
            const uint32_t lo = rd32(blk + 2 + 8 * run), hi = rd32(blk + 2 + 8 * run + 4);
            s[0] = s[1] = d * (0.5f + (float)(hi >> 28)) * 0.25f;
            for (int l = 0; l < 4; ++l) put8(v + 8 * l, g_iq2xxs[(lo >> (8 * l)) & 0xFF], 8, signs_of7(hi >> (7 * l)));
            return 0;
        }
        case LKO_Q2_0: {
            s[0] = s[1] = d;
            for (int j = 0; j < 32; ++j) {
                const int at = 32 * run + j;
                v[j] = (int8_t)(((blk[2 + at / 4] >> (2 * (at % 4))) & 3) - 1);
            }
            return 0;
        }
        default: return -3;
    }
}

int lko_cb_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out) {
    const int len = lko_cb_block_len(dtype), bytes = lko_cb_block_bytes(dtype);
    if (!len) return -3;
    for (size_t b = 0; b < n_blocks; ++b)
        for (int run = 0; run < len / 32; ++run) {
            int8_t v[32];
            float s[2];
            lko_cb_run(dtype, blocks + b * (size_t)bytes, run, v, s);
            /* db * magnitude * (+-1) in the reference: the sign is exact, so db * (float)(signed value) */
            for (int j = 0; j < 32; ++j) out[b * (size_t)len + 32 * run + j] = s[j / 16] * (float)v[j];
        }
    return 0;
}

int lko_cb_dequantize_f64(int dtype, const uint8_t* blocks, size_t n_blocks, double* out) {
    const int len = lko_cb_block_len(dtype), bytes = lko_cb_block_bytes(dtype);
    if (!len) return -3;
    for (size_t b = 0; b < n_blocks; ++b) {
        const uint8_t* blk = blocks + b * (size_t)bytes;
        const double d = rd_d(blk);
        for (int run = 0; run < len / 32; ++run) {
            int8_t v[32];
            float s[2];
            lko_cb_run(dtype, blk, run, v, s);
            /* the scale from its integer fields in f64: no f32 rounding of d * (0.5 + sc) * 0.5 */
            double f[2];
            if (dtype == LKO_IQ3_XXS) f[0] = f[1] = d * (0.5 + (double)(rd32(blk + 66 + 4 * run) >> 28)) * 0.5;
            else if (dtype == LKO_IQ3_S) {
                const uint8_t sc = blk[106 + run / 2];
                f[0] = f[1] = d * (double)(1 + 2 * ((run % 2 == 0) ? (sc & 0x0F) : (sc >> 4)));
            } else if (dtype == LKO_IQ2_S) {
                f[0] = d * (0.5 + (double)(blk[74 + run] & 0x0F)) * 0.25;
                f[1] = d * (0.5 + (double)(blk[74 + run] >> 4)) * 0.25;
            } else if (dtype == LKO_IQ2_XXS) f[0] = f[1] = d * (0.5 + (double)(rd32(blk + 2 + 8 * run + 4) >> 28)) * 0.25;
            else f[0] = f[1] = d;
            for (int j = 0; j < 32; ++j) out[b * (size_t)len + 32 * run + j] = f[j / 16] * (double)v[j];
        }
    }
    return 0;
}

/* The integer dots of the two halves of run `run` against thirty-two activation codes. */
void lko_cb_half_dots(int dtype, const uint8_t* blk, int run, const int8_t* acts, int32_t out[2]) {
    int8_t v[32];
    float s[2];
    lko_cb_run(dtype, blk, run, v, s);
    out[0] = out[1] = 0;
    for (int j = 0; j < 32; ++j) out[j / 16] += (int32_t)v[j] * (int32_t)acts[j];
}

/* One weight row against one activation row (Q8_1 blocks: f16 d, f16 s, 32 codes), the float steps of the
 * reference's scalar dots:
 *   IQ3_XXS, IQ3_S (dot_runs, iq_read.rs:37-48):  total += run_scale * dot * y.d
 *   IQ2_XXS (iq2_xxs_dot.rs:141-170):             acc += ((0.5 + sc) * 0.25) * sum * y.d per run; total + d * acc per block, from -0.0
 *   IQ2_S (iq2_s.rs:72-117):                      block += (d*(0.5+lo)*0.25*half0 + d*(0.5+hi)*0.25*half1) * y.d; blocks summed
 *   Q2_0 (q2_0.rs:113-129):                       total += dot * d * y.d per half */
float lko_cb_dot(int dtype, const uint8_t* w, const uint8_t* y, size_t nb) {
    const int len = lko_cb_block_len(dtype), bytes = lko_cb_block_bytes(dtype), runs = len / 32;
    float total = dtype == LKO_IQ2_XXS ? -0.0f : 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* blk = w + b * (size_t)bytes;
        float block = 0.0f;
        for (int run = 0; run < runs; ++run) {
            const uint8_t* yb = y + (b * (size_t)runs + (size_t)run) * LKO_Q81_BYTES;
            const float yd = rd_d(yb);
            int8_t v[32];
            float s[2];
            lko_cb_run(dtype, blk, run, v, s);
            int32_t half[2] = {0, 0};
            const int8_t* a = (const int8_t*)(yb + 4);
            for (int j = 0; j < 32; ++j) half[j / 16] += (int32_t)v[j] * (int32_t)a[j];
            const int32_t dot = half[0] + half[1];
            if (dtype == LKO_IQ2_S) block += (s[0] * (float)half[0] + s[1] * (float)half[1]) * yd;
            else if (dtype == LKO_IQ2_XXS) {
                const float scale = (0.5f + (float)(rd32(blk + 2 + 8 * run + 4) >> 28)) * 0.25f;
                block += scale * (float)dot * yd;
            } else if (dtype == LKO_Q2_0) total += (float)dot * s[0] * yd;
            else total += s[0] * (float)dot * yd;
        }
        if (dtype == LKO_IQ2_S) total += block;
        else if (dtype == LKO_IQ2_XXS) total = total + rd_d(blk) * block;
    }
    return total;
}

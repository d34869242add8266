/*
 * CPU oracle for the GGUF block-quantized matmul path. TEST INFRASTRUCTURE ONLY: see
 * loken_oracle.h for what it restates, what pins it, and who may call it.
 *
 * Build with -ffp-contract=off: the Rust reference never fuses a multiply and an add, so
 * neither may this file.
 */
#include "loken_oracle.h"
#include "codebook_formats.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------
 * f16 <-> f32. The reference uses the `half` crate (IEEE binary16, round to nearest even);
 * the `d` bytes of scripts/oracle/vectors.txt pin both directions.
 * ---------------------------------------------------------------------------------------- */
float lko_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t lko_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (absx > 0x7F800000u ? 0x0200u | ((absx >> 13) & 0x3FFu) : 0));
    }
    if (absx >= 0x477FF000u) { /* rounds to >= 65520: overflow to inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x33000001u) { /* below half the smallest subnormal: zero */
        return sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;
    uint32_t shift, half_bits;
    if (e < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        const uint32_t q = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1u);
        const uint32_t halfway = 1u << (shift - 1);
        half_bits = q;
        if (rem > halfway || (rem == halfway && (q & 1u))) half_bits += 1;
        return (uint16_t)(sign | half_bits);
    }
    shift = 13;
    {
        const uint32_t q = ((uint32_t)(e + 15) << 10) | ((man >> shift) & 0x3FFu);
        const uint32_t rem = man & 0x1FFFu;
        half_bits = q;
        if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) half_bits += 1; /* carry may bump exp */
    }
    return (uint16_t)(sign | half_bits);
}

int lko_block_len(int dtype) {
    switch (dtype) {
        case LKO_Q8_0: case LKO_Q8_1: case LKO_Q4_0: case LKO_Q4_1: case LKO_Q5_0: case LKO_Q5_1:
        case LKO_IQ4_NL: case LKO_MXFP4: return 32;
        case LKO_Q2_K: case LKO_Q3_K: case LKO_Q4_K: case LKO_Q5_K: case LKO_Q6_K: case LKO_Q8_K: case LKO_IQ4_XS: return 256;
        default: return lko_cb_block_len(dtype);
    }
}

int lko_block_bytes(int dtype) {
    switch (dtype) {
        case LKO_Q8_0: return LKO_Q80_BYTES;
        case LKO_Q4_0: return 18;
        case LKO_Q4_1: return 20;
        case LKO_Q5_0: return 22;
        case LKO_Q5_1: return 24;
        case LKO_IQ4_NL: return 18;
        case LKO_MXFP4: return 17;
        case LKO_Q8_1: return LKO_Q81_BYTES;
        case LKO_Q2_K: return 84;
        case LKO_IQ4_XS: return 136;
        case LKO_Q3_K: return 110;
        case LKO_Q4_K: return LKO_Q4K_BYTES;
        case LKO_Q5_K: return LKO_Q5K_BYTES;
        case LKO_Q6_K: return LKO_Q6K_BYTES;
        case LKO_Q8_K: return LKO_Q8K_BYTES;
        default: return lko_cb_block_bytes(dtype);
    }
}

static inline uint16_t rd_u16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline void wr_u16(uint8_t* p, uint16_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); }
static inline float rd_f32(const uint8_t* p) { float f; memcpy(&f, p, 4); return f; }

/* scale.rs:15-17: f32::round is half away from zero, as roundf. `as i32` saturates. */
static inline int32_t nearest_int(float v) {
    const float r = roundf(v);
    if (r >= 2147483648.0f) return INT32_MAX;
    if (r <= -2147483648.0f) return INT32_MIN;
    if (r != r) return 0;
    return (int32_t)r;
}
/* Rust `f32 as i8` saturates and maps NaN to 0. */
static inline int8_t sat_i8(float r) {
    if (r != r) return 0;
    if (r >= 127.0f) return 127;
    if (r <= -128.0f) return -128;
    return (int8_t)r;
}

/* blocks.rs:145-158 */
void lko_unpack_scales_mins(const uint8_t packed[12], uint8_t scales[8], uint8_t mins[8]) {
    for (int i = 0; i < 4; ++i) {
        scales[i] = packed[i] & 0x3F;
        mins[i] = packed[i + 4] & 0x3F;
    }
    for (int i = 4; i < 8; ++i) {
        const uint8_t low = packed[i + 4];
        scales[i] = (uint8_t)((low & 0x0F) | ((packed[i - 4] >> 6) << 4));
        mins[i] = (uint8_t)((low >> 4) | ((packed[i] >> 6) << 4));
    }
}

/* blocks.rs:167-179 */
void lko_pack_scales_mins(const uint8_t scales[8], const uint8_t mins[8], uint8_t packed[12]) {
    memset(packed, 0, 12);
    for (int i = 0; i < 4; ++i) {
        packed[i] = scales[i] & 0x3F;
        packed[i + 4] = mins[i] & 0x3F;
    }
    for (int i = 4; i < 8; ++i) {
        packed[i + 4] = (uint8_t)((scales[i] & 0x0F) | ((mins[i] & 0x0F) << 4));
        packed[i - 4] |= (uint8_t)((scales[i] >> 4) << 6);
        packed[i] |= (uint8_t)((mins[i] >> 4) << 6);
    }
}

/* Field offsets. Q4_K: d@0 dmin@2 scales@4 qs@16 (q4_k.rs:12-20).
 * Q5_K: d@0 dmin@2 scales@4 qh@16 qs@48 (q5_k.rs:10-16); a value is its Q4_K nibble plus bit s of
 * qh[l] as the fifth bit (q5_k.rs:66-71, 105-106).
 * Q6_K: ql@0 qh@128 scales@192 d@208 (q6_k.rs:8-16). Q8_0: d@0 qs@2. Q8_1: d@0 s@2 qs@4.
 * Q8_K: d(f32)@0 qs@4 bsums@260 (q8_k.rs:13-20). */

/* The signed six-bit code of element `l` of group `g` of half `h` (q6_k.rs:62-70). */
static inline int q6k_code(const uint8_t* blk, int h, int g, int l) {
    const uint8_t* ql = blk + 64 * h;
    const uint8_t* qh = blk + 128 + 32 * h;
    const int span = 32 * (g % 2);
    const int nibble = g < 2 ? 0 : 4;
    const int low = (ql[span + l] >> nibble) & 0x0F;
    const int high = (qh[l] >> (2 * g)) & 0x03;
    return (low | (high << 4)) - 32;
}

/* The five-bit code of element `l` of sub-block `s` (q5_k.rs:66-71). */
static inline int q5k_code(const uint8_t* blk, int s, int l) {
    const uint8_t packed = blk[48 + (s / 2) * 32 + l];
    const int shift = (s % 2 == 0) ? 0 : 4;
    const int fifth = (blk[16 + l] >> s) & 1;
    return ((packed >> shift) & 0x0F) | (fifth << 4);
}

static int legacy_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out);
static int lowbit_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out);
static int iq4xs_dequantize(const uint8_t* blocks, size_t n_blocks, float* out);

int lko_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out) {
    switch (dtype) {
    case LKO_Q4_K: /* q4_k.rs:98-114 */
        for (size_t b = 0; b < n_blocks; ++b) {
            const uint8_t* blk = blocks + b * LKO_Q4K_BYTES;
            float* y = out + b * 256;
            const float d = lko_f16_to_f32(rd_u16(blk));
            const float dmin = lko_f16_to_f32(rd_u16(blk + 2));
            uint8_t sc[8], mn[8];
            lko_unpack_scales_mins(blk + 4, sc, mn);
            for (int s = 0; s < 8; ++s) {
                const uint8_t* group = blk + 16 + (s / 2) * 32;
                const int shift = (s % 2 == 0) ? 0 : 4;
                const float scale = d * (float)sc[s];
                const float offset = dmin * (float)mn[s];
                for (int l = 0; l < 32; ++l) {
                    y[s * 32 + l] = scale * (float)((group[l] >> shift) & 0x0F) - offset;
                }
            }
        }
        return 0;
    case LKO_Q5_K: /* q5_k.rs:95-112 */
        for (size_t b = 0; b < n_blocks; ++b) {
            const uint8_t* blk = blocks + b * LKO_Q5K_BYTES;
            float* y = out + b * 256;
            const float d = lko_f16_to_f32(rd_u16(blk));
            const float dmin = lko_f16_to_f32(rd_u16(blk + 2));
            uint8_t sc[8], mn[8];
            lko_unpack_scales_mins(blk + 4, sc, mn);
            for (int s = 0; s < 8; ++s) {
                const float scale = d * (float)sc[s];
                const float offset = dmin * (float)mn[s];
                for (int l = 0; l < 32; ++l) y[s * 32 + l] = scale * (float)q5k_code(blk, s, l) - offset;
            }
        }
        return 0;
    case LKO_Q6_K: /* q6_k.rs:98-118 */
        for (size_t b = 0; b < n_blocks; ++b) {
            const uint8_t* blk = blocks + b * LKO_Q6K_BYTES;
            float* y = out + b * 256;
            const float d = lko_f16_to_f32(rd_u16(blk + 208));
            const int8_t* scales = (const int8_t*)(blk + 192);
            for (int h = 0; h < 2; ++h)
                for (int g = 0; g < 4; ++g)
                    for (int l = 0; l < 32; ++l) {
                        const int q = q6k_code(blk, h, g, l);
                        y[128 * h + 32 * g + l] = d * (float)scales[8 * h + 2 * g + l / 16] * (float)q;
                    }
        }
        return 0;
    case LKO_Q8_0: /* q8_0.rs:42-49 */
        for (size_t b = 0; b < n_blocks; ++b) {
            const uint8_t* blk = blocks + b * LKO_Q80_BYTES;
            const float d = lko_f16_to_f32(rd_u16(blk));
            for (int l = 0; l < 32; ++l) out[b * 32 + l] = (float)(int8_t)blk[2 + l] * d;
        }
        return 0;
    case LKO_Q8_1: /* q8_1.rs:37-44 */
        for (size_t b = 0; b < n_blocks; ++b) {
            const uint8_t* blk = blocks + b * LKO_Q81_BYTES;
            const float d = lko_f16_to_f32(rd_u16(blk));
            for (int l = 0; l < 32; ++l) out[b * 32 + l] = (float)(int8_t)blk[4 + l] * d;
        }
        return 0;
    case LKO_Q8_K: /* q8_k.rs:42-48 */
        for (size_t b = 0; b < n_blocks; ++b) {
            const uint8_t* blk = blocks + b * LKO_Q8K_BYTES;
            const float d = rd_f32(blk);
            for (int l = 0; l < 256; ++l) out[b * 256 + l] = (float)(int8_t)blk[4 + l] * d;
        }
        return 0;
    case LKO_Q2_K: case LKO_Q3_K:
        return lowbit_dequantize(dtype, blocks, n_blocks, out);
    case LKO_IQ4_XS:
        return iq4xs_dequantize(blocks, n_blocks, out);
    case LKO_IQ2_XXS: case LKO_IQ3_XXS: case LKO_IQ3_S: case LKO_IQ2_S: case LKO_Q2_0:
        return lko_cb_dequantize(dtype, blocks, n_blocks, out);
    default:
        return legacy_dequantize(dtype, blocks, n_blocks, out);
    }
}

/* q8_0.rs:51-67 */
void lko_quantize_q8_0(const float* x, size_t n, uint8_t* out) {
    for (size_t b = 0; b < n / 32; ++b) {
        const float* xb = x + b * 32;
        uint8_t* blk = out + b * LKO_Q80_BYTES;
        float amax = 0.0f;
        for (int l = 0; l < 32; ++l) amax = fmaxf(amax, fabsf(xb[l]));
        const float d = amax / 127.0f;
        wr_u16(blk, lko_f32_to_f16(d));
        const float inv = d != 0.0f ? 1.0f / d : 0.0f;
        for (int l = 0; l < 32; ++l) blk[2 + l] = (uint8_t)sat_i8(roundf(xb[l] * inv));
    }
}

/* q8_1.rs:46-61 */
void lko_quantize_q8_1(const float* x, size_t n, uint8_t* out) {
    for (size_t b = 0; b < n / 32; ++b) {
        const float* xb = x + b * 32;
        uint8_t* blk = out + b * LKO_Q81_BYTES;
        float amax = 0.0f;
        for (int l = 0; l < 32; ++l) amax = fmaxf(amax, fabsf(xb[l]));
        const float d = amax / 127.0f;
        wr_u16(blk, lko_f32_to_f16(d));
        const float inv = d != 0.0f ? 1.0f / d : 0.0f;
        int32_t sum = 0;
        for (int l = 0; l < 32; ++l) {
            const int8_t q = sat_i8(roundf(xb[l] * inv));
            blk[4 + l] = (uint8_t)q;
            sum += q;
        }
        wr_u16(blk + 2, lko_f32_to_f16((float)sum * d));
    }
}

/* q8_k.rs:96-119 */
void lko_quantize_q8_k(const float* x, size_t n, uint8_t* out) {
    for (size_t b = 0; b < n / 256; ++b) {
        const float* xb = x + b * 256;
        uint8_t* blk = out + b * LKO_Q8K_BYTES;
        float extreme = 0.0f;
        for (int l = 0; l < 256; ++l)
            if (fabsf(xb[l]) > fabsf(extreme)) extreme = xb[l];
        if (extreme == 0.0f) {
            memset(blk, 0, LKO_Q8K_BYTES);
            continue;
        }
        const float inv = -127.0f / extreme;
        const float d = 1.0f / inv;
        memcpy(blk, &d, 4);
        int8_t* qs = (int8_t*)(blk + 4);
        for (int l = 0; l < 256; ++l) {
            int32_t q = nearest_int(inv * xb[l]);
            if (q > 127) q = 127;
            qs[l] = (int8_t)q; /* `as i8` wraps; unreachable below -128 since |x| <= |extreme| */
        }
        for (int j = 0; j < 16; ++j) {
            int16_t s = 0;
            for (int l = 0; l < 16; ++l) s = (int16_t)(s + qs[16 * j + l]);
            wr_u16(blk + 260 + 2 * j, (uint16_t)s);
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Integer sums shared by both families.
 * ---------------------------------------------------------------------------------------- */

/* q4_k.rs:138-153 inner `dot`: sub-block s of a Q4_K block against 32 activation codes. */
static inline int32_t q4k_sub_dot(const uint8_t* blk, int s, const int8_t* acts) {
    const uint8_t* group = blk + 16 + (s / 2) * 32;
    const int shift = (s % 2 == 0) ? 0 : 4;
    int32_t dot = 0;
    for (int l = 0; l < 32; ++l) dot += (int32_t)((group[l] >> shift) & 0x0F) * (int32_t)acts[l];
    return dot;
}

/* q5_k.rs:62-73 inner `dot`: the same with the fifth bit. */
static inline int32_t q5k_sub_dot(const uint8_t* blk, int s, const int8_t* acts) {
    int32_t dot = 0;
    for (int l = 0; l < 32; ++l) dot += (int32_t)q5k_code(blk, s, l) * (int32_t)acts[l];
    return dot;
}

/* q6_k.rs:137-160: the sixteen per-16 sums of a Q6_K block against 256 activation codes. */
static inline void q6k_sub_dots(const uint8_t* blk, const int8_t* acts256, int32_t per_sub[16]) {
    for (int j = 0; j < 16; ++j) per_sub[j] = 0;
    for (int h = 0; h < 2; ++h)
        for (int g = 0; g < 4; ++g)
            for (int l = 0; l < 32; ++l)
                per_sub[8 * h + 2 * g + l / 16] +=
                    q6k_code(blk, h, g, l) * (int32_t)acts256[128 * h + 32 * g + l];
}

static inline int32_t i8_dot32(const int8_t* a, const int8_t* b) {
    int32_t dot = 0;
    for (int l = 0; l < 32; ++l) dot += (int32_t)a[l] * (int32_t)b[l];
    return dot;
}

/* ------------------------------------------------------------------------------------------
 * O-A row dots (dot_scalar of each format).
 * ---------------------------------------------------------------------------------------- */

/* q4_k.rs:62-88 */
static float oa_dot_q4k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q4K_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        const int8_t* yq = (const int8_t*)(yb + 4);
        uint8_t sc[8], mn[8];
        lko_unpack_scales_mins(x + 4, sc, mn);
        float scaled = 0.0f, offset = 0.0f;
        for (int s = 0; s < 8; ++s) {
            const int32_t dot = q4k_sub_dot(x, s, yq + 32 * s);
            const int32_t bs = (int32_t)(int16_t)rd_u16(yb + 260 + 4 * s) +
                               (int32_t)(int16_t)rd_u16(yb + 260 + 4 * s + 2);
            scaled += (float)sc[s] * (float)dot;
            offset += (float)mn[s] * (float)bs;
        }
        total += rd_f32(yb) * (lko_f16_to_f32(rd_u16(x)) * scaled - lko_f16_to_f32(rd_u16(x + 2)) * offset);
    }
    return total;
}

/* q5_k.rs:51-80 */
static float oa_dot_q5k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q5K_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        const int8_t* yq = (const int8_t*)(yb + 4);
        uint8_t sc[8], mn[8];
        lko_unpack_scales_mins(x + 4, sc, mn);
        float scaled = 0.0f, offset = 0.0f;
        for (int s = 0; s < 8; ++s) {
            const int32_t dot = q5k_sub_dot(x, s, yq + 32 * s);
            const int32_t bs = (int32_t)(int16_t)rd_u16(yb + 260 + 4 * s) +
                               (int32_t)(int16_t)rd_u16(yb + 260 + 4 * s + 2);
            scaled += (float)sc[s] * (float)dot;
            offset += (float)mn[s] * (float)bs;
        }
        total += rd_f32(yb) * (lko_f16_to_f32(rd_u16(x)) * scaled - lko_f16_to_f32(rd_u16(x + 2)) * offset);
    }
    return total;
}

/* q6_k.rs:51-82 */
static float oa_dot_q6k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q6K_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        int32_t per_sub[16];
        q6k_sub_dots(x, (const int8_t*)(yb + 4), per_sub);
        const int8_t* scales = (const int8_t*)(x + 192);
        float dot = 0.0f;
        for (int j = 0; j < 16; ++j) dot += (float)per_sub[j] * (float)scales[j];
        total += dot * lko_f16_to_f32(rd_u16(x + 208)) * rd_f32(yb);
    }
    return total;
}

/* q8_0.rs:83-97 */
static float oa_dot_q80(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q80_BYTES;
        const uint8_t* yb = y + b * LKO_Q80_BYTES;
        const int32_t dot = i8_dot32((const int8_t*)(x + 2), (const int8_t*)(yb + 2));
        total += (float)dot * lko_f16_to_f32(rd_u16(x)) * lko_f16_to_f32(rd_u16(yb));
    }
    return total;
}

/* dot_exact: q4_k.rs:117-156, q6_k.rs:121-163. */
static float oa_dot_exact_q4k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = -0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q4K_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        const int8_t* yq = (const int8_t*)(yb + 4);
        uint8_t sc[8], mn[8];
        lko_unpack_scales_mins(x + 4, sc, mn);
        int32_t scaled = 0, offset = 0;
        for (int s = 0; s < 8; ++s) {
            scaled += (int32_t)sc[s] * q4k_sub_dot(x, s, yq + 32 * s);
            offset += (int32_t)mn[s] * ((int32_t)(int16_t)rd_u16(yb + 260 + 4 * s) +
                                        (int32_t)(int16_t)rd_u16(yb + 260 + 4 * s + 2));
        }
        total += rd_f32(yb) * (lko_f16_to_f32(rd_u16(x)) * (float)scaled -
                               lko_f16_to_f32(rd_u16(x + 2)) * (float)offset);
    }
    return total;
}

static float oa_dot_exact_q6k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = -0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q6K_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        int32_t per_sub[16];
        q6k_sub_dots(x, (const int8_t*)(yb + 4), per_sub);
        const int8_t* scales = (const int8_t*)(x + 192);
        int32_t scaled = 0;
        for (int j = 0; j < 16; ++j) scaled += (int32_t)scales[j] * per_sub[j];
        total += rd_f32(yb) * (lko_f16_to_f32(rd_u16(x + 208)) * (float)scaled);
    }
    return total;
}

/* ------------------------------------------------------------------------------------------
 * O-B row dots: weight row against k/32 Q8_1 blocks.
 * ---------------------------------------------------------------------------------------- */

/* gguf.cuh:664-685: per sub-block d8*(dot*sc) and d8*(sum*m); d*scaled - dmin*offset. */
static float ob_dot_q4k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q4K_BYTES;
        uint8_t sc[8], mn[8];
        lko_unpack_scales_mins(x + 4, sc, mn);
        float scaled = 0.0f, offset = 0.0f;
        for (int s = 0; s < 8; ++s) {
            const uint8_t* yb = y + (b * 8 + s) * LKO_Q81_BYTES;
            const int8_t* yq = (const int8_t*)(yb + 4);
            const float d8 = lko_f16_to_f32(rd_u16(yb));
            const int32_t dot = q4k_sub_dot(x, s, yq);
            int32_t sum = 0;
            for (int l = 0; l < 32; ++l) sum += yq[l];
            scaled += d8 * (float)(dot * (int32_t)sc[s]);
            offset += d8 * (float)(sum * (int32_t)mn[s]);
        }
        total += lko_f16_to_f32(rd_u16(x)) * scaled - lko_f16_to_f32(rd_u16(x + 2)) * offset;
    }
    return total;
}

/* gguf.cuh:723-748 (vec_dot_q5_K_q8_1_impl_vmmq): the Q4_K combine over the five-bit codes. */
static float ob_dot_q5k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q5K_BYTES;
        uint8_t sc[8], mn[8];
        lko_unpack_scales_mins(x + 4, sc, mn);
        float scaled = 0.0f, offset = 0.0f;
        for (int s = 0; s < 8; ++s) {
            const uint8_t* yb = y + (b * 8 + s) * LKO_Q81_BYTES;
            const int8_t* yq = (const int8_t*)(yb + 4);
            const float d8 = lko_f16_to_f32(rd_u16(yb));
            const int32_t dot = q5k_sub_dot(x, s, yq);
            int32_t sum = 0;
            for (int l = 0; l < 32; ++l) sum += yq[l];
            scaled += d8 * (float)(dot * (int32_t)sc[s]);
            offset += d8 * (float)(sum * (int32_t)mn[s]);
        }
        total += lko_f16_to_f32(rd_u16(x)) * scaled - lko_f16_to_f32(rd_u16(x + 2)) * offset;
    }
    return total;
}

/* gguf.cuh:782-816: sum over the sixteen runs of d8*(dot*sc), times d. */
static float ob_dot_q6k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q6K_BYTES;
        const int8_t* scales = (const int8_t*)(x + 192);
        int8_t acts[256];
        float d8[8];
        for (int s = 0; s < 8; ++s) {
            const uint8_t* yb = y + (b * 8 + s) * LKO_Q81_BYTES;
            memcpy(acts + 32 * s, yb + 4, 32);
            d8[s] = lko_f16_to_f32(rd_u16(yb));
        }
        int32_t per_sub[16];
        q6k_sub_dots(x, acts, per_sub);
        float run = 0.0f;
        for (int j = 0; j < 16; ++j) run += d8[j / 2] * (float)(per_sub[j] * (int32_t)scales[j]);
        total += lko_f16_to_f32(rd_u16(x + 208)) * run;
    }
    return total;
}

/* gguf.cuh:486-495: d8_0 * d8_1 * dot. */
static float ob_dot_q80(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q80_BYTES;
        const uint8_t* yb = y + b * LKO_Q81_BYTES;
        const int32_t dot = i8_dot32((const int8_t*)(x + 2), (const int8_t*)(yb + 4));
        total += lko_f16_to_f32(rd_u16(x)) * lko_f16_to_f32(rd_u16(yb)) * (float)dot;
    }
    return total;
}


/* ------------------------------------------------------------------------------------------
 * The 32-value formats with nibble codes (q4_0.rs, q4_1.rs, q5_0.rs, q5_1.rs): byte j of `qs`
 * holds value j in its low nibble and value j + 16 in its high one; the five-bit formats keep
 * bit v of the little-endian word `qh` as value v's fifth bit. Q4_0 {d, qs} and Q5_0 {d, qh, qs}
 * mean (code - 8 / 16) * d; Q4_1 {d, m, qs} and Q5_1 {d, m, qh, qs} mean code * d + m.
 * ---------------------------------------------------------------------------------------- */
/* IQ4_NL {d, qs} and MXFP4 {e, qs} pack their nibbles the same way but a code names a level of a
 * table: iq4_nl.rs:11-13 (d * LEVELS[code]), mxfp4.rs / blocks.rs:24-42 (KVALUES_MXFP4[code] * the
 * block's E8M0 scale as e8m0_to_fp32_half gives it: 0.5 * 2^(e - 127), denormal patterns below 2). */
static const int8_t LEVELS_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
static const int8_t LEVELS_MXFP4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

static float e8m0_to_f32_half(uint8_t e) {
    const uint32_t bits = e < 2 ? (0x00200000u << e) : ((uint32_t)(e - 1) << 23);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

typedef struct { int bytes, m_at, qh_at, qs_at, bias; const int8_t* levels; } legacy_layout;

static int legacy_layout_of(int dtype, legacy_layout* l) {
    switch (dtype) {
        case LKO_Q4_0: *l = (legacy_layout){18, -1, -1, 2, 8, NULL}; return 1;
        case LKO_Q4_1: *l = (legacy_layout){20, 2, -1, 4, 0, NULL}; return 1;
        case LKO_Q5_0: *l = (legacy_layout){22, -1, 2, 6, 16, NULL}; return 1;
        case LKO_Q5_1: *l = (legacy_layout){24, 2, 4, 8, 0, NULL}; return 1;
        case LKO_IQ4_NL: *l = (legacy_layout){18, -1, -1, 2, 0, LEVELS_IQ4NL}; return 1;
        case LKO_MXFP4: *l = (legacy_layout){17, -1, -1, 1, 0, LEVELS_MXFP4}; return 1;
        default: return 0;
    }
}

/* The unsigned code of value v (q5_0.rs:43-48), or the level it names in a table format. */
static inline float legacy_scale(const uint8_t* blk, int dtype) {
    return dtype == LKO_MXFP4 ? e8m0_to_f32_half(blk[0]) : lko_f16_to_f32(rd_u16(blk));
}

static inline int legacy_code(const uint8_t* blk, const legacy_layout* l, int v) {
    const uint8_t packed = blk[l->qs_at + (v & 15)];
    int code = v < 16 ? (packed & 0x0F) : (packed >> 4);
    if (l->qh_at >= 0) {
        const uint32_t qh = (uint32_t)blk[l->qh_at] | ((uint32_t)blk[l->qh_at + 1] << 8) |
                            ((uint32_t)blk[l->qh_at + 2] << 16) | ((uint32_t)blk[l->qh_at + 3] << 24);
        code |= (int)((qh >> v) & 1u) << 4;
    }
    return l->levels ? (int)l->levels[code] : code;   /* a table format's "code" is its level */
}

/* The integer the CPU dots form (q4_0.rs:104-113, q4_1.rs:104-111): sum of (code - bias) * a. */
static inline int32_t legacy_sub_dot(const uint8_t* blk, const legacy_layout* l, const int8_t* acts) {
    int32_t dot = 0;
    for (int v = 0; v < 32; ++v) dot += (int32_t)(legacy_code(blk, l, v) - l->bias) * (int32_t)acts[v];
    return dot;
}

static int legacy_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out) {
    legacy_layout l;
    if (!legacy_layout_of(dtype, &l)) return -3;
    for (size_t b = 0; b < n_blocks; ++b) {
        const uint8_t* blk = blocks + b * (size_t)l.bytes;
        const float d = legacy_scale(blk, dtype);
        const float m = l.m_at >= 0 ? lko_f16_to_f32(rd_u16(blk + l.m_at)) : 0.0f;
        for (int v = 0; v < 32; ++v) {
            const int code = legacy_code(blk, &l, v);
            out[b * 32 + v] = l.m_at >= 0 ? (float)code * d + m : (float)(code - l.bias) * d;
        }
    }
    return 0;
}

/* Served CPU path: Q4_0 / Q5_0 against Q8_0 blocks, dot * d * y.d (q4_0.rs:96-117); Q4_1 / Q5_1
 * against Q8_1 blocks, dot * d * y.d + m * y.s (q4_1.rs:95-115). */
static float oa_dot_legacy(int dtype, const uint8_t* w, const uint8_t* y, size_t nb) {
    legacy_layout l;
    legacy_layout_of(dtype, &l);
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * (size_t)l.bytes;
        if (l.m_at < 0) {
            const uint8_t* yb = y + b * LKO_Q80_BYTES;
            const int32_t dot = legacy_sub_dot(x, &l, (const int8_t*)(yb + 2));
            total += (float)dot * legacy_scale(x, dtype) * lko_f16_to_f32(rd_u16(yb));
        } else {
            const uint8_t* yb = y + b * LKO_Q81_BYTES;
            const int32_t dot = legacy_sub_dot(x, &l, (const int8_t*)(yb + 4));
            total += (float)dot * lko_f16_to_f32(rd_u16(x)) * lko_f16_to_f32(rd_u16(yb)) +
                     lko_f16_to_f32(rd_u16(x + l.m_at)) * lko_f16_to_f32(rd_u16(yb + 2));
        }
    }
    return total;
}

/* Same codes on the Q8_1 side, the sum of the activation codes taken as the integer it is
 * (cuda/moe/gguf.cuh:436-441 total_biased_codes; :400-405 with the minimum): d * d8 * dot, plus
 * m * (d8 * sum of codes) for the formats with a minimum. */
static float ob_dot_legacy(int dtype, const uint8_t* w, const uint8_t* y, size_t nb) {
    legacy_layout l;
    legacy_layout_of(dtype, &l);
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * (size_t)l.bytes;
        const uint8_t* yb = y + b * LKO_Q81_BYTES;
        const int8_t* yq = (const int8_t*)(yb + 4);
        const float d8 = lko_f16_to_f32(rd_u16(yb));
        const int32_t dot = legacy_sub_dot(x, &l, yq);
        float part = legacy_scale(x, dtype) * d8 * (float)dot;
        if (l.m_at >= 0) {
            int32_t sum = 0;
            for (int v = 0; v < 32; ++v) sum += yq[v];
            part += lko_f16_to_f32(rd_u16(x + l.m_at)) * (d8 * (float)sum);
        }
        total += part;
    }
    return total;
}
static float oa_dot_q40(const uint8_t* w, const uint8_t* y, size_t nb) { return oa_dot_legacy(LKO_Q4_0, w, y, nb); }
static float oa_dot_q41(const uint8_t* w, const uint8_t* y, size_t nb) { return oa_dot_legacy(LKO_Q4_1, w, y, nb); }
static float oa_dot_q50(const uint8_t* w, const uint8_t* y, size_t nb) { return oa_dot_legacy(LKO_Q5_0, w, y, nb); }
static float oa_dot_q51(const uint8_t* w, const uint8_t* y, size_t nb) { return oa_dot_legacy(LKO_Q5_1, w, y, nb); }
static float ob_dot_q40(const uint8_t* w, const uint8_t* y, size_t nb) { return ob_dot_legacy(LKO_Q4_0, w, y, nb); }
static float ob_dot_q41(const uint8_t* w, const uint8_t* y, size_t nb) { return ob_dot_legacy(LKO_Q4_1, w, y, nb); }
static float ob_dot_q50(const uint8_t* w, const uint8_t* y, size_t nb) { return ob_dot_legacy(LKO_Q5_0, w, y, nb); }
static float ob_dot_q51(const uint8_t* w, const uint8_t* y, size_t nb) { return ob_dot_legacy(LKO_Q5_1, w, y, nb); }
static float oa_dot_iq4nl(const uint8_t* w, const uint8_t* y, size_t nb) { return oa_dot_legacy(LKO_IQ4_NL, w, y, nb); }
static float oa_dot_mxfp4(const uint8_t* w, const uint8_t* y, size_t nb) { return oa_dot_legacy(LKO_MXFP4, w, y, nb); }
static float ob_dot_iq4nl(const uint8_t* w, const uint8_t* y, size_t nb) { return ob_dot_legacy(LKO_IQ4_NL, w, y, nb); }
static float ob_dot_mxfp4(const uint8_t* w, const uint8_t* y, size_t nb) { return ob_dot_legacy(LKO_MXFP4, w, y, nb); }


/* ------------------------------------------------------------------------------------------
 * Q2_K {scales[16], qs[64], d, dmin} = 84 bytes (q2_k.rs:15-20) and Q3_K {hmask[32], qs[64],
 * scales[12], d} = 110 bytes (q3_k.rs:10-15): sixteen sub-blocks of sixteen two-bit codes.
 * Sub-block s reads byte 32 * (s / 8) + 16 * (s % 2) + l at shift 2 * ((s % 8) / 2)
 * (q2_k.rs:30-33, q3_k.rs:132-140); positions run 16 s + l, so the 32 values of Q8_1 block j are
 * sub-blocks 2 j and 2 j + 1. Q2_K: d * (sc & 15) * q - dmin * (sc >> 4). Q3_K: d * scale * (q + third),
 * third = -4 where bit j of hmask[16 * (s % 2) + l] is clear; scales six bits less 32 (q3_k.rs:27-37).
 * ---------------------------------------------------------------------------------------- */
static inline int q23k_low(const uint8_t* qs, int s, int l) {
    return (qs[32 * (s / 8) + 16 * (s % 2) + l] >> (2 * ((s % 8) / 2))) & 3;
}
static inline int q3k_value(const uint8_t* blk, int s, int l) {
    const int bit = 4 * (s / 8) + (s % 8) / 2;
    return q23k_low(blk + 32, s, l) + (((blk[16 * (s % 2) + l] >> bit) & 1) ? 0 : -4);
}
static void q3k_scales(const uint8_t* packed, int8_t out[16]) {
    for (int i = 0; i < 16; ++i) {
        const int group = i / 4, j = i % 4;
        const uint8_t byte = packed[j + 4 * (group % 2)];
        const int low = group < 2 ? (byte & 0x0F) : (byte >> 4);
        const int high = (packed[8 + j] >> (2 * group)) & 0x03;
        out[i] = (int8_t)((low | (high << 4)) - 32);
    }
}
/* Sub-block s against its sixteen activation codes: the integers the CPU dots form
 * (q2_k.rs:98-102; q3_k.rs block_sum). */
static inline int32_t q2k_sub_dot(const uint8_t* blk, int s, const int8_t* acts) {
    int32_t dot = 0;
    for (int l = 0; l < 16; ++l) dot += q23k_low(blk + 16, s, l) * (int32_t)acts[l];
    return dot;
}
static inline int32_t q3k_sub_dot(const uint8_t* blk, int s, const int8_t* acts) {
    int32_t dot = 0;
    for (int l = 0; l < 16; ++l) dot += q3k_value(blk, s, l) * (int32_t)acts[l];
    return dot;
}

static int lowbit_dequantize(int dtype, const uint8_t* blocks, size_t n_blocks, float* out) {
    for (size_t b = 0; b < n_blocks; ++b) {
        float* y = out + b * 256;
        if (dtype == LKO_Q2_K) {                                    /* q2_k.rs:51-64 */
            const uint8_t* blk = blocks + b * 84;
            const float d = lko_f16_to_f32(rd_u16(blk + 80)), dmin = lko_f16_to_f32(rd_u16(blk + 82));
            for (int s = 0; s < 16; ++s) {
                const float scale = d * (float)(blk[s] & 0x0F), offset = dmin * (float)(blk[s] >> 4);
                for (int l = 0; l < 16; ++l) y[16 * s + l] = scale * (float)q23k_low(blk + 16, s, l) - offset;
            }
        } else {                                                    /* q3_k.rs:127-146 */
            const uint8_t* blk = blocks + b * 110;
            const float d = lko_f16_to_f32(rd_u16(blk + 108));
            int8_t sc[16];
            q3k_scales(blk + 96, sc);
            for (int s = 0; s < 16; ++s) {
                const float scale = d * (float)sc[s];
                for (int l = 0; l < 16; ++l) y[16 * s + l] = scale * (float)q3k_value(blk, s, l);
            }
        }
    }
    return 0;
}

/* Served CPU path against Q8_K (q2_k.rs:88-109, 124-126; q3_k.rs:161-167 with its combine
 * y.d * (x.d * sum)): integer sums per block, shares added in block order from -0. */
static float oa_dot_q2k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = -0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * 84;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        const int8_t* yq = (const int8_t*)(yb + 4);
        int32_t scaled = 0, offset = 0;
        for (int s = 0; s < 16; ++s) {
            scaled += (int32_t)(x[s] & 0x0F) * q2k_sub_dot(x, s, yq + 16 * s);
            offset += (int32_t)(x[s] >> 4) * (int32_t)(int16_t)rd_u16(yb + 260 + 2 * s);
        }
        total += rd_f32(yb) * (lko_f16_to_f32(rd_u16(x + 80)) * (float)scaled - lko_f16_to_f32(rd_u16(x + 82)) * (float)offset);
    }
    return total;
}
static float oa_dot_q3k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = -0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * 110;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        const int8_t* yq = (const int8_t*)(yb + 4);
        int8_t sc[16];
        q3k_scales(x + 96, sc);
        int32_t sum = 0;
        for (int s = 0; s < 16; ++s) sum += (int32_t)sc[s] * q3k_sub_dot(x, s, yq + 16 * s);
        total += rd_f32(yb) * (lko_f16_to_f32(rd_u16(x + 108)) * (float)sum);
    }
    return total;
}
/* Same codes on the Q8_1 side (cuda/moe/gguf.cuh:524-546 for Q2_K: d * sum d8 * (dot * scale) -
 * dmin * sum d8 * (sum of codes * minimum); Q3_K likewise without a minimum, vec_dot_plane_q3_K). */
static float ob_dot_q2k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * 84;
        float scaled = 0.0f, offset = 0.0f;
        for (int s = 0; s < 16; ++s) {
            const uint8_t* yb = y + (b * 8 + s / 2) * LKO_Q81_BYTES;
            const int8_t* yq = (const int8_t*)(yb + 4) + 16 * (s % 2);
            const float d8 = lko_f16_to_f32(rd_u16(yb));
            int32_t sum = 0;
            for (int l = 0; l < 16; ++l) sum += yq[l];
            scaled += d8 * (float)(q2k_sub_dot(x, s, yq) * (int32_t)(x[s] & 0x0F));
            offset += d8 * (float)(sum * (int32_t)(x[s] >> 4));
        }
        total += lko_f16_to_f32(rd_u16(x + 80)) * scaled - lko_f16_to_f32(rd_u16(x + 82)) * offset;
    }
    return total;
}
static float ob_dot_q3k(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * 110;
        int8_t sc[16];
        q3k_scales(x + 96, sc);
        float scaled = 0.0f;
        for (int s = 0; s < 16; ++s) {
            const uint8_t* yb = y + (b * 8 + s / 2) * LKO_Q81_BYTES;
            const int8_t* yq = (const int8_t*)(yb + 4) + 16 * (s % 2);
            scaled += lko_f16_to_f32(rd_u16(yb)) * (float)(q3k_sub_dot(x, s, yq) * (int32_t)sc[s]);
        }
        total += lko_f16_to_f32(rd_u16(x + 108)) * scaled;
    }
    return total;
}


/* IQ4_XS {d, scales_h u16, scales_l[4], qs[128]} = 136 bytes (iq4_xs.rs:5-10): eight runs of 32
 * values, run ib = bytes 16 ib .. + 16 of qs (byte j: value j low, value j + 16 high) as IQ4_NL
 * levels, times d * (six-bit scale - 32), the scale's low four bits in scales_l, top two in
 * scales_h (iq4_xs.rs:24-37). Its CPU dot pairs it with per-32 activation runs quantized as Q8_1
 * quantizes (q8_k32.rs:44-57) and adds run_scale * dot * y.d per run (iq4_xs.rs:50-62). */
static inline int iq4xs_scale(const uint8_t* blk, int ib) {
    const int low = (blk[4 + ib / 2] >> (4 * (ib % 2))) & 0x0F;
    const int high = (rd_u16(blk + 2) >> (2 * ib)) & 3;
    return (low | (high << 4)) - 32;
}
static inline int32_t iq4xs_sub_dot(const uint8_t* blk, int ib, const int8_t* acts) {
    const uint8_t* q = blk + 8 + 16 * ib;
    int32_t dot = 0;
    for (int j = 0; j < 16; ++j)
        dot += (int32_t)LEVELS_IQ4NL[q[j] & 0x0F] * acts[j] + (int32_t)LEVELS_IQ4NL[q[j] >> 4] * acts[j + 16];
    return dot;
}
static int iq4xs_dequantize(const uint8_t* blocks, size_t n_blocks, float* out) {
    for (size_t b = 0; b < n_blocks; ++b) {
        const uint8_t* blk = blocks + b * 136;
        const float d = lko_f16_to_f32(rd_u16(blk));
        for (int ib = 0; ib < 8; ++ib) {
            const float dl = d * (float)iq4xs_scale(blk, ib);
            const uint8_t* q = blk + 8 + 16 * ib;
            for (int j = 0; j < 16; ++j) {
                out[b * 256 + 32 * ib + j] = dl * (float)LEVELS_IQ4NL[q[j] & 0x0F];
                out[b * 256 + 32 * ib + j + 16] = dl * (float)LEVELS_IQ4NL[q[j] >> 4];
            }
        }
    }
    return 0;
}
/* Both families read Q8_1-quantized runs (the served path's run quantizer is Q8_1's). */
static float dot_iq4xs(const uint8_t* w, const uint8_t* y, size_t nb) {
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * 136;
        const float d = lko_f16_to_f32(rd_u16(x));
        float block = 0.0f;
        for (int ib = 0; ib < 8; ++ib) {
            const uint8_t* yb = y + (b * 8 + ib) * LKO_Q81_BYTES;
            const int32_t dot = iq4xs_sub_dot(x, ib, (const int8_t*)(yb + 4));
            block += d * (float)iq4xs_scale(x, ib) * (float)dot * lko_f16_to_f32(rd_u16(yb));
        }
        total += block;
    }
    return total;
}

typedef float (*row_dot_fn)(const uint8_t* w, const uint8_t* y, size_t nb);

/* the codebook formats (codebook_formats.c): one statement serves both families, the activation
 * codes being the same on either side */
static float dot_iq2xxs(const uint8_t* w, const uint8_t* y, size_t nb) { return lko_cb_dot(LKO_IQ2_XXS, w, y, nb); }
static float dot_iq3xxs(const uint8_t* w, const uint8_t* y, size_t nb) { return lko_cb_dot(LKO_IQ3_XXS, w, y, nb); }
static float dot_iq3s(const uint8_t* w, const uint8_t* y, size_t nb) { return lko_cb_dot(LKO_IQ3_S, w, y, nb); }
static float dot_iq2s(const uint8_t* w, const uint8_t* y, size_t nb) { return lko_cb_dot(LKO_IQ2_S, w, y, nb); }
static float dot_q20(const uint8_t* w, const uint8_t* y, size_t nb) { return lko_cb_dot(LKO_Q2_0, w, y, nb); }
static row_dot_fn cb_dot_of(int dtype) {
    switch (dtype) {
        case LKO_IQ2_XXS: return dot_iq2xxs;
        case LKO_IQ3_XXS: return dot_iq3xxs;
        case LKO_IQ3_S: return dot_iq3s;
        case LKO_IQ2_S: return dot_iq2s;
        case LKO_Q2_0: return dot_q20;
        default: return NULL;
    }
}

static row_dot_fn oa_dot_of(int dtype) {
    switch (dtype) {
        case LKO_Q2_K: return oa_dot_q2k;
        case LKO_IQ4_XS: return dot_iq4xs;
        case LKO_Q3_K: return oa_dot_q3k;
        case LKO_Q4_K: return oa_dot_q4k;
        case LKO_Q5_K: return oa_dot_q5k;
        case LKO_Q6_K: return oa_dot_q6k;
        case LKO_Q8_0: return oa_dot_q80;
        case LKO_Q4_0: return oa_dot_q40;
        case LKO_Q4_1: return oa_dot_q41;
        case LKO_Q5_0: return oa_dot_q50;
        case LKO_Q5_1: return oa_dot_q51;
        case LKO_IQ4_NL: return oa_dot_iq4nl;
        case LKO_MXFP4: return oa_dot_mxfp4;
        default: return cb_dot_of(dtype);
    }
}
static row_dot_fn ob_dot_of(int dtype) {
    switch (dtype) {
        case LKO_Q2_K: return ob_dot_q2k;
        case LKO_IQ4_XS: return dot_iq4xs;
        case LKO_Q3_K: return ob_dot_q3k;
        case LKO_Q4_K: return ob_dot_q4k;
        case LKO_Q5_K: return ob_dot_q5k;
        case LKO_Q6_K: return ob_dot_q6k;
        case LKO_Q8_0: return ob_dot_q80;
        case LKO_Q4_0: return ob_dot_q40;
        case LKO_Q4_1: return ob_dot_q41;
        case LKO_Q5_0: return ob_dot_q50;
        case LKO_Q5_1: return ob_dot_q51;
        case LKO_IQ4_NL: return ob_dot_iq4nl;
        case LKO_MXFP4: return ob_dot_mxfp4;
        default: return cb_dot_of(dtype);
    }
}

/* O-A activation: Q8_K for K-quants, Q8_0 for Q8_0 (BlockFormat::ActivationBlock). */
static size_t oa_act_row_bytes(int dtype, size_t k) {
    if (dtype == LKO_Q8_0 || dtype == LKO_Q4_0 || dtype == LKO_Q5_0 || dtype == LKO_IQ4_NL || dtype == LKO_MXFP4)
        return (k / 32) * LKO_Q80_BYTES;
    if (dtype == LKO_Q4_1 || dtype == LKO_Q5_1 || dtype == LKO_IQ4_XS || lko_cb_is(dtype)) return (k / 32) * LKO_Q81_BYTES;   /* q4_1.rs: BlockQ8_1 */
    return (k / 256) * LKO_Q8K_BYTES;
}
static void oa_quantize_act(int dtype, const float* x, size_t k, uint8_t* out) {
    if (dtype == LKO_Q8_0 || dtype == LKO_Q4_0 || dtype == LKO_Q5_0 || dtype == LKO_IQ4_NL || dtype == LKO_MXFP4)
        lko_quantize_q8_0(x, k, out);
    else if (dtype == LKO_Q4_1 || dtype == LKO_Q5_1 || dtype == LKO_IQ4_XS || lko_cb_is(dtype)) lko_quantize_q8_1(x, k, out);
    else lko_quantize_q8_k(x, k, out);
}

/* tests_repack.rs:704-885 `matmul::<T>`: quantize each lhs row once, then one independent
 * dot per (row, column). Threading in the reference never changes bits, so none is used here. */
int oa_matmul(int dtype, size_t m, size_t k, size_t n, const float* lhs,
              const uint8_t* rhs, size_t rhs_bytes, float* dst) {
    const row_dot_fn dot = oa_dot_of(dtype);
    if (!dot) return -3;
    const size_t blk = (size_t)lko_block_len(dtype);
    if (k % blk != 0) return -1;
    const size_t nb = k / blk;
    if (rhs_bytes != n * nb * (size_t)lko_block_bytes(dtype)) return -2;
    const size_t arow = oa_act_row_bytes(dtype, k);
    uint8_t* act = (uint8_t*)malloc(arow * (m ? m : 1));
    for (size_t r = 0; r < m; ++r) oa_quantize_act(dtype, lhs + r * k, k, act + r * arow);
    const size_t wrow = nb * (size_t)lko_block_bytes(dtype);
    for (size_t r = 0; r < m; ++r)
        for (size_t c = 0; c < n; ++c) dst[r * n + c] = dot(rhs + c * wrow, act + r * arow, nb);
    free(act);
    return 0;
}

/* drivers.rs:2144-2316 `matmul_bytes_multi` (and its `_serial` twin, 2182-2240): expert e's ONE
 * activation row lhs[e] [k] against its own weight rhs[e] [n, k/blk] into outs[e] [n]. The reference
 * shards (expert x column chunk) over its pool; each output is the same `dot` as `matmul_bytes` gives
 * that row alone, so the schedule is not restated. */
int oa_matmul_multi(int dtype, size_t k, size_t n, size_t ne, const uint8_t* const* rhs, const size_t* rhs_bytes,
                    const float* const* lhs, const size_t* lhs_len, float* const* outs, const size_t* outs_len) {
    if (ne == 0) return 0;
    const row_dot_fn dot = oa_dot_of(dtype);
    if (!dot) return -3;
    const size_t blk = (size_t)lko_block_len(dtype);
    if (k == 0 || k % blk != 0) return -1;
    const size_t nb = k / blk, wrow = nb * (size_t)lko_block_bytes(dtype);
    for (size_t e = 0; e < ne; ++e) {
        if (lhs_len[e] != k) return -4;
        if (outs_len[e] != n) return -5;
        if (rhs_bytes[e] != n * wrow) return -2;
    }
    uint8_t* act = (uint8_t*)malloc(oa_act_row_bytes(dtype, k));
    for (size_t e = 0; e < ne; ++e) {
        oa_quantize_act(dtype, lhs[e], k, act);
        for (size_t c = 0; c < n; ++c) outs[e][c] = dot(rhs[e] + c * wrow, act, nb);
    }
    free(act);
    return 0;
}

/* drivers.rs:2318-2425 `matmul_bytes_grouped`: expert e's weight against its lhs_len[e] / k rows into
 * outs[e] [rows, n]; every row quantized once, every output the same `dot` as one GEMV per
 * (expert, row). */
int oa_matmul_grouped(int dtype, size_t k, size_t n, size_t ne, const uint8_t* const* rhs, const size_t* rhs_bytes,
                      const float* const* lhs, const size_t* lhs_len, float* const* outs, const size_t* outs_len) {
    if (ne == 0) return 0;
    const row_dot_fn dot = oa_dot_of(dtype);
    if (!dot) return -3;
    const size_t blk = (size_t)lko_block_len(dtype);
    if (k == 0 || k % blk != 0) return -1;
    const size_t nb = k / blk, wrow = nb * (size_t)lko_block_bytes(dtype), arow = oa_act_row_bytes(dtype, k);
    for (size_t e = 0; e < ne; ++e) {
        if (lhs_len[e] % k != 0) return -4;
        if (outs_len[e] != lhs_len[e] / k * n) return -5;
        if (rhs_bytes[e] != n * wrow) return -2;
    }
    for (size_t e = 0; e < ne; ++e) {
        const size_t rows = lhs_len[e] / k;
        uint8_t* act = (uint8_t*)malloc(arow * (rows ? rows : 1));
        for (size_t r = 0; r < rows; ++r) oa_quantize_act(dtype, lhs[e] + r * k, k, act + r * arow);
        for (size_t c = 0; c < n; ++c)   /* a weight column meets every row of its expert before the next is read */
            for (size_t r = 0; r < rows; ++r) outs[e][r * n + c] = dot(rhs[e] + c * wrow, act + r * arow, nb);
        free(act);
    }
    return 0;
}

int oa_matmul_exact(int dtype, size_t m, size_t k, size_t n, const float* lhs,
                    const uint8_t* rhs, float* dst) {
    row_dot_fn dot;
    if (dtype == LKO_Q4_K) dot = oa_dot_exact_q4k;
    else if (dtype == LKO_Q6_K) dot = oa_dot_exact_q6k;
    else return -3;
    if (k % 256 != 0) return -1;
    const size_t nb = k / 256;
    const size_t arow = nb * LKO_Q8K_BYTES;
    uint8_t* act = (uint8_t*)malloc(arow * (m ? m : 1));
    for (size_t r = 0; r < m; ++r) lko_quantize_q8_k(lhs + r * k, k, act + r * arow);
    const size_t wrow = nb * (size_t)lko_block_bytes(dtype);
    for (size_t r = 0; r < m; ++r)
        for (size_t c = 0; c < n; ++c) dst[r * n + c] = dot(rhs + c * wrow, act + r * arow, nb);
    free(act);
    return 0;
}

int ob_subdots(int dtype, size_t k, size_t n, const uint8_t* rhs, const uint8_t* act,
               int32_t* dots, int32_t* sums) {
    const size_t blk = (size_t)lko_block_len(dtype);
    legacy_layout ll;
    const int legacy = legacy_layout_of(dtype, &ll);
    if (blk == 0 || (!legacy && !lko_cb_is(dtype) && dtype != LKO_IQ4_XS && dtype != LKO_Q2_K && dtype != LKO_Q3_K && dtype != LKO_Q4_K && dtype != LKO_Q5_K && dtype != LKO_Q6_K && dtype != LKO_Q8_0)) return -3;
    if (k % blk != 0) return -1;
    const size_t nb = k / blk;
    const size_t wrow = nb * (size_t)lko_block_bytes(dtype);
    if (sums) {
        for (size_t j = 0; j < k / 32; ++j) {
            const int8_t* yq = (const int8_t*)(act + j * LKO_Q81_BYTES + 4);
            int32_t s = 0;
            for (int l = 0; l < 32; ++l) s += yq[l];
            sums[j] = s;
        }
    }
    for (size_t c = 0; c < n; ++c) {
        const uint8_t* w = rhs + c * wrow;
        if (dtype == LKO_Q4_K) {
            for (size_t b = 0; b < nb; ++b)
                for (int s = 0; s < 8; ++s)
                    dots[c * (k / 32) + b * 8 + s] = q4k_sub_dot(
                        w + b * LKO_Q4K_BYTES, s, (const int8_t*)(act + (b * 8 + s) * LKO_Q81_BYTES + 4));
        } else if (dtype == LKO_IQ4_XS) {
            for (size_t b = 0; b < nb; ++b)
                for (int s = 0; s < 8; ++s)
                    dots[c * (k / 32) + b * 8 + s] = iq4xs_sub_dot(
                        w + b * 136, s, (const int8_t*)(act + (b * 8 + s) * LKO_Q81_BYTES + 4));
        } else if (lko_cb_is(dtype)) {   /* two integers per run of 32: its halves */
            const size_t runs = blk / 32;
            for (size_t b = 0; b < nb; ++b)
                for (size_t r = 0; r < runs; ++r)
                    lko_cb_half_dots(dtype, w + b * (size_t)lko_block_bytes(dtype), (int)r,
                                     (const int8_t*)(act + (b * runs + r) * LKO_Q81_BYTES + 4), dots + c * (k / 16) + 2 * (b * runs + r));
        } else if (dtype == LKO_Q2_K || dtype == LKO_Q3_K) {
            for (size_t b = 0; b < nb; ++b)
                for (int s = 0; s < 16; ++s) {
                    const int8_t* a = (const int8_t*)(act + (b * 8 + s / 2) * LKO_Q81_BYTES + 4) + 16 * (s % 2);
                    dots[c * (k / 16) + b * 16 + s] = dtype == LKO_Q2_K ? q2k_sub_dot(w + b * 84, s, a)
                                                                        : q3k_sub_dot(w + b * 110, s, a);
                }
        } else if (dtype == LKO_Q5_K) {
            for (size_t b = 0; b < nb; ++b)
                for (int s = 0; s < 8; ++s)
                    dots[c * (k / 32) + b * 8 + s] = q5k_sub_dot(
                        w + b * LKO_Q5K_BYTES, s, (const int8_t*)(act + (b * 8 + s) * LKO_Q81_BYTES + 4));
        } else if (dtype == LKO_Q6_K) {
            for (size_t b = 0; b < nb; ++b) {
                int8_t acts[256];
                for (int s = 0; s < 8; ++s) memcpy(acts + 32 * s, act + (b * 8 + s) * LKO_Q81_BYTES + 4, 32);
                q6k_sub_dots(w + b * LKO_Q6K_BYTES, acts, dots + c * (k / 16) + b * 16);
            }
        } else if (legacy) {
            for (size_t b = 0; b < nb; ++b)
                dots[c * nb + b] = legacy_sub_dot(w + b * (size_t)ll.bytes, &ll,
                                                  (const int8_t*)(act + b * LKO_Q81_BYTES + 4));
        } else {
            for (size_t b = 0; b < nb; ++b)
                dots[c * nb + b] = i8_dot32((const int8_t*)(w + b * LKO_Q80_BYTES + 2),
                                            (const int8_t*)(act + b * LKO_Q81_BYTES + 4));
        }
    }
    return 0;
}

int ob_matmul_q8_1(int dtype, size_t m, size_t k, size_t n, const uint8_t* act,
                   size_t act_stride_blocks, const uint8_t* rhs, float* dst) {
    const row_dot_fn dot = ob_dot_of(dtype);
    if (!dot) return -3;
    const size_t blk = (size_t)lko_block_len(dtype);
    if (k % blk != 0) return -1;
    const size_t nb = k / blk;
    const size_t wrow = nb * (size_t)lko_block_bytes(dtype);
    for (size_t r = 0; r < m; ++r)
        for (size_t c = 0; c < n; ++c)
            dst[r * n + c] = dot(rhs + c * wrow, act + r * act_stride_blocks * LKO_Q81_BYTES, nb);
    return 0;
}

int ob_matmul(int dtype, size_t m, size_t k, size_t n, const float* lhs,
              const uint8_t* rhs, float* dst) {
    if (k % 32 != 0) return -1;
    const size_t arow = (k / 32) * LKO_Q81_BYTES;
    uint8_t* act = (uint8_t*)malloc(arow * (m ? m : 1));
    for (size_t r = 0; r < m; ++r) lko_quantize_q8_1(lhs + r * k, k, act + r * arow);
    const int rc = ob_matmul_q8_1(dtype, m, k, n, act, k / 32, rhs, dst);
    free(act);
    return rc;
}

/* The real-number value of every weight of a row, in f64 from the block fields (no f32
 * rounding of scale*q - offset). */
static int dequant_row_f64(int dtype, const uint8_t* w, size_t nb, double* out) {
    if (dtype == LKO_Q4_K) {
        for (size_t b = 0; b < nb; ++b) {
            const uint8_t* x = w + b * LKO_Q4K_BYTES;
            const double d = lko_f16_to_f32(rd_u16(x)), dmin = lko_f16_to_f32(rd_u16(x + 2));
            uint8_t sc[8], mn[8];
            lko_unpack_scales_mins(x + 4, sc, mn);
            for (int s = 0; s < 8; ++s) {
                const uint8_t* group = x + 16 + (s / 2) * 32;
                const int shift = (s % 2 == 0) ? 0 : 4;
                for (int l = 0; l < 32; ++l)
                    out[b * 256 + s * 32 + l] = d * sc[s] * (double)((group[l] >> shift) & 0x0F) - dmin * mn[s];
            }
        }
        return 0;
    }
    if (dtype == LKO_Q5_K) {
        for (size_t b = 0; b < nb; ++b) {
            const uint8_t* x = w + b * LKO_Q5K_BYTES;
            const double d = lko_f16_to_f32(rd_u16(x)), dmin = lko_f16_to_f32(rd_u16(x + 2));
            uint8_t sc[8], mn[8];
            lko_unpack_scales_mins(x + 4, sc, mn);
            for (int s = 0; s < 8; ++s)
                for (int l = 0; l < 32; ++l)
                    out[b * 256 + s * 32 + l] = d * sc[s] * (double)q5k_code(x, s, l) - dmin * mn[s];
        }
        return 0;
    }
    if (dtype == LKO_Q6_K) {
        for (size_t b = 0; b < nb; ++b) {
            const uint8_t* x = w + b * LKO_Q6K_BYTES;
            const double d = lko_f16_to_f32(rd_u16(x + 208));
            const int8_t* scales = (const int8_t*)(x + 192);
            for (int h = 0; h < 2; ++h)
                for (int g = 0; g < 4; ++g)
                    for (int l = 0; l < 32; ++l)
                        out[b * 256 + 128 * h + 32 * g + l] =
                            d * (double)scales[8 * h + 2 * g + l / 16] * (double)q6k_code(x, h, g, l);
        }
        return 0;
    }
    if (dtype == LKO_Q8_0) {
        for (size_t b = 0; b < nb; ++b) {
            const uint8_t* x = w + b * LKO_Q80_BYTES;
            const double d = lko_f16_to_f32(rd_u16(x));
            for (int l = 0; l < 32; ++l) out[b * 32 + l] = d * (double)(int8_t)x[2 + l];
        }
        return 0;
    }
    if (lko_cb_is(dtype)) return lko_cb_dequantize_f64(dtype, w, nb, out);
    if (dtype == LKO_IQ4_XS) {
        for (size_t b = 0; b < nb; ++b) {
            const uint8_t* x = w + b * 136;
            const double d = lko_f16_to_f32(rd_u16(x));
            for (int ib = 0; ib < 8; ++ib)
                for (int j = 0; j < 16; ++j) {
                    const uint8_t q = x[8 + 16 * ib + j];
                    out[b * 256 + 32 * ib + j] = d * iq4xs_scale(x, ib) * LEVELS_IQ4NL[q & 0x0F];
                    out[b * 256 + 32 * ib + j + 16] = d * iq4xs_scale(x, ib) * LEVELS_IQ4NL[q >> 4];
                }
        }
        return 0;
    }
    if (dtype == LKO_Q2_K || dtype == LKO_Q3_K) {
        for (size_t b = 0; b < nb; ++b) {
            const uint8_t* x = w + b * (size_t)(dtype == LKO_Q2_K ? 84 : 110);
            int8_t sc3[16];
            if (dtype == LKO_Q3_K) q3k_scales(x + 96, sc3);
            for (int s = 0; s < 16; ++s)
                for (int l = 0; l < 16; ++l) {
                    if (dtype == LKO_Q2_K)
                        out[b * 256 + 16 * s + l] = (double)lko_f16_to_f32(rd_u16(x + 80)) * (x[s] & 0x0F) * q23k_low(x + 16, s, l) -
                                                    (double)lko_f16_to_f32(rd_u16(x + 82)) * (x[s] >> 4);
                    else
                        out[b * 256 + 16 * s + l] = (double)lko_f16_to_f32(rd_u16(x + 108)) * sc3[s] * q3k_value(x, s, l);
                }
        }
        return 0;
    }
    legacy_layout ll;
    if (legacy_layout_of(dtype, &ll)) {
        for (size_t b = 0; b < nb; ++b) {
            const uint8_t* x = w + b * (size_t)ll.bytes;
            const double d = legacy_scale(x, dtype);
            const double m = ll.m_at >= 0 ? lko_f16_to_f32(rd_u16(x + ll.m_at)) : 0.0;
            for (int v = 0; v < 32; ++v) out[b * 32 + v] = d * (double)(legacy_code(x, &ll, v) - ll.bias) + m;
        }
        return 0;
    }
    return -3;
}

int ob_matmul_f64(int dtype, size_t m, size_t k, size_t n, const float* lhs,
                  const uint8_t* rhs, double* dst) {
    const size_t blk = (size_t)lko_block_len(dtype);
    if (blk == 0) return -3;
    if (k % blk != 0 || k % 32 != 0) return -1;
    const size_t nb = k / blk;
    const size_t wrow = nb * (size_t)lko_block_bytes(dtype);
    const size_t arow = (k / 32) * LKO_Q81_BYTES;
    uint8_t* act = (uint8_t*)malloc(arow);
    float* xa = (float*)malloc(sizeof(float) * k * (m ? m : 1));
    double* wd = (double*)malloc(sizeof(double) * k);
    int rc = 0;
    for (size_t r = 0; r < m; ++r) {
        lko_quantize_q8_1(lhs + r * k, k, act);
        lko_dequantize(LKO_Q8_1, act, k / 32, xa + r * k); /* q*d is exact in f32 */
    }
    for (size_t c = 0; c < n && rc == 0; ++c) {
        rc = dequant_row_f64(dtype, rhs + c * wrow, nb, wd);
        if (rc != 0) break;
        for (size_t r = 0; r < m; ++r) {
            double acc = 0.0;
            for (size_t i = 0; i < k; ++i) acc += wd[i] * (double)xa[r * k + i];
            dst[r * n + c] = acc;
        }
    }
    free(act); free(xa); free(wd);
    return rc;
}

/* ------------------------------------------------------------------------------------------
 * Router and MoE.
 * ---------------------------------------------------------------------------------------- */

void lko_topk_softmax(const float* logits, size_t tokens, size_t n_experts, size_t topk,
                      int renorm, int32_t* ids, float* weights) {
    float* p = (float*)malloc(sizeof(float) * n_experts);
    uint8_t* taken = (uint8_t*)malloc(n_experts);
    for (size_t t = 0; t < tokens; ++t) {
        const float* row = logits + t * n_experts;
        float mx = row[0];
        for (size_t e = 1; e < n_experts; ++e) mx = fmaxf(mx, row[e]);
        float sum = 0.0f;
        for (size_t e = 0; e < n_experts; ++e) { p[e] = expf(row[e] - mx); sum += p[e]; }
        for (size_t e = 0; e < n_experts; ++e) p[e] /= sum;
        memset(taken, 0, n_experts);
        float wsum = 0.0f;
        for (size_t j = 0; j < topk; ++j) {
            size_t best = n_experts;
            for (size_t e = 0; e < n_experts; ++e)
                if (!taken[e] && (best == n_experts || p[e] > p[best])) best = e;
            taken[best] = 1;
            ids[t * topk + j] = (int32_t)best;
            weights[t * topk + j] = p[best];
            wsum += p[best];
        }
        if (renorm)
            for (size_t j = 0; j < topk; ++j) weights[t * topk + j] /= wsum;
    }
    free(p); free(taken);
}

void lko_group_by_expert(const int32_t* ids, size_t pairs, int32_t* sorted_slots,
                         int32_t* sorted_experts) {
    int32_t max_e = 0;
    for (size_t i = 0; i < pairs; ++i) if (ids[i] > max_e) max_e = ids[i];
    size_t at = 0;
    for (int32_t e = 0; e <= max_e; ++e)
        for (size_t i = 0; i < pairs; ++i)
            if (ids[i] == e) { sorted_slots[at] = (int32_t)i; sorted_experts[at] = e; ++at; }
}

int lko_moe_forward(int family, int dt_gu, int dt_down, size_t tokens, size_t hidden, size_t ffn,
                    size_t n_experts, size_t topk, const float* x, const uint8_t* gate,
                    const uint8_t* up, const uint8_t* down, const int32_t* ids,
                    const float* weights, float* h_sorted, float* out) {
    const row_dot_fn dot_gu = family ? ob_dot_of(dt_gu) : oa_dot_of(dt_gu);
    const row_dot_fn dot_dn = family ? ob_dot_of(dt_down) : oa_dot_of(dt_down);
    if (!dot_gu || !dot_dn) return -3;
    if (hidden % (size_t)lko_block_len(dt_gu) != 0 || ffn % (size_t)lko_block_len(dt_down) != 0) return -1;
    (void)n_experts;
    const size_t pairs = tokens * topk;
    const size_t nb_gu = hidden / (size_t)lko_block_len(dt_gu);
    const size_t nb_dn = ffn / (size_t)lko_block_len(dt_down);
    const size_t wrow_gu = nb_gu * (size_t)lko_block_bytes(dt_gu);
    const size_t wrow_dn = nb_dn * (size_t)lko_block_bytes(dt_down);
    const size_t arow_x = family ? (hidden / 32) * LKO_Q81_BYTES : oa_act_row_bytes(dt_gu, hidden);
    const size_t arow_h = family ? (ffn / 32) * LKO_Q81_BYTES : oa_act_row_bytes(dt_down, ffn);

    int32_t* slots = (int32_t*)malloc(sizeof(int32_t) * (pairs ? pairs : 1));
    int32_t* experts = (int32_t*)malloc(sizeof(int32_t) * (pairs ? pairs : 1));
    lko_group_by_expert(ids, pairs, slots, experts);

    uint8_t* xq = (uint8_t*)malloc(arow_x * (tokens ? tokens : 1));
    for (size_t t = 0; t < tokens; ++t) {
        if (family) lko_quantize_q8_1(x + t * hidden, hidden, xq + t * arow_x);
        else oa_quantize_act(dt_gu, x + t * hidden, hidden, xq + t * arow_x);
    }
    float* h = (float*)malloc(sizeof(float) * (pairs ? pairs : 1) * ffn);
    for (size_t j = 0; j < pairs; ++j) {
        const size_t e = (size_t)experts[j];
        const uint8_t* act = xq + ((size_t)slots[j] / topk) * arow_x;
        for (size_t r = 0; r < ffn; ++r) {
            const float g = dot_gu(gate + (e * ffn + r) * wrow_gu, act, nb_gu);
            const float u = dot_gu(up + (e * ffn + r) * wrow_gu, act, nb_gu);
            h[j * ffn + r] = u * (g / (1.0f + expf(-g)));
        }
    }
    if (h_sorted) memcpy(h_sorted, h, sizeof(float) * pairs * ffn);
    uint8_t* hq = (uint8_t*)malloc(arow_h * (pairs ? pairs : 1));
    for (size_t j = 0; j < pairs; ++j) {
        if (family) lko_quantize_q8_1(h + j * ffn, ffn, hq + j * arow_h);
        else oa_quantize_act(dt_down, h + j * ffn, ffn, hq + j * arow_h);
    }
    for (size_t i = 0; i < tokens * hidden; ++i) out[i] = 0.0f;
    for (size_t j = 0; j < pairs; ++j) {
        const size_t e = (size_t)experts[j];
        const size_t t = (size_t)slots[j] / topk;
        const float tw = weights[slots[j]];
        for (size_t r = 0; r < hidden; ++r)
            out[t * hidden + r] += tw * dot_dn(down + (e * hidden + r) * wrow_dn, hq + j * arow_h, nb_dn);
    }
    free(slots); free(experts); free(xq); free(h); free(hq);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Decode-step producers (RMSNorm family, split activation): src/inference/cuda/mmvq_gguf.cu.
 * ---------------------------------------------------------------------------------------- */

float lko_inv_rms_wide(const float* row, size_t cols, float eps) {
    float tree[256];
    for (size_t t = 0; t < 256; ++t) {          /* :811-817, the build contracts sum += v * v */
        float part = 0.0f;
        for (size_t i = t; i < cols; i += 256) part = fmaf(row[i], row[i], part);
        tree[t] = part;
    }
    for (size_t s = 128; s > 0; s >>= 1)        /* :820-823 */
        for (size_t t = 0; t < s; ++t) tree[t] += tree[t + s];
    return 1.0f / sqrtf(tree[0] / (float)cols + eps);
}

void lko_norm_rows(int mode, const float* x, const float* w_first, const float* residual, const float* w,
                   float* mid, float* out, float eps_first, float eps, size_t cols, size_t rows) {
    float* srow = (float*)malloc(sizeof(float) * cols);
    for (size_t r = 0; r < rows; ++r) {
        const size_t off = r * cols;
        for (size_t i = 0; i < cols; ++i) {
            float v = x[off + i];
            if (mode == 1) { v = v + residual[off + i]; mid[off + i] = v; }
            srow[i] = v;
        }
        if (mode == 2) {
            const float rms_first = lko_inv_rms_wide(srow, cols, eps_first);
            for (size_t i = 0; i < cols; ++i) {
                const float y = (srow[i] * rms_first) * w_first[i];   /* :914-916 */
                const float xr = y + residual[off + i];
                srow[i] = xr;
                mid[off + i] = xr;
            }
        }
        const float rms = lko_inv_rms_wide(srow, cols, eps);
        for (size_t i = 0; i < cols; ++i) out[off + i] = (srow[i] * rms) * w[i];
    }
    free(srow);
}

void lko_split_act_mul(const float* gu, float* out, size_t n, size_t rows, int act) {
    for (size_t r = 0; r < rows; ++r)
        for (size_t i = 0; i < n; ++i) {
            const float g = gu[r * 2 * n + i], u = gu[r * 2 * n + n + i];
            float a;
            if (act == 0) {
                a = g / (1.0f + expf(-g));
            } else {
                const float k0 = 0.7978845608028654f, k1 = 0.044715f;
                a = 0.5f * g * (1.0f + tanhf(k0 * (g + k1 * g * g * g)));
            }
            out[r * n + i] = a * u;
        }
}

void lko_topk_sigmoid(const float* logits, const float* bias, size_t tokens, size_t n_experts, size_t topk,
                      int renorm, float scale, int32_t* ids, float* weights) {
    float* p = (float*)malloc(sizeof(float) * n_experts);
    float* sel = (float*)malloc(sizeof(float) * n_experts);
    for (size_t t = 0; t < tokens; ++t) {
        const float* row = logits + t * n_experts;
        for (size_t e = 0; e < n_experts; ++e) {
            p[e] = 1.0f / (1.0f + expf(-row[e]));
            sel[e] = p[e] + (bias ? bias[e] : 0.0f);
        }
        float sum = 0.0f;
        for (size_t j = 0; j < topk; ++j) {
            size_t best = 0;
            for (size_t e = 1; e < n_experts; ++e)
                if (sel[e] > sel[best]) best = e;          /* strict: the lower index wins a tie */
            ids[t * topk + j] = (int32_t)best;
            weights[t * topk + j] = p[best];
            sum += p[best];
            sel[best] = -INFINITY;
        }
        const float inv = renorm ? 1.0f / fmaxf(sum, 6.103515625e-5f) : 1.0f;
        for (size_t j = 0; j < topk; ++j) weights[t * topk + j] = weights[t * topk + j] * inv * scale;
    }
    free(p); free(sel);
}

/*
 * Timed CPU baseline: the served CPU quantized matmul (O-A semantics) with AVX2 integer
 * kernels and a worker pool. TEST / BENCHMARK INFRASTRUCTURE ONLY, like the scalar oracle
 * beside it: the shipped library never links it.
 *
 * Follows the shape of the reference's vector path: integer sums of a block in vector lanes
 * (src/tensor/quant_cpu/avx/superblock.rs:327-414 for q4_K, :586-698 for q6_K, avx/block32.rs
 * for q8_0), one f32 fold per block, one worker per core grabbing column chunks of
 * clamp(n / (threads * 8), 16, 256) from an atomic counter (tests_repack.rs:707-718,
 * gemv_pool.rs:186-203), several activation rows served per weight column in tiles of at most
 * eight (tests_repack.rs:822-860). The f32 fold is per block from exact integer sums (the
 * `combine` step, q4_k.rs:154-156, q6_k.rs:161-163), so results differ from the scalar dot
 * only by float summation order; tests hold it to the reference's own vector-vs-scalar bound
 * 1e-3 * max(|ref|, 1) (avx/parity.rs:50-56).
 *
 * Falls back to the scalar oracle when the CPU lacks AVX2.
 */
#define _GNU_SOURCE
#include "loken_oracle.h"

#include <immintrin.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>

static inline float f16_to_f32_hw(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t rd16(const uint8_t* p) { uint16_t v; memcpy(&v, p, 2); return v; }

static inline int32_t hsum_i32_8(__m256i v) {
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x4E));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xB1));
    return _mm_cvtsi128_si32(s);
}

/* Q4_K row against Q8_K row. */
static float dot_q4k_q8k_avx2(const uint8_t* w, const uint8_t* y, size_t nb) {
    const __m256i nib = _mm256_set1_epi8(0x0F);
    const __m256i ones = _mm256_set1_epi16(1);
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q4K_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        uint8_t sc[8], mn[8];
        lko_unpack_scales_mins(x + 4, sc, mn);
        float yd;
        memcpy(&yd, yb, 4);
        const int8_t* acts = (const int8_t*)(yb + 4);
        const int16_t* bsums = (const int16_t*)(yb + 260);
        __m256i acc = _mm256_setzero_si256();
        int32_t offset = 0;
        for (int j = 0; j < 4; ++j) {
            const __m256i packed = _mm256_loadu_si256((const __m256i*)(x + 16 + 32 * j));
            const __m256i lo = _mm256_and_si256(packed, nib);
            const __m256i hi = _mm256_and_si256(_mm256_srli_epi16(packed, 4), nib);
            const __m256i a_lo = _mm256_loadu_si256((const __m256i*)(acts + 64 * j));
            const __m256i a_hi = _mm256_loadu_si256((const __m256i*)(acts + 64 * j + 32));
            const __m256i p_lo = _mm256_madd_epi16(_mm256_maddubs_epi16(lo, a_lo), ones);
            const __m256i p_hi = _mm256_madd_epi16(_mm256_maddubs_epi16(hi, a_hi), ones);
            acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(p_lo, _mm256_set1_epi32(sc[2 * j])));
            acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(p_hi, _mm256_set1_epi32(sc[2 * j + 1])));
            offset += (int32_t)mn[2 * j] * ((int32_t)bsums[4 * j] + bsums[4 * j + 1]);
            offset += (int32_t)mn[2 * j + 1] * ((int32_t)bsums[4 * j + 2] + bsums[4 * j + 3]);
        }
        const int32_t scaled = hsum_i32_8(acc);
        total += yd * (f16_to_f32_hw(rd16(x)) * (float)scaled - f16_to_f32_hw(rd16(x + 2)) * (float)offset);
    }
    return total;
}

/* Q6_K row against Q8_K row: codes kept unsigned 0..63, the 32 folded in through bsums. */
static float dot_q6k_q8k_avx2(const uint8_t* w, const uint8_t* y, size_t nb) {
    const __m256i nib = _mm256_set1_epi8(0x0F);
    const __m256i two = _mm256_set1_epi8(0x03);
    float total = 0.0f;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q6K_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        const int8_t* scales = (const int8_t*)(x + 192);
        float yd;
        memcpy(&yd, yb, 4);
        const int8_t* acts = (const int8_t*)(yb + 4);
        const int16_t* bsums = (const int16_t*)(yb + 260);
        int32_t scaled = 0;
        for (int h = 0; h < 2; ++h) {
            const __m256i ql0 = _mm256_loadu_si256((const __m256i*)(x + 64 * h));
            const __m256i ql1 = _mm256_loadu_si256((const __m256i*)(x + 64 * h + 32));
            const __m256i qh = _mm256_loadu_si256((const __m256i*)(x + 128 + 32 * h));
            __m256i code[4];
            code[0] = _mm256_or_si256(_mm256_and_si256(ql0, nib),
                                      _mm256_slli_epi16(_mm256_and_si256(qh, two), 4));
            code[1] = _mm256_or_si256(_mm256_and_si256(ql1, nib),
                                      _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(qh, 2), two), 4));
            code[2] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(ql0, 4), nib),
                                      _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(qh, 4), two), 4));
            code[3] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(ql1, 4), nib),
                                      _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(qh, 6), two), 4));
            for (int g = 0; g < 4; ++g) {
                const __m256i a = _mm256_loadu_si256((const __m256i*)(acts + 128 * h + 32 * g));
                const __m256i p16 = _mm256_maddubs_epi16(code[g], a);
                const __m256i p32 = _mm256_madd_epi16(p16, _mm256_set1_epi16(1));
                /* lanes 0-3: values 0..15, lanes 4-7: values 16..31 */
                __m128i lo = _mm256_castsi256_si128(p32), hi = _mm256_extracti128_si256(p32, 1);
                lo = _mm_add_epi32(lo, _mm_shuffle_epi32(lo, 0x4E));
                lo = _mm_add_epi32(lo, _mm_shuffle_epi32(lo, 0xB1));
                hi = _mm_add_epi32(hi, _mm_shuffle_epi32(hi, 0x4E));
                hi = _mm_add_epi32(hi, _mm_shuffle_epi32(hi, 0xB1));
                const int j = 8 * h + 2 * g;
                scaled += (int32_t)scales[j] * (_mm_cvtsi128_si32(lo) - 32 * (int32_t)bsums[j]);
                scaled += (int32_t)scales[j + 1] * (_mm_cvtsi128_si32(hi) - 32 * (int32_t)bsums[j + 1]);
            }
        }
        total += yd * (f16_to_f32_hw(rd16(x + 208)) * (float)scaled);
    }
    return total;
}

/* Q8_0 row against Q8_0 row. */
static float dot_q80_q80_avx2(const uint8_t* w, const uint8_t* y, size_t nb) {
    __m256 acc = _mm256_setzero_ps();
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q80_BYTES;
        const uint8_t* yb = y + b * LKO_Q80_BYTES;
        const __m256i a = _mm256_loadu_si256((const __m256i*)(x + 2));
        const __m256i c = _mm256_loadu_si256((const __m256i*)(yb + 2));
        const __m256i p16 = _mm256_maddubs_epi16(_mm256_sign_epi8(a, a), _mm256_sign_epi8(c, a));
        const __m256i p32 = _mm256_madd_epi16(p16, _mm256_set1_epi16(1));
        const float d = f16_to_f32_hw(rd16(x)) * f16_to_f32_hw(rd16(yb));
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(p32), acc);
    }
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(acc), _mm256_extractf128_ps(acc, 1));
    s = _mm_add_ps(s, _mm_movehl_ps(s, s));
    s = _mm_add_ss(s, _mm_movehdup_ps(s));
    return _mm_cvtss_f32(s);
}

typedef float (*row_dot_fn)(const uint8_t*, const uint8_t*, size_t);

typedef struct {
    row_dot_fn dot;
    size_t m, n, nb, wrow, arow, chunk_cols, n_chunks;
    const uint8_t* rhs;
    const uint8_t* act;
    float* dst;
    atomic_size_t next;
} job_t;

static void* worker(void* arg) {
    job_t* j = (job_t*)arg;
    for (;;) {
        const size_t c = atomic_fetch_add(&j->next, 1);
        if (c >= j->n_chunks) break;
        const size_t col0 = c * j->chunk_cols;
        const size_t col1 = col0 + j->chunk_cols < j->n ? col0 + j->chunk_cols : j->n;
        for (size_t r0 = 0; r0 < j->m; r0 += 8) {
            const size_t r1 = r0 + 8 < j->m ? r0 + 8 : j->m;
            for (size_t col = col0; col < col1; ++col)
                for (size_t r = r0; r < r1; ++r)
                    j->dst[r * j->n + col] = j->dot(j->rhs + col * j->wrow, j->act + r * j->arow, j->nb);
        }
    }
    return NULL;
}

int lko_cpu_has_avx2(void) {
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") && __builtin_cpu_supports("f16c");
}

/* dst[m,n] = lhs[m,k] x rhs, O-A semantics, `threads` workers (>= 1). Returns 0 on success,
 * the scalar oracle's error codes otherwise. */
int oa_matmul_fast(int dtype, size_t m, size_t k, size_t n, const float* lhs,
                   const uint8_t* rhs, size_t rhs_bytes, float* dst, int threads) {
    if (!lko_cpu_has_avx2()) return oa_matmul(dtype, m, k, n, lhs, rhs, rhs_bytes, dst);
    row_dot_fn dot;
    size_t blk, wblk, ablk, aval;
    switch (dtype) {
        case LKO_Q4_K: dot = dot_q4k_q8k_avx2; blk = 256; wblk = LKO_Q4K_BYTES; ablk = LKO_Q8K_BYTES; aval = 256; break;
        case LKO_Q6_K: dot = dot_q6k_q8k_avx2; blk = 256; wblk = LKO_Q6K_BYTES; ablk = LKO_Q8K_BYTES; aval = 256; break;
        case LKO_Q8_0: dot = dot_q80_q80_avx2; blk = 32; wblk = LKO_Q80_BYTES; ablk = LKO_Q80_BYTES; aval = 32; break;
        default: return -3;
    }
    if (k % blk != 0) return -1;
    if (rhs_bytes != n * (k / blk) * wblk) return -2;
    if (threads < 1) threads = 1;
    job_t job;
    job.dot = dot; job.m = m; job.n = n; job.nb = k / blk; job.wrow = job.nb * wblk;
    job.arow = (k / aval) * ablk; job.rhs = rhs; job.dst = dst;
    uint8_t* act = (uint8_t*)malloc(job.arow * (m ? m : 1));
    for (size_t r = 0; r < m; ++r) {
        if (dtype == LKO_Q8_0) lko_quantize_q8_0(lhs + r * k, k, act + r * job.arow);
        else lko_quantize_q8_k(lhs + r * k, k, act + r * job.arow);
    }
    job.act = act;
    size_t chunk = n / ((size_t)threads * 8);
    if (chunk < 16) chunk = 16;
    if (chunk > 256) chunk = 256;
    if (chunk > n) chunk = n ? n : 1;
    job.chunk_cols = chunk;
    job.n_chunks = (n + chunk - 1) / chunk;
    atomic_init(&job.next, 0);
    pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
    for (int t = 1; t < threads; ++t) pthread_create(&tid[t], NULL, worker, &job);
    worker(&job);
    for (int t = 1; t < threads; ++t) pthread_join(tid[t], NULL);
    free(tid);
    free(act);
    return 0;
}

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
 * Drivers: the per-column dot above for every format (oa_matmul_fast); the path loken actually
 * serves Q4_K decode with (oa_matmul_q4k_x8): rows repacked eight at a time and one group dot per
 * eight output columns; and the prefill forms over the same repacked weights, one pool chunk per
 * column group with the rows in tiles of eight (oa_matmul_q4k_x8_tiled, oa_matmul_q6k_x8_tiled:
 * matmul_q4k_repacked_tiled / matmul_q6k_repacked_tiled, drivers.rs:231-406). All run on ONE
 * persistent pool of workers (no thread is created per call).
 *
 * Falls back to the scalar oracle when the CPU lacks AVX2.
 */
#define _GNU_SOURCE
#include "loken_oracle.h"

#include <immintrin.h>
#include <pthread.h>
#include <sched.h>
#include <stdatomic.h>
#include <stdio.h>
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

/* The same dot for up to four activation rows in one pass over the weight row
 * (vec_dot_q4k_q8k_many, avx/superblock.rs:425-490): a block's scales and nibble vectors are
 * formed once and spent on every row; each row then runs the one-row kernel's own operations in
 * its order, so out[t] carries the bits of dot_q4k_q8k_avx2(w, ys[t]). */
#define LKO_MANY_ROWS 4
static void dot_q4k_q8k_many4_avx2(const uint8_t* w, const uint8_t* const* ys, size_t rows, size_t nb, float* out) {
    const __m256i nib = _mm256_set1_epi8(0x0F);
    const __m256i ones = _mm256_set1_epi16(1);
    float total[LKO_MANY_ROWS] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* x = w + b * LKO_Q4K_BYTES;
        uint8_t sc[8], mn[8];
        lko_unpack_scales_mins(x + 4, sc, mn);
        const float d = f16_to_f32_hw(rd16(x)), dmin = f16_to_f32_hw(rd16(x + 2));
        __m256i code[8], scale[8];
        for (int j = 0; j < 4; ++j) {
            const __m256i packed = _mm256_loadu_si256((const __m256i*)(x + 16 + 32 * j));
            code[2 * j] = _mm256_and_si256(packed, nib);
            code[2 * j + 1] = _mm256_and_si256(_mm256_srli_epi16(packed, 4), nib);
            scale[2 * j] = _mm256_set1_epi32(sc[2 * j]);
            scale[2 * j + 1] = _mm256_set1_epi32(sc[2 * j + 1]);
        }
        for (size_t t = 0; t < rows; ++t) {
            const uint8_t* yb = ys[t] + b * LKO_Q8K_BYTES;
            float yd;
            memcpy(&yd, yb, 4);
            const int8_t* acts = (const int8_t*)(yb + 4);
            const int16_t* bsums = (const int16_t*)(yb + 260);
            __m256i acc = _mm256_setzero_si256();
            int32_t offset = 0;
            for (int j = 0; j < 4; ++j) {
                const __m256i a_lo = _mm256_loadu_si256((const __m256i*)(acts + 64 * j));
                const __m256i a_hi = _mm256_loadu_si256((const __m256i*)(acts + 64 * j + 32));
                const __m256i p_lo = _mm256_madd_epi16(_mm256_maddubs_epi16(code[2 * j], a_lo), ones);
                const __m256i p_hi = _mm256_madd_epi16(_mm256_maddubs_epi16(code[2 * j + 1], a_hi), ones);
                acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(p_lo, scale[2 * j]));
                acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(p_hi, scale[2 * j + 1]));
                offset += (int32_t)mn[2 * j] * ((int32_t)bsums[4 * j] + bsums[4 * j + 1]);
                offset += (int32_t)mn[2 * j + 1] * ((int32_t)bsums[4 * j + 2] + bsums[4 * j + 3]);
            }
            total[t] += yd * (d * (float)hsum_i32_8(acc) - dmin * (float)offset);
        }
    }
    for (size_t t = 0; t < rows; ++t) out[t] = total[t];
}
void lko_dot_q4k_q8k_many(const uint8_t* w, const uint8_t* const* ys, size_t rows, size_t nb, float* out) {
    for (size_t t0 = 0; t0 < rows; t0 += LKO_MANY_ROWS)
        dot_q4k_q8k_many4_avx2(w, ys + t0, rows - t0 < LKO_MANY_ROWS ? rows - t0 : LKO_MANY_ROWS, nb, out + t0);
}

/* The 512-bit twin (avx512/superblock.rs:20-90): a 64-byte load holds two of the block's 32-byte runs,
 * one VNNI byte dot-product covers the low (or high) nibbles of both against their activations, and
 * the integer sums are those of the 256-bit kernel, so the folded result carries its bits. */
__attribute__((target("avx2,fma,f16c,avx512f,avx512bw,avx512vl,avx512dq,avx512vnni")))
static float dot_q4k_q8k_avx512(const uint8_t* w, const uint8_t* y, size_t nb) {
    const __m512i nib = _mm512_set1_epi8(0x0F);
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
        __m512i acc = _mm512_setzero_si512();
        int32_t offset = 0;
        for (int h = 0; h < 2; ++h) {
            /* runs 2h and 2h + 1 of the nibbles; a run's low nibbles meet activations 64 j .. 64 j + 31,
             * its high nibbles 64 j + 32 .. 64 j + 63 */
            const __m512i packed = _mm512_loadu_si512((const void*)(x + 16 + 64 * h));
            const __m512i lo = _mm512_and_si512(packed, nib);
            const __m512i hi = _mm512_and_si512(_mm512_srli_epi16(packed, 4), nib);
            const __m256i a0 = _mm256_loadu_si256((const __m256i*)(acts + 128 * h));
            const __m256i a1 = _mm256_loadu_si256((const __m256i*)(acts + 128 * h + 32));
            const __m256i a2 = _mm256_loadu_si256((const __m256i*)(acts + 128 * h + 64));
            const __m256i a3 = _mm256_loadu_si256((const __m256i*)(acts + 128 * h + 96));
            const __m512i a_lo = _mm512_inserti64x4(_mm512_castsi256_si512(a0), a2, 1);
            const __m512i a_hi = _mm512_inserti64x4(_mm512_castsi256_si512(a1), a3, 1);
            const __m512i s_lo = _mm512_inserti64x4(_mm512_set1_epi32(sc[4 * h]), _mm256_set1_epi32(sc[4 * h + 2]), 1);
            const __m512i s_hi = _mm512_inserti64x4(_mm512_set1_epi32(sc[4 * h + 1]), _mm256_set1_epi32(sc[4 * h + 3]), 1);
            acc = _mm512_add_epi32(acc, _mm512_mullo_epi32(_mm512_dpbusd_epi32(_mm512_setzero_si512(), lo, a_lo), s_lo));
            acc = _mm512_add_epi32(acc, _mm512_mullo_epi32(_mm512_dpbusd_epi32(_mm512_setzero_si512(), hi, a_hi), s_hi));
            for (int r = 0; r < 2; ++r) {
                const int j = 2 * h + r;
                offset += (int32_t)mn[2 * j] * ((int32_t)bsums[4 * j] + bsums[4 * j + 1]);
                offset += (int32_t)mn[2 * j + 1] * ((int32_t)bsums[4 * j + 2] + bsums[4 * j + 3]);
            }
        }
        const int32_t scaled = _mm512_reduce_add_epi32(acc);
        total += yd * (f16_to_f32_hw(rd16(x)) * (float)scaled - f16_to_f32_hw(rd16(x + 2)) * (float)offset);
    }
    return total;
}
int lko_cpu_has_avx512(void) {
    return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512vl") &&
           __builtin_cpu_supports("avx512dq") && __builtin_cpu_supports("avx512vnni");
}
/* One Q4_K row against one Q8_K row through the 256-bit (wide = 0) or 512-bit (wide = 1) kernel. */
float lko_dot_q4k_q8k(int wide, const uint8_t* w, const uint8_t* y, size_t nb) {
    return wide ? dot_q4k_q8k_avx512(w, y, nb) : dot_q4k_q8k_avx2(w, y, nb);
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

/* ---------------------------------------------------------------------------------------------
 * Persistent worker pool (the shape of gemv_pool::Pool, src/tensor/quant_cpu/gemv_pool.rs:74-365):
 * workers are created once, one per physical core the process may run on (:186-203), and stay
 * alive; a job is published by bumping a generation counter, workers spin on it for a bounded
 * budget and then sleep on a condition variable; chunks are grabbed from one atomic counter and the
 * caller works alongside the workers and returns when every chunk has been finished.
 * ------------------------------------------------------------------------------------------- */
typedef void (*chunk_fn)(void* ctx, size_t chunk);

typedef struct {
    pthread_t* tid;
    int workers;                 /* threads beside the caller */
    atomic_uint generation;      /* bumped once per job */
    atomic_size_t next, done;    /* next chunk to grab; chunks finished */
    atomic_int active;           /* workers inside pool_drain: a job's state is not reused while one is */
    size_t n_chunks;
    chunk_fn fn;
    void* ctx;
    pthread_mutex_t mu;
    pthread_cond_t wake;
    atomic_int sleepers;
    atomic_int stop;
} pool_t;

static pool_t g_pool;
static pthread_mutex_t g_pool_mu = PTHREAD_MUTEX_INITIALIZER;
static int g_pool_threads = 0;
#define POOL_SPIN 20000   /* polls of the generation counter before a worker goes to sleep */

static void pool_drain(pool_t* p) {
    for (;;) {
        const size_t c = atomic_fetch_add(&p->next, 1);
        if (c >= p->n_chunks) break;
        p->fn(p->ctx, c);
        atomic_fetch_add(&p->done, 1);
    }
}

static void* pool_worker(void* arg) {
    pool_t* p = (pool_t*)arg;
    unsigned seen = atomic_load(&p->generation);
    for (;;) {
        int spins = 0;
        while (atomic_load_explicit(&p->generation, memory_order_acquire) == seen && !atomic_load(&p->stop)) {
            if (++spins < POOL_SPIN) {
                _mm_pause();
                continue;
            }
            pthread_mutex_lock(&p->mu);
            atomic_fetch_add(&p->sleepers, 1);
            while (atomic_load(&p->generation) == seen && !atomic_load(&p->stop)) pthread_cond_wait(&p->wake, &p->mu);
            atomic_fetch_sub(&p->sleepers, 1);
            pthread_mutex_unlock(&p->mu);
        }
        if (atomic_load(&p->stop)) return NULL;
        /* Entering is announced BEFORE the generation is read: pool_run bumps the generation and then
         * waits for `active` to fall to zero, so either it sees this worker and waits for it, or this
         * worker sees the new generation's state whole. */
        atomic_fetch_add(&p->active, 1);
        seen = atomic_load(&p->generation);
        pool_drain(p);
        atomic_fetch_sub(&p->active, 1);
    }
}

/* Physical cores this process may run on: distinct first entries of the siblings lists of the
 * CPUs in the affinity mask. Falls back to the number of CPUs in the mask. */
int lko_physical_cores(void) {
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof set, &set) != 0) return 1;
    int cores = 0, logical = 0;
    for (int cpu = 0; cpu < CPU_SETSIZE; ++cpu) {
        if (!CPU_ISSET(cpu, &set)) continue;
        ++logical;
        char path[128];
        snprintf(path, sizeof path, "/sys/devices/system/cpu/cpu%d/topology/thread_siblings_list", cpu);
        FILE* f = fopen(path, "r");
        int first = cpu;
        if (f) {
            if (fscanf(f, "%d", &first) != 1) first = cpu;
            fclose(f);
        }
        if (first == cpu) ++cores;   /* a core is counted at its lowest-numbered sibling */
    }
    return cores > 0 ? cores : (logical > 0 ? logical : 1);
}
int lko_logical_cpus(void) {
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof set, &set) != 0) return 1;
    return CPU_COUNT(&set);
}

/* Starts (or resizes) the pool: `threads` callers-plus-workers in all; 0 = one per physical core.
 * Returns the thread count in use. */
int lko_pool_start(int threads) {
    if (threads <= 0) threads = lko_physical_cores();
    pthread_mutex_lock(&g_pool_mu);
    if (g_pool_threads != threads) {
        if (g_pool_threads > 0) {   /* stop the old workers */
            atomic_store(&g_pool.stop, 1);
            pthread_mutex_lock(&g_pool.mu);
            pthread_cond_broadcast(&g_pool.wake);
            pthread_mutex_unlock(&g_pool.mu);
            for (int t = 0; t < g_pool.workers; ++t) pthread_join(g_pool.tid[t], NULL);
            free(g_pool.tid);
            pthread_mutex_destroy(&g_pool.mu);
            pthread_cond_destroy(&g_pool.wake);
        }
        memset(&g_pool, 0, sizeof g_pool);
        pthread_mutex_init(&g_pool.mu, NULL);
        pthread_cond_init(&g_pool.wake, NULL);
        g_pool.workers = threads - 1;
        g_pool.tid = (pthread_t*)calloc((size_t)(threads > 1 ? threads - 1 : 1), sizeof(pthread_t));
        int started = 0;
        if (g_pool.tid)
            for (; started < g_pool.workers; ++started)
                if (pthread_create(&g_pool.tid[started], NULL, pool_worker, &g_pool) != 0) break;
        g_pool.workers = started;
        g_pool_threads = started + 1;
    }
    const int n = g_pool_threads;
    pthread_mutex_unlock(&g_pool_mu);
    return n;
}

/* Runs fn(ctx, c) for c in [0, n_chunks) on the pool; returns when all are done. One job at a time. */
static void pool_run(size_t n_chunks, chunk_fn fn, void* ctx) {
    pool_t* p = &g_pool;
    p->fn = fn;
    p->ctx = ctx;
    p->n_chunks = n_chunks;
    atomic_store(&p->next, 0);
    atomic_store(&p->done, 0);
    atomic_fetch_add_explicit(&p->generation, 1, memory_order_release);
    if (atomic_load(&p->sleepers) > 0) {
        pthread_mutex_lock(&p->mu);
        pthread_cond_broadcast(&p->wake);
        pthread_mutex_unlock(&p->mu);
    }
    pool_drain(p);
    while (atomic_load_explicit(&p->done, memory_order_acquire) < n_chunks) _mm_pause();
    /* A worker that woke late may still be inside pool_drain (its grab found no chunk left, or it is
     * about to look): the next job's fn / ctx / counters are written only once nobody is in there,
     * so a stale grab can never be compared against the next job's chunk count. */
    while (atomic_load_explicit(&p->active, memory_order_acquire) != 0) _mm_pause();
}

/* ---------------------------------------------------------------------------------------------
 * The served Q4_K path: rows repacked eight at a time (BlockQ4Kx8, repack_q4k.rs:17-68) and one
 * group dot per eight output columns (gemv_group_scalar states the sums, :174-219; the AVX2
 * form is gemv_group_avx2_plain, :913-...; driver matmul_q4k_plain_pre, drivers.rs:61-95).
 *
 * Group block (2*8 f16 d and dmin, 8 x 12 packed scale bytes, 1024 bytes of nibbles): source byte
 * p of row j of the eight sits at qs[(p / 8) * 64 + j * 8 + p % 8], so step kk of the sixteen
 * holds eight bytes of every row side by side: values 8 (kk % 4) .. + 8 of sub-blocks 2 (kk / 4)
 * (low nibbles) and 2 (kk / 4) + 1 (high nibbles).
 *   out[j] = sum over blocks of  d_j * act.d * sum_s sc_js * dot_js  -  dmin_j * act.d * sum_s m_js * bsum_s
 * with every integer exact and the two float sums kept apart until the end, as the reference's.
 * ------------------------------------------------------------------------------------------- */
#define LKO_Q4KX8_BYTES (32 + 96 + 1024)

void lko_repack_q4k_x8(const uint8_t* rhs, size_t n, size_t nb, uint8_t* out) {
    for (size_t g = 0; g < n / 8; ++g)
        for (size_t b = 0; b < nb; ++b) {
            uint8_t* dst = out + (g * nb + b) * LKO_Q4KX8_BYTES;
            for (size_t j = 0; j < 8; ++j) {
                const uint8_t* src = rhs + ((g * 8 + j) * nb + b) * LKO_Q4K_BYTES;
                memcpy(dst + 2 * j, src, 2);             /* d */
                memcpy(dst + 16 + 2 * j, src + 2, 2);    /* dmin */
                memcpy(dst + 32 + 12 * j, src + 4, 12);  /* the row's own packed scales */
                for (size_t p = 0; p < 128; ++p) dst[128 + (p / 8) * 64 + j * 8 + (p % 8)] = src[16 + p];
            }
        }
}

/* Eight output columns from one group's `nb` blocks against one Q8_K row. */
static void gemv_group_q4k_x8(const uint8_t* grp, const uint8_t* y, size_t nb, float out[8]) {
    const __m256i nib = _mm256_set1_epi8(0x0F);
    __m256 acc = _mm256_setzero_ps(), acc_min = _mm256_setzero_ps();
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* blk = grp + b * LKO_Q4KX8_BYTES;
        const uint8_t* yb = y + b * LKO_Q8K_BYTES;
        float yd;
        memcpy(&yd, yb, 4);
        const int8_t* acts = (const int8_t*)(yb + 4);
        const int16_t* bsums = (const int16_t*)(yb + 260);
        /* the eight rows' scales and mins, sub-block major: tab[s][j] */
        int16_t sc[8][8], mn[8][8];
        for (int j = 0; j < 8; ++j) {
            uint8_t s8[8], m8[8];
            lko_unpack_scales_mins(blk + 32 + 12 * j, s8, m8);
            for (int s = 0; s < 8; ++s) { sc[s][j] = s8[s]; mn[s][j] = m8[s]; }
        }
        /* rows 0-3 in `ia`, rows 4-7 in `ib`: two int32 partials per row */
        __m256i ia = _mm256_setzero_si256(), ib = _mm256_setzero_si256();
        const uint8_t* qs = blk + 128;
        for (int pair = 0; pair < 4; ++pair) {
            __m256i lo_a = _mm256_setzero_si256(), lo_b = lo_a, hi_a = lo_a, hi_b = lo_a;
            for (int kk = 0; kk < 4; ++kk) {
                const __m256i qa = _mm256_loadu_si256((const __m256i*)(qs + (pair * 4 + kk) * 64));
                const __m256i qb = _mm256_loadu_si256((const __m256i*)(qs + (pair * 4 + kk) * 64 + 32));
                int64_t a_lo8, a_hi8;   /* the same eight activation codes against every row */
                memcpy(&a_lo8, acts + pair * 64 + kk * 8, 8);
                memcpy(&a_hi8, acts + pair * 64 + 32 + kk * 8, 8);
                const __m256i a_lo = _mm256_set1_epi64x(a_lo8), a_hi = _mm256_set1_epi64x(a_hi8);
                /* sixteen-bit partials: at most 4 steps x 2 products x 15 x 127, inside int16 */
                lo_a = _mm256_add_epi16(lo_a, _mm256_maddubs_epi16(_mm256_and_si256(qa, nib), a_lo));
                lo_b = _mm256_add_epi16(lo_b, _mm256_maddubs_epi16(_mm256_and_si256(qb, nib), a_lo));
                hi_a = _mm256_add_epi16(hi_a, _mm256_maddubs_epi16(_mm256_and_si256(_mm256_srli_epi16(qa, 4), nib), a_hi));
                hi_b = _mm256_add_epi16(hi_b, _mm256_maddubs_epi16(_mm256_and_si256(_mm256_srli_epi16(qb, 4), nib), a_hi));
            }
            /* each row's scale over its four sixteen-bit lanes: multiply, widen and pair-add in one */
            const int16_t* s0 = sc[2 * pair];
            const int16_t* s1 = sc[2 * pair + 1];
#define ROWS4(t, o) _mm256_setr_epi16(t[o], t[o], t[o], t[o], t[o + 1], t[o + 1], t[o + 1], t[o + 1], t[o + 2], t[o + 2], \
                                      t[o + 2], t[o + 2], t[o + 3], t[o + 3], t[o + 3], t[o + 3])
            ia = _mm256_add_epi32(ia, _mm256_add_epi32(_mm256_madd_epi16(lo_a, ROWS4(s0, 0)), _mm256_madd_epi16(hi_a, ROWS4(s1, 0))));
            ib = _mm256_add_epi32(ib, _mm256_add_epi32(_mm256_madd_epi16(lo_b, ROWS4(s0, 4)), _mm256_madd_epi16(hi_b, ROWS4(s1, 4))));
#undef ROWS4
        }
        /* [r0 r0 r1 r1 | r2 r2 r3 r3] and [r4 ..] -> one int32 per row, rows in lane order */
        const __m256i h = _mm256_hadd_epi32(ia, ib);   /* r0 r1 r4 r5 | r2 r3 r6 r7 */
        const __m256i sums = _mm256_permutevar8x32_epi32(h, _mm256_setr_epi32(0, 1, 4, 5, 2, 3, 6, 7));
        /* the min term: sum_s m_js * (bsums[2s] + bsums[2s+1]) */
        __m256i im = _mm256_setzero_si256();
        for (int s = 0; s < 8; ++s) {
            const int32_t bs = (int32_t)bsums[2 * s] + bsums[2 * s + 1];
            const __m256i m = _mm256_cvtepi16_epi32(_mm_loadu_si128((const __m128i*)mn[s]));
            im = _mm256_add_epi32(im, _mm256_mullo_epi32(m, _mm256_set1_epi32(bs)));
        }
        const __m256 d = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)blk));
        const __m256 dmin = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(blk + 16)));
        const __m256 ydv = _mm256_set1_ps(yd);
        acc = _mm256_fmadd_ps(_mm256_cvtepi32_ps(sums), _mm256_mul_ps(d, ydv), acc);
        acc_min = _mm256_fmadd_ps(_mm256_cvtepi32_ps(im), _mm256_mul_ps(dmin, ydv), acc_min);
    }
    _mm256_storeu_ps(out, _mm256_sub_ps(acc, acc_min));
}

typedef struct {
    size_t m, n, nb, groups, chunk;
    const uint8_t* x8;
    const uint8_t* act;   /* m rows of nb Q8_K blocks */
    float* dst;
} x8_job_t;

static void x8_chunk(void* ctx, size_t c) {
    const x8_job_t* j = (const x8_job_t*)ctx;
    const size_t g1 = (c + 1) * j->chunk < j->groups ? (c + 1) * j->chunk : j->groups;
    for (size_t g = c * j->chunk; g < g1; ++g) {
        const uint8_t* grp = j->x8 + g * j->nb * LKO_Q4KX8_BYTES;
        /* every activation row against the group while its blocks are in cache */
        for (size_t r = 0; r < j->m; ++r) {
            float out8[8];
            gemv_group_q4k_x8(grp, j->act + r * j->nb * LKO_Q8K_BYTES, j->nb, out8);
            memcpy(j->dst + r * j->n + g * 8, out8, sizeof out8);
        }
    }
}

/* dst[m, n] = lhs[m, k] x repacked Q4_K weights (`x8` from lko_repack_q4k_x8; n a multiple of 8),
 * Q8_K activations, on the persistent pool (started on first use, one worker per physical core
 * unless lko_pool_start chose otherwise). Column groups are dealt one chunk per thread
 * (drivers.rs:71-76). Returns 0, -1 (k not whole blocks), -4 (n not a multiple of 8), -5 (no memory). */
int oa_matmul_q4k_x8(size_t m, size_t k, size_t n, const float* lhs, const uint8_t* x8, float* dst) {
    if (k % LKO_QK_K != 0) return -1;
    if (n % 8 != 0) return -4;
    if (!lko_cpu_has_avx2()) return -3;
    const int threads = lko_pool_start(g_pool_threads > 0 ? g_pool_threads : 0);
    x8_job_t job;
    job.m = m; job.n = n; job.nb = k / LKO_QK_K; job.groups = n / 8; job.x8 = x8; job.dst = dst;
    uint8_t* act = (uint8_t*)malloc(job.nb * LKO_Q8K_BYTES * (m ? m : 1));
    if (!act) return -5;
    for (size_t r = 0; r < m; ++r) lko_quantize_q8_k(lhs + r * k, k, act + r * job.nb * LKO_Q8K_BYTES);
    job.act = act;
    job.chunk = (job.groups + (size_t)threads - 1) / (size_t)threads;
    if (job.chunk < 1) job.chunk = 1;
    pool_run((job.groups + job.chunk - 1) / job.chunk, x8_chunk, &job);
    free(act);
    return 0;
}

typedef float (*row_dot_fn)(const uint8_t*, const uint8_t*, size_t);

typedef struct {
    row_dot_fn dot;
    size_t m, n, nb, wrow, arow, chunk_cols, n_chunks;
    const uint8_t* rhs;
    const uint8_t* act;
    float* dst;
} job_t;

static void column_chunk(void* ctx, size_t c) {
    const job_t* j = (const job_t*)ctx;
    const size_t col0 = c * j->chunk_cols;
    const size_t col1 = col0 + j->chunk_cols < j->n ? col0 + j->chunk_cols : j->n;
    for (size_t r0 = 0; r0 < j->m; r0 += 8) {
        const size_t r1 = r0 + 8 < j->m ? r0 + 8 : j->m;
        for (size_t col = col0; col < col1; ++col)
            for (size_t r = r0; r < r1; ++r)
                j->dst[r * j->n + col] = j->dot(j->rhs + col * j->wrow, j->act + r * j->arow, j->nb);
    }
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
    threads = lko_pool_start(threads < 1 ? 1 : threads);
    job_t job;
    job.dot = dot; job.m = m; job.n = n; job.nb = k / blk; job.wrow = job.nb * wblk;
    job.arow = (k / aval) * ablk; job.rhs = rhs; job.dst = dst;
    uint8_t* act = (uint8_t*)malloc(job.arow * (m ? m : 1));
    if (!act) return -5;
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
    pool_run(job.n_chunks, column_chunk, &job);
    free(act);
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * The served prefill path: matmul_q4k_repacked_tiled (drivers.rs:231-339). The activation rows
 * are quantized to Q8_K in parallel over rows (quantize_act_q8k, :179-205), then ONE pool chunk
 * per group of eight columns computes all m rows of its columns, rows in tiles of eight. Inside a
 * tile the reference accumulates one row at a time and decodes the weight nibbles again per row
 * (its comment at :252-259: holding eight rows' partials spills); each row's eight sums are the
 * decode path's group dot, so the tile is that dot called per row and the result of a row does
 * not depend on m (the tests hold the driver to that, bit for bit).
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    size_t k, nb;
    const float* lhs;
    uint8_t* act;
} quant_job_t;

static void quant_row_chunk(void* ctx, size_t r) {
    const quant_job_t* j = (const quant_job_t*)ctx;
    lko_quantize_q8_k(j->lhs + r * j->k, j->k, j->act + r * j->nb * LKO_Q8K_BYTES);
}

static void x8_tiled_chunk(void* ctx, size_t g) {
    const x8_job_t* j = (const x8_job_t*)ctx;
    const uint8_t* grp = j->x8 + g * j->nb * LKO_Q4KX8_BYTES;
    for (size_t r = 0; r < j->m; r += 8) {
        const size_t mt = j->m - r < 8 ? j->m - r : 8;
        float local[64];
        for (size_t t = 0; t < mt; ++t) gemv_group_q4k_x8(grp, j->act + (r + t) * j->nb * LKO_Q8K_BYTES, j->nb, local + 8 * t);
        for (size_t t = 0; t < mt; ++t) memcpy(j->dst + (r + t) * j->n + g * 8, local + 8 * t, 8 * sizeof(float));
    }
}

int oa_matmul_q4k_x8_tiled(size_t m, size_t k, size_t n, const float* lhs, const uint8_t* x8, float* dst) {
    if (k % LKO_QK_K != 0) return -1;
    if (n % 8 != 0) return -4;
    if (!lko_cpu_has_avx2()) return -3;
    (void)lko_pool_start(g_pool_threads > 0 ? g_pool_threads : 0);
    x8_job_t job;
    job.m = m; job.n = n; job.nb = k / LKO_QK_K; job.groups = n / 8; job.x8 = x8; job.dst = dst; job.chunk = 1;
    uint8_t* act = (uint8_t*)malloc(job.nb * LKO_Q8K_BYTES * (m ? m : 1));
    if (!act) return -5;
    quant_job_t qj = {k, job.nb, lhs, act};
    pool_run(m, quant_row_chunk, &qj);
    job.act = act;
    pool_run(job.groups, x8_tiled_chunk, &job);
    free(act);
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Q6_K repacked eight rows at a time (BlockQ6Kx8, repack_q6k.rs:17-64: the planes are copied per
 * column, nothing is re-laid) and its prefill driver matmul_q6k_repacked_tiled (drivers.rs:
 * 341-406). Group block: 8 f16 d, 8 x 16 int8 scales, 8 x 128 bytes ql, 8 x 64 bytes qh.
 * The group dot follows gemm_group_avx2 (repack_q6k.rs:139-212): a column's 256 codes are decoded
 * ONCE per tile as unsigned 0..63, meet every row of the tile, and the zero point 32 comes off per
 * row as 32 * sum_g scale_g * bsum_g from the Q8_K row's sums of sixteen. Integers exact:
 *   out[r][j] += d_j * act_r.d * (sum_g scale_jg * dot_jg(unsigned) - 32 * sum_g scale_jg * bsum_rg)
 * ------------------------------------------------------------------------------------------- */
#define LKO_Q6KX8_BYTES (16 + 128 + 1024 + 512)

void lko_repack_q6k_x8(const uint8_t* rhs, size_t n, size_t nb, uint8_t* out) {
    for (size_t g = 0; g < n / 8; ++g)
        for (size_t b = 0; b < nb; ++b) {
            uint8_t* dst = out + (g * nb + b) * LKO_Q6KX8_BYTES;
            for (size_t j = 0; j < 8; ++j) {
                /* a Q6_K block: ql[128], qh[64], scales[16], d */
                const uint8_t* src = rhs + ((g * 8 + j) * nb + b) * LKO_Q6K_BYTES;
                memcpy(dst + 2 * j, src + 208, 2);
                memcpy(dst + 16 + 16 * j, src + 192, 16);
                memcpy(dst + 144 + 128 * j, src, 128);
                memcpy(dst + 1168 + 64 * j, src + 128, 64);
            }
        }
}

/* One group's `nb` blocks against `mt` (1..8) Q8_K rows: out[r * 8 + j], added to. */
static void gemm_group_q6k_x8(const uint8_t* grp, const uint8_t* const* rows, size_t mt, size_t nb, float* out) {
    const __m256i m4 = _mm256_set1_epi8(0xF), m2 = _mm256_set1_epi8(3);
    for (size_t l = 0; l < nb; ++l) {
        const uint8_t* blk = grp + l * LKO_Q6KX8_BYTES;
        for (int j = 0; j < 8; ++j) {
            const uint8_t* qlp = blk + 144 + 128 * j;
            const uint8_t* qhp = blk + 1168 + 64 * j;
            const int8_t* scp = (const int8_t*)(blk + 16 + 16 * j);
            __m256i wdec[8];
            for (int half = 0; half < 2; ++half) {
                const __m256i ql1 = _mm256_loadu_si256((const __m256i*)(qlp + 64 * half));
                const __m256i ql2 = _mm256_loadu_si256((const __m256i*)(qlp + 64 * half + 32));
                const __m256i qh = _mm256_loadu_si256((const __m256i*)(qhp + 32 * half));
                const __m256i h0 = _mm256_slli_epi16(_mm256_and_si256(qh, m2), 4);
                const __m256i h1 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(qh, 2), m2), 4);
                const __m256i h2 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(qh, 4), m2), 4);
                const __m256i h3 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(qh, 6), m2), 4);
                wdec[4 * half + 0] = _mm256_or_si256(_mm256_and_si256(ql1, m4), h0);
                wdec[4 * half + 1] = _mm256_or_si256(_mm256_and_si256(ql2, m4), h1);
                wdec[4 * half + 2] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(ql1, 4), m4), h2);
                wdec[4 * half + 3] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(ql2, 4), m4), h3);
            }
            /* chunk c of 32 codes spans the groups 2c (low sixteen) and 2c + 1 (high sixteen) */
            __m256i sv[8];
            for (int c = 0; c < 8; ++c)
                sv[c] = _mm256_insertf128_si256(_mm256_castsi128_si256(_mm_set1_epi16(scp[2 * c])), _mm_set1_epi16(scp[2 * c + 1]), 1);
            const __m256i scales16 = _mm256_cvtepi8_epi16(_mm_loadu_si128((const __m128i*)scp));
            const float dj = f16_to_f32_hw(rd16(blk + 2 * j));
            for (size_t r = 0; r < mt; ++r) {
                const uint8_t* yb = rows[r] + l * LKO_Q8K_BYTES;
                float yd;
                memcpy(&yd, yb, 4);
                const int8_t* q8 = (const int8_t*)(yb + 4);
                __m256i sumi = _mm256_setzero_si256();
                for (int c = 0; c < 8; ++c) {
                    const __m256i q = _mm256_loadu_si256((const __m256i*)(q8 + 32 * c));
                    sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(_mm256_maddubs_epi16(wdec[c], q), sv[c]));
                }
                const __m256i bsums = _mm256_loadu_si256((const __m256i*)(yb + 260));
                const __m256i corr = _mm256_slli_epi32(_mm256_madd_epi16(bsums, scales16), 5);
                const int32_t s = hsum_i32_8(_mm256_sub_epi32(sumi, corr));
                out[r * 8 + j] += dj * yd * (float)s;
            }
        }
    }
}

typedef struct {
    size_t m, n, nb;
    const uint8_t* x8;
    const uint8_t* act;
    float* dst;
} q6x8_job_t;

static void q6x8_tiled_chunk(void* ctx, size_t g) {
    const q6x8_job_t* j = (const q6x8_job_t*)ctx;
    const uint8_t* grp = j->x8 + g * j->nb * LKO_Q6KX8_BYTES;
    for (size_t r = 0; r < j->m; r += 8) {
        const size_t mt = j->m - r < 8 ? j->m - r : 8;
        const uint8_t* rows[8];
        for (size_t t = 0; t < mt; ++t) rows[t] = j->act + (r + t) * j->nb * LKO_Q8K_BYTES;
        float local[64];
        memset(local, 0, sizeof local);
        gemm_group_q6k_x8(grp, rows, mt, j->nb, local);
        for (size_t t = 0; t < mt; ++t) memcpy(j->dst + (r + t) * j->n + g * 8, local + 8 * t, 8 * sizeof(float));
    }
}

int oa_matmul_q6k_x8_tiled(size_t m, size_t k, size_t n, const float* lhs, const uint8_t* x8, float* dst) {
    if (k % LKO_QK_K != 0) return -1;
    if (n % 8 != 0) return -4;
    if (!lko_cpu_has_avx2()) return -3;
    (void)lko_pool_start(g_pool_threads > 0 ? g_pool_threads : 0);
    q6x8_job_t job;
    job.m = m; job.n = n; job.nb = k / LKO_QK_K; job.x8 = x8; job.dst = dst;
    uint8_t* act = (uint8_t*)malloc(job.nb * LKO_Q8K_BYTES * (m ? m : 1));
    if (!act) return -5;
    quant_job_t qj = {k, job.nb, lhs, act};
    pool_run(m, quant_row_chunk, &qj);
    job.act = act;
    pool_run(n / 8, q6x8_tiled_chunk, &job);
    free(act);
    return 0;
}

/* The scalar statement of the Q6_K group dot (gemv_group_scalar, repack_q6k.rs:96-123: "THE ORACLE"):
 * signed codes, one float fold per block and column. */
void lko_gemv_group_q6k_x8_scalar(const uint8_t* grp, const uint8_t* y, size_t nb, float out[8]) {
    float sumf[8] = {0};
    for (size_t l = 0; l < nb; ++l) {
        const uint8_t* blk = grp + l * LKO_Q6KX8_BYTES;
        const uint8_t* yb = y + l * LKO_Q8K_BYTES;
        float yd;
        memcpy(&yd, yb, 4);
        const int8_t* a = (const int8_t*)(yb + 4);
        for (int j = 0; j < 8; ++j) {
            const uint8_t* ql = blk + 144 + 128 * j;
            const uint8_t* qh = blk + 1168 + 64 * j;
            const int8_t* sc = (const int8_t*)(blk + 16 + 16 * j);
            int8_t aux[256];
            for (int jj = 0; jj < 256; jj += 128) {
                const uint8_t* q4 = ql + jj / 2;
                const uint8_t* qhh = qh + jj / 4;
                for (int e = 0; e < 32; ++e) {
                    aux[jj + e] = (int8_t)((int)((q4[e] & 0xF) | ((qhh[e] & 3) << 4)) - 32);
                    aux[jj + e + 32] = (int8_t)((int)((q4[e + 32] & 0xF) | (((qhh[e] >> 2) & 3) << 4)) - 32);
                    aux[jj + e + 64] = (int8_t)((int)((q4[e] >> 4) | (((qhh[e] >> 4) & 3) << 4)) - 32);
                    aux[jj + e + 96] = (int8_t)((int)((q4[e + 32] >> 4) | (((qhh[e] >> 6) & 3) << 4)) - 32);
                }
            }
            int32_t sumi = 0;
            for (int g = 0; g < 16; ++g) {
                int32_t gs = 0;
                for (int e = 0; e < 16; ++e) gs += (int32_t)aux[16 * g + e] * (int32_t)a[16 * g + e];
                sumi += (int32_t)sc[g] * gs;
            }
            sumf[j] += f16_to_f32_hw(rd16(blk + 2 * j)) * yd * (float)sumi;
        }
    }
    memcpy(out, sumf, sizeof sumf);
}

/* ---------------------------------------------------------------------------------------------
 * The MoE block on the pool: the scalar oracle's block (lko_moe_forward) over chunks of tokens, a
 * token's result depending on its own routed pairs only. The timed CPU figure beside the card's.
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    int family, dt_gu, dt_down, rc;
    size_t tokens, hidden, ffn, n_experts, topk, per;
    const float* x;
    const uint8_t *gate, *up, *down;
    const int32_t* ids;
    const float* weights;
    float* out;
} moe_job_t;

static void moe_chunk(void* ctx, size_t c) {
    moe_job_t* j = (moe_job_t*)ctx;
    const size_t t0 = c * j->per, t1 = t0 + j->per < j->tokens ? t0 + j->per : j->tokens;
    const int rc = lko_moe_forward(j->family, j->dt_gu, j->dt_down, t1 - t0, j->hidden, j->ffn, j->n_experts, j->topk,
                                   j->x + t0 * j->hidden, j->gate, j->up, j->down, j->ids + t0 * j->topk,
                                   j->weights + t0 * j->topk, NULL, j->out + t0 * j->hidden);
    if (rc) j->rc = rc;
}

int lko_moe_forward_pool(int family, int dt_gu, int dt_down, size_t tokens, size_t hidden, size_t ffn, size_t n_experts,
                         size_t topk, const float* x, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                         const int32_t* ids, const float* weights, float* out) {
    const int threads = lko_pool_start(g_pool_threads > 0 ? g_pool_threads : 0);
    moe_job_t job = {family, dt_gu, dt_down, 0, tokens, hidden, ffn, n_experts, topk, 1, x, gate, up, down, ids, weights, out};
    job.per = (tokens + (size_t)threads * 4 - 1) / ((size_t)threads * 4);
    if (job.per < 1) job.per = 1;
    pool_run((tokens + job.per - 1) / job.per, moe_chunk, &job);
    return job.rc;
}

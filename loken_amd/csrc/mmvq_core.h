// Row engines of the mat-vec family: one wave forms the dot products of R consecutive weight
// rows (of NW same-shaped weight matrices at once) against B staged Q8_1 activation rows, and
// hands each finished row to an epilogue. The plain mat-vec, the fused gate/up pair, grouped
// launches and the per-pair MoE decode kernels are all this engine with a different epilogue
// and a different way of choosing the weight slab.
//
// What each format computes follows loken's definitions: src/tensor/quant_cpu/format/q4_k.rs:62-88,
// q6_k.rs:51-82, q8_0.rs:83-97 for the integer sums, and the Q8_1-side combine of
// cuda/moe/gguf.cuh:664-685 (Q4_K), 782-816 (Q6_K), 486-495 (Q8_0).
#pragma once

#include "lk_common.h"

namespace mmvq {

constexpr int WG = 256;            // threads per workgroup
constexpr int WAVES = WG / LK_WAVE;

// --------------------------------------------------------------------------------------------
// Integer cores: what one lane forms from its 16 weight bytes. Shared by the mat-vec kernels and
// the sub-block-dot probe, so the probe shows the integers the product is built from.
// --------------------------------------------------------------------------------------------

// Q4_K: 16 bytes of qs = values l..l+15 of sub-block 2p (low nibbles) and of 2p+1 (high nibbles).
// Adds their products with the matching 16 activation codes of each sub-block into d_lo / d_hi.
static __device__ __forceinline__ void q4k_dots(const uint4& q, const uint4& a_lo, const uint4& a_hi,
                                                int& d_lo, int& d_hi) {
    uint4 lo, hi;
    lo.x = q.x & 0x0F0F0F0Fu; hi.x = (q.x >> 4) & 0x0F0F0F0Fu;
    lo.y = q.y & 0x0F0F0F0Fu; hi.y = (q.y >> 4) & 0x0F0F0F0Fu;
    lo.z = q.z & 0x0F0F0F0Fu; hi.z = (q.z >> 4) & 0x0F0F0F0Fu;
    lo.w = q.w & 0x0F0F0F0Fu; hi.w = (q.w >> 4) & 0x0F0F0F0Fu;
    d_lo = dot16(lo, a_lo, d_lo);
    d_hi = dot16(hi, a_hi, d_hi);
}

// The (scale, min) pairs of sub-blocks 2p, 2p+1 from the 12 packed bytes (words w1..w3 of the
// block header): scales in bits 0-7 / 8-15 of `sc`, mins likewise in `mn`. Sub-blocks 0-3 keep
// their six bits in one byte; 4-7 take a nibble from bytes 8-11 and two bits from the top of
// bytes 0-7. The selectors depend on the lane only, so they are built once outside any loop.
struct Q4KScaleSel {
    uint32_t shift, first, mask_main, mask_top;
    __device__ __forceinline__ explicit Q4KScaleSel(int p)
        : shift(16 * (p & 1)), first(p < 2), mask_main(p < 2 ? 0x3F3Fu : 0x0F0Fu), mask_top(p < 2 ? 0u : 0x3030u) {}
    __device__ __forceinline__ void unpack(uint32_t w1, uint32_t w2, uint32_t w3, uint32_t& sc, uint32_t& mn) const {
        const uint32_t a = w1 >> shift, b = w2 >> shift, c = w3 >> shift;
        sc = ((first ? a : c) & mask_main) | ((a >> 2) & mask_top);
        mn = ((first ? b : (c >> 4)) & mask_main) | ((b >> 2) & mask_top);
    }
};

// Q6_K: 16 bytes of ql and the 16 bytes of qh over the same l give two runs of 16 signed codes:
// run A in group g0 (low nibbles, qh bits 2*g0), run B in group g0+2 (high nibbles, bits 2*g0+4).
static __device__ __forceinline__ uint32_t q6k_word(uint32_t ql, uint32_t qh, int nib_shift, int hi_shift) {
    const uint32_t code = ((ql >> nib_shift) & 0x0F0F0F0Fu) | (((qh >> hi_shift) & 0x03030303u) << 4);
    // per byte: code - 32 as a signed byte (code <= 63, so +0x60 cannot carry into the next byte)
    return (code + 0x60606060u) ^ 0x80808080u;
}
static __device__ __forceinline__ void q6k_dots(const uint4& ql, const uint4& qh, int g0,
                                                const uint4& a_a, const uint4& a_b, int& d_a, int& d_b) {
    uint4 ca, cb;
    const int s = 2 * g0;
    ca.x = q6k_word(ql.x, qh.x, 0, s); cb.x = q6k_word(ql.x, qh.x, 4, s + 4);
    ca.y = q6k_word(ql.y, qh.y, 0, s); cb.y = q6k_word(ql.y, qh.y, 4, s + 4);
    ca.z = q6k_word(ql.z, qh.z, 0, s); cb.z = q6k_word(ql.z, qh.z, 4, s + 4);
    ca.w = q6k_word(ql.w, qh.w, 0, s); cb.w = q6k_word(ql.w, qh.w, 4, s + 4);
    d_a = dot16(ca, a_a, 0);
    d_b = dot16(cb, a_b, 0);
}

// --------------------------------------------------------------------------------------------
// Activation staging. Formats differ only in where a Q8_1 block's two 16-byte halves land.
// LDS per activation row: `n_iter` passes x `PLANES` planes x 1024 bytes of codes, then the
// scale table (SCF floats per Q8_1 block).
// --------------------------------------------------------------------------------------------

struct FmtQ4K {
    static constexpr int BLOCK_BYTES = Q4K_BYTES, BLOCK_LEN = 256;
    static constexpr int VPI = 4096;   // values per wave pass: 16 super-blocks, 4 lanes each
    static constexpr int PLANES = 4, SCF = 2;
    // j: Q8_1 block index inside the pass (0..127), lh: which 16-byte half of its codes.
    // Lane (block lb, pair p) reads plane (2 * odd + lh) at lane * 16.
    static __device__ __forceinline__ int slot(int j, int lh) {
        const int lb = j >> 3, s = j & 7;
        return ((s & 1) * 2 + lh) * 1024 + (lb * 4 + (s >> 1)) * 16;
    }
};
struct FmtQ6K {
    static constexpr int BLOCK_BYTES = Q6K_BYTES, BLOCK_LEN = 256;
    static constexpr int VPI = 2048;
    static constexpr int PLANES = 2, SCF = 1;
    static __device__ __forceinline__ int slot(int j, int lh) {
        const int lb = j >> 3, s = j & 7, h = s >> 2, g = s & 3;
        return (g >> 1) * 1024 + (lb * 8 + h * 4 + (g & 1) * 2 + lh) * 16;
    }
};
struct FmtQ80 {
    static constexpr int BLOCK_BYTES = Q80_BYTES, BLOCK_LEN = 32;
    static constexpr int VPI = 1024;
    static constexpr int PLANES = 1, SCF = 1;
    static __device__ __forceinline__ int slot(int j, int lh) { return j * 32 + lh * 16; }
};

template <class F>
static __host__ __device__ constexpr int lds_bytes_per_row(int n_iter) {
    return n_iter * F::VPI + n_iter * (F::VPI / 32) * F::SCF * 4;
}

// Stage `batch` Q8_1 rows. k32 = real Q8_1 blocks per row; the rest of the last pass is zeroed.
template <class F, int B>
static __device__ __forceinline__ void stage_activation(uint8_t* lds, const uint8_t* __restrict__ vy,
                                                        int k32, int n_iter, int stride_col_y) {
    const int per_pass = F::VPI / 32;
    const int total = n_iter * per_pass;
    const int row_bytes = lds_bytes_per_row<F>(n_iter);
    for (int j = threadIdx.x; j < total; j += WG) {
        const int it = j / per_pass, ji = j % per_pass;
#pragma unroll
        for (int c = 0; c < B; ++c) {
            uint8_t* row = lds + c * row_bytes;
            float* sc = (float*)(row + n_iter * F::VPI);
            uint4 lo = make_uint4(0, 0, 0, 0), hi = make_uint4(0, 0, 0, 0);
            float d8 = 0.f, ds = 0.f;
            if (j < k32) {
                const uint32_t* src = (const uint32_t*)(vy + ((size_t)c * stride_col_y + j) * Q81_BYTES);
                const uint32_t head = src[0];
                lo = make_uint4(src[1], src[2], src[3], src[4]);
                hi = make_uint4(src[5], src[6], src[7], src[8]);
                d8 = f16_bits_to_f32(head & 0xFFFFu);
                if (F::SCF == 2) {
                    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
                    ds = d8 * (float)dot16(ones, hi, dot16(ones, lo, 0));
                }
            }
            uint8_t* codes = row + it * F::PLANES * 1024;
            *(uint4*)(codes + F::slot(ji, 0)) = lo;
            *(uint4*)(codes + F::slot(ji, 1)) = hi;
            if (F::SCF == 2) {
                *(float2*)(sc + 2 * j) = make_float2(d8, ds);
            } else {
                sc[j] = d8;
            }
        }
    }
}


// The same staging from f32 rows: the workgroup quantizes each 32-value block itself, with the
// steps of the stand-alone quantizer (d = amax/127 rounded to f16, codes = round_half_away(x *
// (1/d)) with d before its rounding, integer code sum), so the staged bytes are the ones the
// two-launch path stages. Eight lanes own a block, four values each.
template <class F, int B>
static __device__ __forceinline__ void stage_activation_f32(uint8_t* lds, const float* __restrict__ x, int k32,
                                                            int n_iter, int x_stride) {
#pragma clang fp contract(off)
    const int per_pass = F::VPI / 32;
    const int total = n_iter * per_pass;
    const int row_bytes = lds_bytes_per_row<F>(n_iter);
    constexpr int U = 4;  // loads issued together: the lane exchanges below would otherwise
                          // serialize one memory latency per 1024 values
    for (int t0 = threadIdx.x; t0 < total * 8; t0 += WG * U) {
#pragma unroll
        for (int c = 0; c < B; ++c) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int t = t0 + u * WG, j = t >> 3, l8 = t & 7;
                v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (t < total * 8 && j < k32) v[u] = *(const float4*)(x + (size_t)c * x_stride + j * 32 + l8 * 4);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int t = t0 + u * WG, j = t >> 3, l8 = t & 7;
                if (t >= total * 8) break;
                const int it = j / per_pass, ji = j % per_pass;
                float amax = fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w)));
                amax = fmaxf(amax, __shfl_xor(amax, 1));
                amax = fmaxf(amax, __shfl_xor(amax, 2));
                amax = fmaxf(amax, __shfl_xor(amax, 4));
                const float d = amax / 127.0f;
                const float inv = d != 0.0f ? 1.0f / d : 0.0f;
                const int q0 = (int)roundf(v[u].x * inv), q1 = (int)roundf(v[u].y * inv);
                const int q2 = (int)roundf(v[u].z * inv), q3 = (int)roundf(v[u].w * inv);
                int sum = q0 + q1 + q2 + q3;
                sum += __shfl_xor(sum, 1);
                sum += __shfl_xor(sum, 2);
                sum += __shfl_xor(sum, 4);
                uint8_t* row = lds + c * row_bytes;
                uint8_t* codes = row + it * F::PLANES * 1024;
                *(uint32_t*)(codes + F::slot(ji, l8 >> 2) + 4 * (l8 & 3)) =
                    (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
                    ((uint32_t)(q3 & 0xFF) << 24);
                if (l8 == 0) {
                    float* sc = (float*)(row + n_iter * F::VPI);
                    const float d8 = __half2float(__float2half_rn(d));
                    if (F::SCF == 2) {
                        *(float2*)(sc + 2 * j) = make_float2(d8, d8 * (float)sum);
                    } else {
                        sc[j] = d8;
                    }
                }
            }
        }
    }
}

// What a workgroup computes: rows of `vx[0..NW)` against the B activation rows at `vy`.
template <int NW>
struct RowJob {
    const uint8_t* vx[NW];
    const uint8_t* vy;
    int nb;            // format blocks per weight row
    int n;             // weight rows
    int stride_col_y;  // Q8_1 blocks between activation rows
    int tile_stride;   // row tiles between a wave's consecutive tiles
    int tile_first;    // first row tile of wave 0 of this workgroup
    int act_stride_f32 = 0;  // non-zero: `vy` holds f32 activation rows this many floats apart,
                             // quantized to Q8_1 by the workgroup itself while staging
};

// The activation as the engines stage it, whichever form it arrives in.
template <class F, int B, int NW>
static __device__ __forceinline__ void stage_job(uint8_t* lds, const RowJob<NW>& job, int k32, int n_iter) {
    if (job.act_stride_f32)
        stage_activation_f32<F, B>(lds, (const float*)job.vy, k32, n_iter, job.act_stride_f32);
    else
        stage_activation<F, B>(lds, job.vy, k32, n_iter, job.stride_col_y);
}

// ---------------------------------------------------------------------------------------------
// Q4_K: 4 lanes per super-block (32 bytes of qs each = two whole sub-blocks), 16 super-blocks
// per wave pass, loads of the next step in flight while the current one is consumed.
// epi(row, col, totals[NW]) runs on lane 0 for every finished (row, activation row).
// ---------------------------------------------------------------------------------------------
template <int B, int R, int NW, class Epi>
static __device__ __forceinline__ void rows_q4k(const RowJob<NW>& job, uint8_t* lds, Epi&& epi) {
    const int nb = job.nb, n = job.n;
    const int n_iter = (nb + 15) >> 4;
    const int row_bytes = lds_bytes_per_row<FmtQ4K>(n_iter);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lb = lane >> 2, p = lane & 3;
    const Q4KScaleSel sel(p);
    const uint32_t hdr_off = lb * Q4K_BYTES, qs_off = hdr_off + 16 + 32 * p;
    const size_t row_stride = (size_t)nb * Q4K_BYTES;
    const int n_tiles = (n + R - 1) / R;
    constexpr int RW = R * NW;

    struct Frag {
        uint4 hdr[RW], q0[RW], q1[RW];
    };
    // One pass (16 super-blocks) of R rows of every matrix into registers. A lane past the row
    // end re-reads the row's last block and drops its d / dmin, so it adds nothing.
    auto load = [&](Frag& f, int tile, int it) {
        const bool valid = it * 16 + lb < nb;
        const uint32_t back = valid ? 0u : (uint32_t)(it * 16 + lb - (nb - 1)) * Q4K_BYTES;
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = min(tile * R + r, n - 1);
                const uint8_t* bp = job.vx[w] + row * row_stride + (size_t)it * (16 * Q4K_BYTES);
                Frag& g = f;
                g.hdr[w * R + r] = *(const uint4*)(bp + (hdr_off - back));
                g.q0[w * R + r] = *(const uint4*)(bp + (qs_off - back));
                g.q1[w * R + r] = *(const uint4*)(bp + (qs_off - back + 16));
                if (!valid) g.hdr[w * R + r].x = 0;
            }
    };

    float acc[RW][B];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

    auto compute = [&](const Frag& f, int tile, int it) {
        float d[RW], dmin[RW], scl[RW], sch[RW], ml[RW], mh[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            uint32_t sc, mn;
            sel.unpack(f.hdr[r].y, f.hdr[r].z, f.hdr[r].w, sc, mn);
            d[r] = f16_bits_to_f32(f.hdr[r].x & 0xFFFFu);
            dmin[r] = f16_bits_to_f32(f.hdr[r].x >> 16);
            scl[r] = (float)(sc & 0xFFu);
            sch[r] = (float)(sc >> 8);
            ml[r] = (float)(mn & 0xFFu);
            mh[r] = (float)(mn >> 8);
        }
#pragma unroll
        for (int c = 0; c < B; ++c) {
            const uint8_t* rowl = lds + c * row_bytes;
            const uint8_t* codes = rowl + it * 4096 + lane * 16;
            const uint4 a00 = *(const uint4*)(codes);
            const uint4 a01 = *(const uint4*)(codes + 1024);
            const uint4 a10 = *(const uint4*)(codes + 2048);
            const uint4 a11 = *(const uint4*)(codes + 3072);
            const float4 s4 = *(const float4*)(rowl + n_iter * 4096 + (size_t)((it * 16 + lb) * 8 + 2 * p) * 8);
#pragma unroll
            for (int r = 0; r < RW; ++r) {
                int d_lo = 0, d_hi = 0;
                q4k_dots(f.q0[r], a00, a10, d_lo, d_hi);
                q4k_dots(f.q1[r], a01, a11, d_lo, d_hi);
                const float u = (scl[r] * s4.x) * (float)d_lo + (sch[r] * s4.z) * (float)d_hi;
                const float w = ml[r] * s4.y + mh[r] * s4.w;
                acc[r][c] += d[r] * u - dmin[r] * w;
            }
        }
        if (it == n_iter - 1) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int c = 0; c < B; ++c) {
                    float tot[NW];
#pragma unroll
                    for (int w = 0; w < NW; ++w) {
                        tot[w] = wave_sum(acc[w * R + r][c]);
                        acc[w * R + r][c] = 0.f;
                    }
                    if (lane == 0 && tile * R + r < n) epi(tile * R + r, c, tot);
                }
        }
    };

    // The first weight loads go out before the activation is staged, so the two memory
    // latencies overlap instead of adding up (most of a small matrix's run time).
    int tile = job.tile_first + wave, it = 0;
    Frag fa, fb;
    if (tile < n_tiles) load(fa, tile, 0);
    stage_job<FmtQ4K, B>(lds, job, nb * 8, n_iter);
    __syncthreads();
    if (tile >= n_tiles) return;
    // Steps are (tile, pass) pairs in order; the loads of step i+1 are issued before step i is
    // consumed, ping-ponging between two register fragments.
    for (;;) {
        int nt = tile, ni = it + 1;
        if (ni == n_iter) { ni = 0; nt += job.tile_stride; }
        if (nt < n_tiles) load(fb, nt, ni);
        compute(fa, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
        nt = tile; ni = it + 1;
        if (ni == n_iter) { ni = 0; nt += job.tile_stride; }
        if (nt < n_tiles) load(fa, nt, ni);
        compute(fb, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
    }
}

// ---------------------------------------------------------------------------------------------
// Q6_K: 8 lanes per super-block (16 bytes of ql + the matching 16 of qh = two runs of 16 codes).
// ---------------------------------------------------------------------------------------------
template <int B, int R, int NW, class Epi>
static __device__ __forceinline__ void rows_q6k(const RowJob<NW>& job, uint8_t* lds, Epi&& epi) {
    const int nb = job.nb, n = job.n;
    const int n_iter = (nb + 7) >> 3;
    const int row_bytes = lds_bytes_per_row<FmtQ6K>(n_iter);
    stage_job<FmtQ6K, B>(lds, job, nb * 8, n_iter);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lb = lane >> 3, ch = lane & 7;
    const int h = ch >> 2, g0 = (ch >> 1) & 1, lh = ch & 1;
    const size_t row_stride = (size_t)nb * Q6K_BYTES;
    const int n_tiles = (n + R - 1) / R;
    constexpr int RW = R * NW;

    for (int tile = job.tile_first + wave; tile < n_tiles; tile += job.tile_stride) {
        const int row0 = tile * R;
        float acc[RW][B];
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

        for (int it = 0; it < n_iter; ++it) {
            const int blk = it * 8 + lb;
            const bool valid = blk < nb;
            const int blk_c = valid ? blk : nb - 1;
            uint4 ql[RW], qh[RW];
            float dsa[RW], dsb[RW];
#pragma unroll
            for (int w = 0; w < NW; ++w)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int row = min(row0 + r, n - 1);
                    const uint8_t* bp = job.vx[w] + row * row_stride + (size_t)blk_c * Q6K_BYTES;
                    ql[w * R + r] = *(const uint4_a2*)(bp + 16 * ch);
                    qh[w * R + r] = *(const uint4_a2*)(bp + 128 + 16 * (2 * h + lh));
                    const int sa = ((const int8_t*)bp)[192 + 8 * h + 2 * g0 + lh];
                    const int sb = ((const int8_t*)bp)[192 + 8 * h + 2 * g0 + 4 + lh];
                    const float d = valid ? f16_bits_to_f32(*(const uint16_t*)(bp + 208)) : 0.f;
                    dsa[w * R + r] = d * (float)sa;
                    dsb[w * R + r] = d * (float)sb;
                }
#pragma unroll
            for (int c = 0; c < B; ++c) {
                const uint8_t* rowl = lds + c * row_bytes;
                const uint8_t* codes = rowl + it * 2048;
                const uint4 a_a = *(const uint4*)(codes + lane * 16);
                const uint4 a_b = *(const uint4*)(codes + 1024 + lane * 16);
                const float* sc = (const float*)(rowl + n_iter * 2048);
                const float d8a = sc[blk * 8 + 4 * h + g0];
                const float d8b = sc[blk * 8 + 4 * h + g0 + 2];
#pragma unroll
                for (int r = 0; r < RW; ++r) {
                    int d_a, d_b;
                    q6k_dots(ql[r], qh[r], g0, a_a, a_b, d_a, d_b);
                    acc[r][c] += dsa[r] * (d8a * (float)d_a) + dsb[r] * (d8b * (float)d_b);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < B; ++c) {
                float tot[NW];
#pragma unroll
                for (int w = 0; w < NW; ++w) tot[w] = wave_sum(acc[w * R + r][c]);
                if (lane == 0 && row0 + r < n) epi(row0 + r, c, tot);
            }
    }
}

// ---------------------------------------------------------------------------------------------
// Q8_0: 2 lanes per 32-value block, 32 blocks per wave pass.
// ---------------------------------------------------------------------------------------------
template <int B, int R, int NW, class Epi>
static __device__ __forceinline__ void rows_q80(const RowJob<NW>& job, uint8_t* lds, Epi&& epi) {
    const int nb = job.nb, n = job.n;
    const int n_iter = (nb + 31) >> 5;
    const int row_bytes = lds_bytes_per_row<FmtQ80>(n_iter);
    stage_job<FmtQ80, B>(lds, job, nb, n_iter);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lb = lane >> 1, lh = lane & 1;
    const size_t row_stride = (size_t)nb * Q80_BYTES;
    const int n_tiles = (n + R - 1) / R;
    constexpr int RW = R * NW;

    for (int tile = job.tile_first + wave; tile < n_tiles; tile += job.tile_stride) {
        const int row0 = tile * R;
        float acc[RW][B];
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

        for (int it = 0; it < n_iter; ++it) {
            const int blk = it * 32 + lb;
            const bool valid = blk < nb;
            const int blk_c = valid ? blk : nb - 1;
            uint4 q[RW];
            float d[RW];
#pragma unroll
            for (int w = 0; w < NW; ++w)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int row = min(row0 + r, n - 1);
                    const uint8_t* bp = job.vx[w] + row * row_stride + (size_t)blk_c * Q80_BYTES;
                    q[w * R + r] = *(const uint4_a2*)(bp + 2 + 16 * lh);
                    d[w * R + r] = valid ? f16_bits_to_f32(*(const uint16_t*)bp) : 0.f;
                }
#pragma unroll
            for (int c = 0; c < B; ++c) {
                const uint8_t* rowl = lds + c * row_bytes;
                const uint4 a = *(const uint4*)(rowl + it * 1024 + lane * 16);
                const float d8 = ((const float*)(rowl + n_iter * 1024))[blk];
#pragma unroll
                for (int r = 0; r < RW; ++r) acc[r][c] += (d[r] * d8) * (float)dot16(q[r], a, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < B; ++c) {
                float tot[NW];
#pragma unroll
                for (int w = 0; w < NW; ++w) tot[w] = wave_sum(acc[w * R + r][c]);
                if (lane == 0 && row0 + r < n) epi(row0 + r, c, tot);
            }
    }
}

// Format tags: which engine serves a ggml type, and its LDS footprint.
struct EngQ4K {
    using Fmt = FmtQ4K;
    template <int B, int R, int NW, class Epi>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e) { rows_q4k<B, R, NW>(j, lds, e); }
};
struct EngQ6K {
    using Fmt = FmtQ6K;
    template <int B, int R, int NW, class Epi>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e) { rows_q6k<B, R, NW>(j, lds, e); }
};
struct EngQ80 {
    using Fmt = FmtQ80;
    template <int B, int R, int NW, class Epi>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e) { rows_q80<B, R, NW>(j, lds, e); }
};

template <class F>
static inline int n_iter_of(int nb) {
    const int per = F::VPI / F::BLOCK_LEN;
    return (nb + per - 1) / per;
}
template <class F>
static inline int lds_bytes_for(int nb, int batch) {
    return batch * lds_bytes_per_row<F>(n_iter_of<F>(nb));
}

static inline int block_len_of(int wtype) {
    switch (wtype) {
        case LK_TYPE_Q4_K: case LK_TYPE_Q6_K: return 256;
        case LK_TYPE_Q8_0: return 32;
        default: return 0;
    }
}
static inline int block_bytes_of(int wtype) {
    switch (wtype) {
        case LK_TYPE_Q4_K: return Q4K_BYTES;
        case LK_TYPE_Q6_K: return Q6K_BYTES;
        case LK_TYPE_Q8_0: return Q80_BYTES;
        default: return 0;
    }
}

}  // namespace mmvq

// Decode mat-vec: GGUF weight rows (Q4_K / Q6_K / Q8_0) against 1..8 Q8_1 activation rows.
//
// Bandwidth work, so the design is about bytes in flight, not arithmetic:
//   * a lane loads 16 weight bytes per instruction (global_load_dwordx4) and a wave takes whole
//     super-blocks side by side: Q4_K / Q6_K 8 lanes per 256-value block (8 blocks = 2048 values
//     per wave pass), Q8_0 2 lanes per 32-value block (32 blocks = 1024 values per pass);
//   * a wave owns R consecutive weight rows end to end (no cross-wave reduction), issues the
//     loads of all R rows before it consumes any, and persists over row tiles;
//   * the Q8_1 activation is staged ONCE per workgroup into LDS, re-laid so that the 16 bytes a
//     lane needs sit at lane*16 of a plane (conflict-free ds_read_b128), with its f16 scales
//     widened to f32 and, for Q4_K, d8 * sum(codes) precomputed for the min term;
//   * 6-bit scales / mins are unpacked in registers from the 16-byte block header;
//   * integer products are v_dot4_i32_i8; the per-lane f32 partials meet in one wave64 DPP
//     reduction per row.
//
// What each format computes follows loken's definitions: src/tensor/quant_cpu/format/q4_k.rs:62-88,
// q6_k.rs:51-82, q8_0.rs:83-97 for the integer sums, and the Q8_1-side combine of
// cuda/moe/gguf.cuh:664-685 (Q4_K), 782-816 (Q6_K), 486-495 (Q8_0).

#include "lk_common.h"

#include <cstdlib>
#include <mutex>
#include <unordered_map>

namespace {

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

template <typename T>
static __device__ __forceinline__ void store_out(T* dst, int stride_col_dst, int col, int row, float v,
                                                 const float* bias) {
    if (bias) v += bias[row];
    dst[(size_t)col * stride_col_dst + row] = from_f32<T>(v);
}

// --------------------------------------------------------------------------------------------
// Q4_K
// --------------------------------------------------------------------------------------------
template <int B, int R, typename T>
__global__ __launch_bounds__(WG) void mmvq_q4k_kernel(const uint8_t* __restrict__ vx,
                                                      const uint8_t* __restrict__ vy, T* __restrict__ dst,
                                                      int nb, int n, int stride_col_y, int stride_col_dst,
                                                      const float* __restrict__ bias) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int n_iter = (nb + 15) >> 4;
    const int row_bytes = lds_bytes_per_row<FmtQ4K>(n_iter);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lb = lane >> 2, p = lane & 3;
    const Q4KScaleSel sel(p);
    const uint32_t hdr_off = lb * Q4K_BYTES, qs_off = hdr_off + 16 + 32 * p;
    const size_t row_stride = (size_t)nb * Q4K_BYTES;
    const int n_tiles = (n + R - 1) / R;
    const int tile_stride = gridDim.x * WAVES;

    struct Frag {
        uint4 hdr[R], q0[R], q1[R];
    };
    // One pass (16 super-blocks) of R rows into registers. Lanes past the row end hold zeros:
    // d = dmin = 0 and the staged activation tail is zero, so they add nothing.
    auto load = [&](Frag& f, int tile, int it) {
        const bool valid = it * 16 + lb < nb;
        // an out-of-range lane re-reads the row's last block and drops its d / dmin
        const uint32_t back = valid ? 0u : (uint32_t)(it * 16 + lb - (nb - 1)) * Q4K_BYTES;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = min(tile * R + r, n - 1);
            const uint8_t* bp = vx + row * row_stride + (size_t)it * (16 * Q4K_BYTES);
            f.hdr[r] = *(const uint4*)(bp + (hdr_off - back));
            f.q0[r] = *(const uint4*)(bp + (qs_off - back));
            f.q1[r] = *(const uint4*)(bp + (qs_off - back + 16));
            if (!valid) f.hdr[r].x = 0;
        }
    };

    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

    auto compute = [&](const Frag& f, int tile, int it) {
        float d[R], dmin[R], scl[R], sch[R], ml[R], mh[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
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
            for (int r = 0; r < R; ++r) {
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
                    const float total = wave_sum(acc[r][c]);
                    acc[r][c] = 0.f;
                    if (lane == 0 && tile * R + r < n) store_out(dst, stride_col_dst, c, tile * R + r, total, bias);
                }
        }
    };

    // Steps are (tile, pass) pairs in order; the loads of step i+1 are issued before step i is
    // consumed, ping-ponging between two register fragments.
    // The first weight loads go out before the activation is staged, so the two memory
    // latencies overlap instead of adding up (it is most of a small matrix's run time).
    int tile = blockIdx.x * WAVES + wave, it = 0;
    Frag fa, fb;
    if (tile < n_tiles) load(fa, tile, 0);
    stage_activation<FmtQ4K, B>(lds, vy, nb * 8, n_iter, stride_col_y);
    __syncthreads();
    if (tile >= n_tiles) return;
    for (;;) {
        int nt = tile, ni = it + 1;
        if (ni == n_iter) { ni = 0; nt += tile_stride; }
        if (nt < n_tiles) load(fb, nt, ni);
        compute(fa, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
        nt = tile; ni = it + 1;
        if (ni == n_iter) { ni = 0; nt += tile_stride; }
        if (nt < n_tiles) load(fa, nt, ni);
        compute(fb, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
    }
}

// --------------------------------------------------------------------------------------------
// Q6_K
// --------------------------------------------------------------------------------------------
template <int B, int R, typename T>
__global__ __launch_bounds__(WG) void mmvq_q6k_kernel(const uint8_t* __restrict__ vx,
                                                      const uint8_t* __restrict__ vy, T* __restrict__ dst,
                                                      int nb, int n, int stride_col_y, int stride_col_dst,
                                                      const float* __restrict__ bias) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int n_iter = (nb + 7) >> 3;
    const int row_bytes = lds_bytes_per_row<FmtQ6K>(n_iter);
    stage_activation<FmtQ6K, B>(lds, vy, nb * 8, n_iter, stride_col_y);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lb = lane >> 3, ch = lane & 7;
    const int h = ch >> 2, g0 = (ch >> 1) & 1, lh = ch & 1;
    const size_t row_stride = (size_t)nb * Q6K_BYTES;

    for (int tile = blockIdx.x * WAVES + wave; tile * R < n; tile += gridDim.x * WAVES) {
        const int row0 = tile * R;
        float acc[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

        for (int it = 0; it < n_iter; ++it) {
            const int blk = it * 8 + lb;
            const bool valid = blk < nb;
            const int blk_c = valid ? blk : nb - 1;
            uint4 ql[R], qh[R];
            float dsa[R], dsb[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = min(row0 + r, n - 1);
                const uint8_t* bp = vx + row * row_stride + (size_t)blk_c * Q6K_BYTES;
                ql[r] = *(const uint4_a2*)(bp + 16 * ch);
                qh[r] = *(const uint4_a2*)(bp + 128 + 16 * (2 * h + lh));
                const int sa = ((const int8_t*)bp)[192 + 8 * h + 2 * g0 + lh];
                const int sb = ((const int8_t*)bp)[192 + 8 * h + 2 * g0 + 4 + lh];
                const float d = valid ? f16_bits_to_f32(*(const uint16_t*)(bp + 208)) : 0.f;
                dsa[r] = d * (float)sa;
                dsb[r] = d * (float)sb;
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
                for (int r = 0; r < R; ++r) {
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
                const float total = wave_sum(acc[r][c]);
                if (lane == 0 && row0 + r < n) store_out(dst, stride_col_dst, c, row0 + r, total, bias);
            }
    }
}

// --------------------------------------------------------------------------------------------
// Q8_0
// --------------------------------------------------------------------------------------------
template <int B, int R, typename T>
__global__ __launch_bounds__(WG) void mmvq_q80_kernel(const uint8_t* __restrict__ vx,
                                                      const uint8_t* __restrict__ vy, T* __restrict__ dst,
                                                      int nb, int n, int stride_col_y, int stride_col_dst,
                                                      const float* __restrict__ bias) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int n_iter = (nb + 31) >> 5;
    const int row_bytes = lds_bytes_per_row<FmtQ80>(n_iter);
    stage_activation<FmtQ80, B>(lds, vy, nb, n_iter, stride_col_y);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lb = lane >> 1, lh = lane & 1;
    const size_t row_stride = (size_t)nb * Q80_BYTES;

    for (int tile = blockIdx.x * WAVES + wave; tile * R < n; tile += gridDim.x * WAVES) {
        const int row0 = tile * R;
        float acc[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

        for (int it = 0; it < n_iter; ++it) {
            const int blk = it * 32 + lb;
            const bool valid = blk < nb;
            const int blk_c = valid ? blk : nb - 1;
            uint4 q[R];
            float d[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = min(row0 + r, n - 1);
                const uint8_t* bp = vx + row * row_stride + (size_t)blk_c * Q80_BYTES;
                q[r] = *(const uint4_a2*)(bp + 2 + 16 * lh);
                d[r] = valid ? f16_bits_to_f32(*(const uint16_t*)bp) : 0.f;
            }
#pragma unroll
            for (int c = 0; c < B; ++c) {
                const uint8_t* rowl = lds + c * row_bytes;
                const uint4 a = *(const uint4*)(rowl + it * 1024 + lane * 16);
                const float d8 = ((const float*)(rowl + n_iter * 1024))[blk];
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r][c] += (d[r] * d8) * (float)dot16(q[r], a, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < B; ++c) {
                const float total = wave_sum(acc[r][c]);
                if (lane == 0 && row0 + r < n) store_out(dst, stride_col_dst, c, row0 + r, total, bias);
            }
    }
}

// --------------------------------------------------------------------------------------------
// Sub-block-dot probe: one wave per (row, pass), activation read straight from global memory.
// --------------------------------------------------------------------------------------------
static __device__ __forceinline__ void load_act16(const uint8_t* vy, int q81_block, int lh, uint4& a) {
    const uint32_t* src = (const uint32_t*)(vy + (size_t)q81_block * Q81_BYTES) + 1 + 4 * lh;
    a = make_uint4(src[0], src[1], src[2], src[3]);
}

__global__ __launch_bounds__(64) void subdots_q4k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7, p = ch >> 1, lh = ch & 1;
    int d_lo = 0, d_hi = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q4K_BYTES;
        const uint4 q = *(const uint4*)(bp + 16 + 16 * ch);
        uint4 a_lo, a_hi;
        load_act16(vy, blk * 8 + 2 * p, lh, a_lo);
        load_act16(vy, blk * 8 + 2 * p + 1, lh, a_hi);
        q4k_dots(q, a_lo, a_hi, d_lo, d_hi);
    }
    d_lo += __shfl_xor(d_lo, 1);
    d_hi += __shfl_xor(d_hi, 1);
    if (blk < nb && lh == 0) {
        int32_t* out = dots + (size_t)row * nb * 8 + blk * 8 + 2 * p;
        out[0] = d_lo;
        out[1] = d_hi;
    }
}

__global__ __launch_bounds__(64) void subdots_q6k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7;
    const int h = ch >> 2, g0 = (ch >> 1) & 1, lh = ch & 1;
    if (blk >= nb) return;
    const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q6K_BYTES;
    const uint4 ql = *(const uint4_a2*)(bp + 16 * ch);
    const uint4 qh = *(const uint4_a2*)(bp + 128 + 16 * (2 * h + lh));
    uint4 a_a, a_b;
    load_act16(vy, blk * 8 + 4 * h + g0, lh, a_a);
    load_act16(vy, blk * 8 + 4 * h + g0 + 2, lh, a_b);
    int d_a, d_b;
    q6k_dots(ql, qh, g0, a_a, a_b, d_a, d_b);
    int32_t* out = dots + (size_t)row * nb * 16 + blk * 16;
    out[8 * h + 2 * g0 + lh] = d_a;
    out[8 * h + 2 * (g0 + 2) + lh] = d_b;
}

__global__ __launch_bounds__(64) void subdots_q80_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 32 + (lane >> 1), lh = lane & 1;
    int d = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q80_BYTES;
        const uint4 q = *(const uint4_a2*)(bp + 2 + 16 * lh);
        uint4 a;
        load_act16(vy, blk, lh, a);
        d = dot16(q, a, 0);
    }
    d += __shfl_xor(d, 1);
    if (blk < nb && lh == 0) dots[(size_t)row * nb + blk] = d;
}

__global__ void act_sums_kernel(const uint8_t* __restrict__ vy, int32_t* __restrict__ sums, int k32) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= k32) return;
    uint4 lo, hi;
    load_act16(vy, j, 0, lo);
    load_act16(vy, j, 1, hi);
    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
    sums[j] = dot16(ones, hi, dot16(ones, lo, 0));
}

// --------------------------------------------------------------------------------------------
// Host dispatch
// --------------------------------------------------------------------------------------------
struct MmvqArgs {
    const uint8_t* vx;
    const uint8_t* vy;
    void* dst;
    int nb, n, stride_col_y, stride_col_dst;
    const float* bias;
    hipStream_t stream;
};

template <class F>
static int n_iter_of(int nb) {
    const int per = F::VPI / F::BLOCK_LEN;
    return (nb + per - 1) / per;
}

// Launch geometry. `R` rows per wave and the number of resident workgroups per CU set how many
// bytes are in flight; both have measured optima well below "as many as fit" (HBM throughput
// drops when too many requests are outstanding). LK_TUNE_R / LK_TUNE_WGS_PER_CU override the
// built-in choice for measurement runs.
static int tune_env(const char* name) {
    const char* v = getenv(name);
    return v ? atoi(v) : 0;
}

template <class FMT, int B, int R, typename T, typename K>
static int launch_rows(K kernel, const MmvqArgs& a, int wgs_per_cu) {
    const int lds_bytes = B * lds_bytes_per_row<FMT>(n_iter_of<FMT>(a.nb));
    const LkDevice& dev = lk_device();
    if (lds_bytes > dev.lds_bytes) return LK_ERR_ARG;
    // Per kernel instance and LDS size: raise the dynamic-LDS limit once and ask the runtime how
    // many workgroups a CU holds. Cached, so steady-state launches (and launches recorded into a
    // graph) make no runtime query.
    static std::mutex mu;
    static std::unordered_map<int, int> resident_by_lds;
    int resident = 0;
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = resident_by_lds.find(lds_bytes);
        if (it == resident_by_lds.end()) {
            if (lds_bytes > 48 * 1024 &&
                hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
                (void)hipGetLastError();
                return LK_ERR_LAUNCH;
            }
            int r = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)kernel, WG, (size_t)lds_bytes) != hipSuccess || r < 1) {
                (void)hipGetLastError();
                r = 1;
            }
            it = resident_by_lds.emplace(lds_bytes, r).first;
        }
        resident = it->second;
    }
    const int tiles = (a.n + R - 1) / R;
    const int wgs_needed = (tiles + WAVES - 1) / WAVES;
    // Persistent grid: exactly as many workgroups as are resident at once, so no workgroup waits
    // for a slot and each wave walks several row tiles.
    static const int forced = tune_env("LK_TUNE_WGS_PER_CU");
    const int cap = forced > 0 ? forced : wgs_per_cu;
    const int per_cu = resident > cap ? cap : resident;
    const int grid = wgs_needed < dev.cus * per_cu ? wgs_needed : dev.cus * per_cu;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(WG), lds_bytes, a.stream, a.vx, a.vy, (T*)a.dst, a.nb,
                       a.n, a.stride_col_y, a.stride_col_dst, a.bias);
    return lk_launch_status();
}

#define LK_DEFINE_LAUNCHER(NAME, KERNEL, FMT, ROWS1, ROWSN, WGS_PER_CU)                                \
    template <int B, typename T>                                                                      \
    static int NAME(const MmvqArgs& a) {                                                              \
        static const int forced_r = tune_env("LK_TUNE_R");                                            \
        if (B == 1 && forced_r == 1) return launch_rows<FMT, B, 1, T>(KERNEL<B, 1, T>, a, WGS_PER_CU); \
        if (B == 1 && forced_r == 2) return launch_rows<FMT, B, 2, T>(KERNEL<B, 2, T>, a, WGS_PER_CU); \
        if (B == 1 && forced_r == 4) return launch_rows<FMT, B, 4, T>(KERNEL<B, 4, T>, a, WGS_PER_CU); \
        constexpr int R = (B == 1) ? ROWS1 : ROWSN;                                                   \
        return launch_rows<FMT, B, R, T>(KERNEL<B, R, T>, a, WGS_PER_CU);                             \
    }

LK_DEFINE_LAUNCHER(launch_q4k, mmvq_q4k_kernel, FmtQ4K, 2, 2, 8)
LK_DEFINE_LAUNCHER(launch_q6k, mmvq_q6k_kernel, FmtQ6K, 2, 2, 8)
LK_DEFINE_LAUNCHER(launch_q80, mmvq_q80_kernel, FmtQ80, 2, 2, 8)

#define LK_BATCH_SWITCH(FN, T)                                                                         \
    switch (batch) {                                                                                  \
        case 1: return FN<1, T>(a);                                                                   \
        case 2: return FN<2, T>(a);                                                                   \
        case 3: return FN<3, T>(a);                                                                   \
        case 4: return FN<4, T>(a);                                                                   \
        case 5: return FN<5, T>(a);                                                                   \
        case 6: return FN<6, T>(a);                                                                   \
        case 7: return FN<7, T>(a);                                                                   \
        case 8: return FN<8, T>(a);                                                                   \
        default: return LK_ERR_ARG;                                                                   \
    }

template <typename T>
static int dispatch_type(int wtype, int batch, const MmvqArgs& a) {
    switch (wtype) {
        case LK_TYPE_Q4_K: LK_BATCH_SWITCH(launch_q4k, T)
        case LK_TYPE_Q6_K: LK_BATCH_SWITCH(launch_q6k, T)
        case LK_TYPE_Q8_0: LK_BATCH_SWITCH(launch_q80, T)
        default: return LK_ERR_TYPE;
    }
}

static int block_len_of(int wtype) {
    switch (wtype) {
        case LK_TYPE_Q4_K: case LK_TYPE_Q6_K: return 256;
        case LK_TYPE_Q8_0: return 32;
        default: return 0;
    }
}

}  // namespace

extern "C" int lk_mmvq(int wtype, const void* vx, const void* vy_q8_1, void* dst, int dst_type,
                       int ncols_x, int nrows_x, int batch, int stride_col_y, int stride_col_dst,
                       const float* bias, int decode_order, void* stream) {
    (void)decode_order;  // a row's sum never depends on batch here
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (nrows_x == 0) return LK_OK;
    if (!vx || !vy_q8_1 || !dst || ncols_x <= 0 || nrows_x < 0 || ncols_x % bl != 0) return LK_ERR_ARG;
    if (batch < 1 || batch > 8 || stride_col_y < ncols_x / 32 || stride_col_dst < nrows_x) return LK_ERR_ARG;
    if (((uintptr_t)vy_q8_1 & 3) != 0) return LK_ERR_ARG;
    if (wtype == LK_TYPE_Q4_K && ((uintptr_t)vx & 15) != 0) return LK_ERR_ARG;
    if (((uintptr_t)vx & 1) != 0) return LK_ERR_ARG;
    MmvqArgs a{(const uint8_t*)vx, (const uint8_t*)vy_q8_1, dst, ncols_x / bl, nrows_x,
               stride_col_y, stride_col_dst, bias, (hipStream_t)stream};
    switch (dst_type) {
        case LK_TYPE_F32: return dispatch_type<float>(wtype, batch, a);
        case LK_TYPE_F16: return dispatch_type<__half>(wtype, batch, a);
        case LK_TYPE_BF16: return dispatch_type<__hip_bfloat16>(wtype, batch, a);
        default: return LK_ERR_TYPE;
    }
}

extern "C" int lk_mmvq_subdots(int wtype, const void* vx, const void* vy_q8_1, int32_t* dots,
                               int32_t* sums, int ncols_x, int nrows_x, void* stream) {
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (!vx || !vy_q8_1 || !dots || ncols_x <= 0 || nrows_x <= 0 || ncols_x % bl != 0) return LK_ERR_ARG;
    if (nrows_x > 65535) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int nb = ncols_x / bl;
    const uint8_t* w = (const uint8_t*)vx;
    const uint8_t* y = (const uint8_t*)vy_q8_1;
    if (wtype == LK_TYPE_Q4_K) {
        hipLaunchKernelGGL(subdots_q4k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else if (wtype == LK_TYPE_Q6_K) {
        hipLaunchKernelGGL(subdots_q6k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else {
        hipLaunchKernelGGL(subdots_q80_kernel, dim3((nb + 31) / 32, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    }
    if (sums) {
        const int k32 = ncols_x / 32;
        hipLaunchKernelGGL(act_sums_kernel, dim3((k32 + 255) / 256), dim3(256), 0, s, y, sums, k32);
    }
    return lk_launch_status();
}

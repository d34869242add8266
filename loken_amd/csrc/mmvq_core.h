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

// The same with the high nibbles left in place: a byte of (q & 0xF0) ^ 0x80, read as signed, is
// 16 * nibble - 128, so the dot product with the activation codes is 16 * d_hi - 128 * sum(codes).
// The caller starts `x_hi` at 128 * (sum of the sub-block's activation codes) and receives
// 16 * d_hi exactly; the mask and the flip are one three-operand bit instruction per dword where
// the shift and mask of q4k_dots are two.
static __device__ __forceinline__ void q4k_dots_biased(const uint4& q, const uint4& a_lo, const uint4& a_hi,
                                                       uint32_t flip, int& d_lo, int& x_hi) {
    uint4 lo, hx;
    lo.x = q.x & 0x0F0F0F0Fu; hx.x = (q.x & 0xF0F0F0F0u) ^ flip;
    lo.y = q.y & 0x0F0F0F0Fu; hx.y = (q.y & 0xF0F0F0F0u) ^ flip;
    lo.z = q.z & 0x0F0F0F0Fu; hx.z = (q.z & 0xF0F0F0F0u) ^ flip;
    lo.w = q.w & 0x0F0F0F0Fu; hx.w = (q.w & 0xF0F0F0F0u) ^ flip;
    d_lo = dot16(lo, a_lo, d_lo);
    x_hi = dot16(hx, a_hi, x_hi);
}

// A lane's share of a Q4_K row from one pair of sub-blocks (2p: low nibbles, 2p + 1: high):
//   d * (scl * d8a * d_lo + sch * d8b * d_hi) - dmin * (ml * sa + mh * sb),  sa = d8a * sum(codes of 2p), sb likewise.
// Every engine forms it here, with the roundings written out, so that a row carries the same
// bits whichever engine served it. `d8b` and `d_hi` may arrive as d8b / 16 and 16 * d_hi
// (q4k_dots_biased): powers of two move through the roundings unchanged.
static __device__ __forceinline__ float q4k_pair_share(float d, float dmin, float scl, float sch, float ml, float mh,
                                                       float d8a, float d8b, float sa, float sb, float d_lo, float d_hi) {
#pragma clang fp contract(off)
    const float ka = scl * d8a, kb = sch * d8b;
    const float hi = kb * d_hi, mb = mh * sb;
    const float u = __builtin_fmaf(ka, d_lo, hi);
    const float w = __builtin_fmaf(ml, sa, mb);
    const float off = dmin * w;
    return __builtin_fmaf(d, u, -off);
}

// Q5_K: the same 16 bytes of qs plus the 16 bytes of qh over the same l; bit 2p of a qh byte is
// the fifth bit (worth 16) of that value in sub-block 2p, bit 2p+1 in sub-block 2p+1
// (src/tensor/quant_cpu/format/q5_k.rs:66-71). `hs` arrives already shifted right by 2p.
static __device__ __forceinline__ void q5k_dots(const uint4& q, const uint4& hs, const uint4& a_lo, const uint4& a_hi,
                                                int& d_lo, int& d_hi) {
    uint4 lo, hi;
    lo.x = (q.x & 0x0F0F0F0Fu) | ((hs.x << 4) & 0x10101010u); hi.x = ((q.x >> 4) & 0x0F0F0F0Fu) | ((hs.x << 3) & 0x10101010u);
    lo.y = (q.y & 0x0F0F0F0Fu) | ((hs.y << 4) & 0x10101010u); hi.y = ((q.y >> 4) & 0x0F0F0F0Fu) | ((hs.y << 3) & 0x10101010u);
    lo.z = (q.z & 0x0F0F0F0Fu) | ((hs.z << 4) & 0x10101010u); hi.z = ((q.z >> 4) & 0x0F0F0F0Fu) | ((hs.z << 3) & 0x10101010u);
    lo.w = (q.w & 0x0F0F0F0Fu) | ((hs.w << 4) & 0x10101010u); hi.w = ((q.w >> 4) & 0x0F0F0F0Fu) | ((hs.w << 3) & 0x10101010u);
    d_lo = dot16(lo, a_lo, d_lo);
    d_hi = dot16(hi, a_hi, d_hi);
}
static __device__ __forceinline__ uint4 shr4(const uint4& v, int s) {
    return make_uint4(v.x >> s, v.y >> s, v.z >> s, v.w >> s);
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

// Q6_K with the codes left unsigned (0..63): 16 bytes of each half-row of ql (`ql0` = l, `ql1` =
// l + 32) and the 16 bytes of qh over the same l give 16 codes of each of the half's four
// 32-value groups. The caller starts each accumulator at -32 * (sum of that run's activation
// codes), which yields the integer the signed form gives.
static __device__ __forceinline__ void q6k_dots_biased(const uint4& ql0, const uint4& ql1, const uint4& qh,
                                                       const uint4 (&a)[4], int (&dot)[4]) {
    uint4 c[4];
#define LK_Q6K_RAW(f)                                                       \
    c[0].f = (ql0.f & 0x0F0F0F0Fu) | ((qh.f << 4) & 0x30303030u);             \
    c[1].f = (ql1.f & 0x0F0F0F0Fu) | ((qh.f << 2) & 0x30303030u);             \
    c[2].f = ((ql0.f >> 4) & 0x0F0F0F0Fu) | (qh.f & 0x30303030u);             \
    c[3].f = ((ql1.f >> 4) & 0x0F0F0F0Fu) | ((qh.f >> 2) & 0x30303030u);
    LK_Q6K_RAW(x) LK_Q6K_RAW(y) LK_Q6K_RAW(z) LK_Q6K_RAW(w)
#undef LK_Q6K_RAW
#pragma unroll
    for (int g = 0; g < 4; ++g) dot[g] = dot16(c[g], a[g], dot[g]);
}

// Q6_K: the scales of the four groups of a half (`sc`: the half's 8 scale bytes) for run `lh` (0: the
// groups' first 16 values, 1: their last 16), times the super-block's d.
static __device__ __forceinline__ void q6k_run_scales(float d, const uint2& sc, int lh, float (&ds)[4]) {
    ds[0] = d * (float)(int)__builtin_amdgcn_sbfe(sc.x, 8 * lh, 8);
    ds[1] = d * (float)(int)__builtin_amdgcn_sbfe(sc.x, 8 * lh + 16, 8);
    ds[2] = d * (float)(int)__builtin_amdgcn_sbfe(sc.y, 8 * lh, 8);
    ds[3] = d * (float)(int)__builtin_amdgcn_sbfe(sc.y, 8 * lh + 16, 8);
}
// A lane's share of a Q6_K row from its runs of the four groups, added to `acc`. Every kernel that
// must give a row the same bits forms the share here.
static __device__ __forceinline__ void q6k_half_share(float& acc, const float (&ds)[4], const float4& d8,
                                                      const int (&dot)[4]) {
    acc += ds[0] * (d8.x * (float)dot[0]) + ds[2] * (d8.z * (float)dot[2]);
    acc += ds[1] * (d8.y * (float)dot[1]) + ds[3] * (d8.w * (float)dot[3]);
}

// --------------------------------------------------------------------------------------------
// Activation staging. Formats differ only in where a Q8_1 block's two 16-byte halves land.
// LDS per activation row: `n_iter` passes x `PLANES` planes x 1024 bytes of codes, then the
// scale table, SCF dwords per Q8_1 block: d; with SCF 2 also d * (sum of the block's codes),
// interleaved; with SCF 3 three arrays one after the other: d, then -32 * (sum of codes) of every
// block's first 16 values, then of its last 16, as integers.
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
// Q5_K stages its activation as Q4_K does: the two formats share sub-blocks, scales and mins.
struct FmtQ5K : FmtQ4K {
    static constexpr int BLOCK_BYTES = Q5K_BYTES;
};
struct FmtQ6K {
    static constexpr int BLOCK_BYTES = Q6K_BYTES, BLOCK_LEN = 256;
    static constexpr int VPI = 4096;   // 16 super-blocks per wave pass, 4 lanes each
    static constexpr int PLANES = 4, SCF = 3;
    // Lane (block lb, half h, 16-run lh) reads plane g (the 32-value group inside the half) at lane * 16.
    static __device__ __forceinline__ int slot(int j, int lh) {
        const int lb = j >> 3, s = j & 7, h = s >> 2, g = s & 3;
        return g * 1024 + (lb * 4 + h * 2 + lh) * 16;
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

// Staging runs in two halves so that an engine can put its first weight loads between them:
// `stage_issue` sends the loads of the first round of activation data (per thread: one Q8_1 block,
// or 16 floats) and `stage_finish` turns them into the LDS image and walks the later rounds.
// Loads return in issue order, so the activation (small, usually in L2) must be asked for BEFORE
// the weights (HBM) or the staging would wait for the weights as well. Only launches of up to
// two activation rows hoist the first round; wider ones would hold too many registers.
template <int B>
struct ActRegs {
    static constexpr int ROWS = B <= 2 ? B : 0;
    uint32_t head[ROWS ? ROWS : 1];   // a Q8_1 block: d and s, then the two halves of its codes
    uint4 lo[ROWS ? ROWS : 1], hi[ROWS ? ROWS : 1];
    float4 x[ROWS ? ROWS : 1][4];
};

// One Q8_1 block (j-th of its row; `real` false past the row's end) into the LDS image of `row`.
template <class F>
static __device__ __forceinline__ void put_q8_1_block(uint8_t* row, int n_iter, int j, bool real, uint32_t head,
                                                      uint4 lo, uint4 hi) {
    const int per_pass = F::VPI / 32, total = n_iter * per_pass;
    const int it = j / per_pass, ji = j % per_pass;
    float* sc = (float*)(row + n_iter * F::VPI);
    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
    if (!real) {
        lo = hi = make_uint4(0, 0, 0, 0);
        head = 0;
    }
    const float d8 = f16_bits_to_f32(head & 0xFFFFu);
    uint8_t* codes = row + it * F::PLANES * 1024;
    *(uint4*)(codes + F::slot(ji, 0)) = lo;
    *(uint4*)(codes + F::slot(ji, 1)) = hi;
    if (F::SCF == 2) {
        *(float2*)(sc + 2 * j) = make_float2(d8, d8 * (float)dot16(ones, hi, dot16(ones, lo, 0)));
    } else if (F::SCF == 3) {
        sc[j] = d8;
        ((int*)sc)[total + j] = -32 * dot16(ones, lo, 0);
        ((int*)sc)[2 * total + j] = -32 * dot16(ones, hi, 0);
    } else {
        sc[j] = d8;
    }
}

// A Q8_1 block as three loads that land where they are used (36-byte blocks are dword aligned).
static __device__ __forceinline__ void load_q8_1_block(const uint8_t* __restrict__ p, uint32_t& head, uint4& lo,
                                                       uint4& hi) {
    // The two offsets pass through an opaque statement: seen as p + 4 and p + 20 the compiler
    // fuses the loads into 16 + 16 + 4 bytes from p and then has to wait for them on the spot to
    // shuffle the registers back into `lo` and `hi`.
    int off_lo = 4, off_hi = 20;
    asm("" : "+v"(off_lo));
    asm("" : "+v"(off_hi));
    head = *(const uint32_t*)p;
    lo = *(const uint4_a4*)(p + off_lo);
    hi = *(const uint4_a4*)(p + off_hi);
}

// Every thread loads (a thread past the row's end re-reads its last block and drops it later):
// a load under a branch would make the wave wait for it where the branch ends.
template <class F, int B>
static __device__ __forceinline__ void stage_issue_q8_1(ActRegs<B>& ar, const uint8_t* __restrict__ vy, int k32,
                                                        int stride_col_y) {
    const int j = min((int)threadIdx.x, k32 - 1);
#pragma unroll
    for (int c = 0; c < ActRegs<B>::ROWS; ++c)
        load_q8_1_block(vy + ((size_t)c * stride_col_y + j) * Q81_BYTES, ar.head[c], ar.lo[c], ar.hi[c]);
}

// Stage `batch` Q8_1 rows. k32 = real Q8_1 blocks per row; the rest of the last pass is zeroed.
template <class F, int B>
static __device__ __forceinline__ void stage_finish_q8_1(const ActRegs<B>& ar, uint8_t* lds,
                                                         const uint8_t* __restrict__ vy, int k32, int n_iter,
                                                         int stride_col_y) {
    const int total = n_iter * (F::VPI / 32);
    const int row_bytes = lds_bytes_per_row<F>(n_iter);
    int j = threadIdx.x;
    if (ActRegs<B>::ROWS) {
        if (j < total) {
#pragma unroll
            for (int c = 0; c < ActRegs<B>::ROWS; ++c)
                put_q8_1_block<F>(lds + c * row_bytes, n_iter, j, j < k32, ar.head[c], ar.lo[c], ar.hi[c]);
        }
        j += WG;
    }
    for (; j < total; j += WG) {
#pragma unroll
        for (int c = 0; c < B; ++c) {
            uint32_t head;
            uint4 lo, hi;
            load_q8_1_block(vy + ((size_t)c * stride_col_y + min(j, k32 - 1)) * Q81_BYTES, head, lo, hi);
            put_q8_1_block<F>(lds + c * row_bytes, n_iter, j, j < k32, head, lo, hi);
        }
    }
}

// The same staging from f32 rows: the workgroup quantizes each 32-value block itself, with the
// steps of the stand-alone quantizer (d = amax/127 rounded to f16, codes = round_half_away(x *
// (1/d)) with d before its rounding, integer code sum), so the staged bytes are the ones the
// two-launch path stages. Eight lanes own a block, four values each; item t is lane t & 7 of
// block t >> 3. All eight lanes of a block call this together.
template <class F>
static __device__ __forceinline__ void put_f32_quad(uint8_t* row, int n_iter, int k32, int t, float4 v) {
#pragma clang fp contract(off)
    const int per_pass = F::VPI / 32, total = n_iter * per_pass;
    const int j = t >> 3, l8 = t & 7;
    if (j >= k32) v = make_float4(0.f, 0.f, 0.f, 0.f);   // padding of the last pass
    const int it = j / per_pass, ji = j % per_pass;
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = max8(amax);
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const int q0 = (int)roundf(v.x * inv), q1 = (int)roundf(v.y * inv);
    const int q2 = (int)roundf(v.z * inv), q3 = (int)roundf(v.w * inv);
    int half_sum;   // lanes 0-3: the block's first 16 values, 4-7: the rest
    const int sum = sum8(q0 + q1 + q2 + q3, half_sum);
    uint8_t* codes = row + it * F::PLANES * 1024;
    *(uint32_t*)(codes + F::slot(ji, l8 >> 2) + 4 * (l8 & 3)) =
        (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
        ((uint32_t)(q3 & 0xFF) << 24);
    float* sc = (float*)(row + n_iter * F::VPI);
    if (l8 == 0) {
        const float d8 = __half2float(__float2half_rn(d));
        if (F::SCF == 2) {
            *(float2*)(sc + 2 * j) = make_float2(d8, d8 * (float)sum);
        } else if (F::SCF == 3) {
            sc[j] = d8;
            ((int*)sc)[total + j] = -32 * half_sum;
        } else {
            sc[j] = d8;
        }
    }
    if (F::SCF == 3 && l8 == 4) ((int*)sc)[2 * total + j] = -32 * half_sum;
}

constexpr int F32_ROUND = 4;  // float4 loads a thread issues together: the lane exchanges would
                              // otherwise serialize one memory latency per 1024 values

template <class F, int B>
static __device__ __forceinline__ void load_f32_round(float4 (&v)[F32_ROUND], const float* __restrict__ x, int t0,
                                                      int items, int k32) {
#pragma unroll
    for (int u = 0; u < F32_ROUND; ++u) {
        // past the row's end: re-read its last quad (dropped by the caller), never a branch
        const int t = min(t0 + u * WG, k32 * 8 - 1);
        v[u] = *(const float4*)(x + (size_t)t * 4);
    }
}

template <class F, int B>
static __device__ __forceinline__ void stage_issue_f32(ActRegs<B>& ar, const float* __restrict__ x, int k32,
                                                       int n_iter, int x_stride) {
    const int items = n_iter * (F::VPI / 32) * 8;
#pragma unroll
    for (int c = 0; c < ActRegs<B>::ROWS; ++c) load_f32_round<F, B>(ar.x[c], x + (size_t)c * x_stride, threadIdx.x, items, k32);
}

template <class F, int B>
static __device__ __forceinline__ void stage_finish_f32(const ActRegs<B>& ar, uint8_t* lds, const float* __restrict__ x,
                                                        int k32, int n_iter, int x_stride) {
    const int items = n_iter * (F::VPI / 32) * 8;
    const int row_bytes = lds_bytes_per_row<F>(n_iter);
    int t0 = threadIdx.x;
    if (ActRegs<B>::ROWS) {
#pragma unroll
        for (int c = 0; c < ActRegs<B>::ROWS; ++c)
#pragma unroll
            for (int u = 0; u < F32_ROUND; ++u)
                if (t0 + u * WG < items) put_f32_quad<F>(lds + c * row_bytes, n_iter, k32, t0 + u * WG, ar.x[c][u]);
        t0 += WG * F32_ROUND;
    }
    for (; t0 < items; t0 += WG * F32_ROUND) {
#pragma unroll
        for (int c = 0; c < B; ++c) {
            float4 v[F32_ROUND];
            load_f32_round<F, B>(v, x + (size_t)c * x_stride, t0, items, k32);
#pragma unroll
            for (int u = 0; u < F32_ROUND; ++u)
                if (t0 + u * WG < items) put_f32_quad<F>(lds + c * row_bytes, n_iter, k32, t0 + u * WG, v[u]);
        }
    }
}

// What a workgroup computes: rows of `vx[0..NW)` against the B activation rows at `vy`.
template <int NW>
struct RowJob {
    gbytes_t vx[NW];
    const uint8_t* vy;
    int nb;            // format blocks per weight row
    int n;             // weight rows
    int stride_col_y;  // Q8_1 blocks between activation rows
    int tile_stride;   // row tiles between a wave's consecutive tiles
    int tile_first;    // first row tile of wave 0 of this workgroup
    int act_stride_f32 = 0;  // non-zero: `vy` holds f32 activation rows this many floats apart,
                             // quantized to Q8_1 by the workgroup itself while staging
    // A wave's tiles: it starts at tile_first + wave * wave_stride, walks run_len consecutive tiles
    // (a power of two; the run starts on a multiple of it) and then jumps tile_stride from the
    // run's last tile. The defaults give the plain round-robin tile, tile + tile_stride, ...
    int wave_stride = 1;
    int run_len = 1;
};

template <int NW>
static __device__ __forceinline__ int next_tile(const RowJob<NW>& job, int t) {
    return (job.run_len > 1 && ((t + 1) & (job.run_len - 1))) ? t + 1 : t + job.tile_stride;
}

struct NoTileHook {
    __device__ __forceinline__ void operator()(int) const {}
};

// Keeps the loads written before it ahead of the loads written after it in the instruction
// stream. Without it the compiler is free to sink an activation load towards its first use,
// which lies past the weight loads, and loads return in issue order.
static __device__ __forceinline__ void load_fence(const void* p) {
    asm volatile("" : : "s"(p) : "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// The activation as the engines stage it, whichever form it arrives in, with `mid` (the engine's
// first weight loads) between the two halves. Each form runs `mid` in its own branch: merged
// after the branch, the wait for the activation data could no longer tell how many loads are
// ahead of the weights and would wait for part of them too.
template <class F, int B, int NW, class Mid>
static __device__ __forceinline__ void stage_around(uint8_t* lds, const RowJob<NW>& job, int k32, int n_iter, Mid&& mid) {
    ActRegs<B> ar;
    if (job.act_stride_f32) {
        stage_issue_f32<F, B>(ar, (const float*)job.vy, k32, n_iter, job.act_stride_f32);
        load_fence(job.vy);
        mid();
        load_fence(job.vy);
        stage_finish_f32<F, B>(ar, lds, (const float*)job.vy, k32, n_iter, job.act_stride_f32);
    } else {
        stage_issue_q8_1<F, B>(ar, job.vy, k32, job.stride_col_y);
        load_fence(job.vy);
        mid();
        load_fence(job.vy);
        stage_finish_q8_1<F, B>(ar, lds, job.vy, k32, n_iter, job.stride_col_y);
    }
}

// ---------------------------------------------------------------------------------------------
// Q4_K: 4 lanes per super-block (32 bytes of qs each = two whole sub-blocks), 16 super-blocks
// per wave pass, loads of the next step in flight while the current one is consumed.
// epi(row, col, totals[NW]) runs on lane 0 for every finished (row, activation row).
// ---------------------------------------------------------------------------------------------
// Short rows: a pass has 16 super-block slots of 4 lanes; a row of at most 8 (4) super-blocks
// would leave half (three quarters) of the lanes idle, so 2 (4) rows share a pass, each in its
// own 32 (16) lanes. The MoE expert matrices (k = 2048, 768) and small dense models live here.
static __host__ __device__ __forceinline__ int q4k_rows_per_pass(int nb) { return nb <= 4 ? 4 : nb <= 8 ? 2 : 1; }

// Totals of the four rows of 16 lanes, every lane returns all four.
static __device__ __forceinline__ void row16_sums(float v, float (&q)[4]) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    const int bits = __float_as_int(v);
    q[0] = __int_as_float(__builtin_amdgcn_readlane(bits, 0));
    q[1] = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    q[2] = __int_as_float(__builtin_amdgcn_readlane(bits, 32));
    q[3] = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
}

// done(tile) runs on every lane of the wave once the tile's rows have been handed to epi.
// PACK false: one row per pass, all of this a compile-time 1 / 16 (the long-row kernels pay
// nothing for the short-row form); PACK true: rows per pass from the row length.
template <int B, int R, int NW, bool PACK, bool Q5, class Epi, class Done>
static __device__ __forceinline__ void rows_q4k(const RowJob<NW>& job, uint8_t* lds, Epi&& epi, Done&& done) {
    // Q5_K: the Q4_K header, then 32 bytes of fifth bits, then the nibbles
    constexpr int BB = Q5 ? Q5K_BYTES : Q4K_BYTES, QS0 = Q5 ? 48 : 16;
    const int nb = job.nb, n = job.n;
    const int n_iter_lds = (nb + 15) >> 4;   // passes of the staged activation (its layout)
    const int row_bytes = lds_bytes_per_row<FmtQ4K>(n_iter_lds);
    // rows side by side in a pass (tile runs keep the plain form)
    const int RP = (!PACK || job.run_len > 1) ? 1 : q4k_rows_per_pass(nb);
    const int S = PACK ? 16 / RP : 16;       // super-block slots of one row in a pass
    const int n_iter = (nb + S - 1) / S;     // passes per tile (1 whenever RP > 1)
    const int TR = R * RP;                   // rows per tile

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lb = lane >> 2, p = lane & 3;
    const int slot = lb & (S - 1), rp = lb / S;
    const Q4KScaleSel sel(p);
    const uint32_t hdr_off = slot * BB, qs_off = hdr_off + QS0 + 32 * p;
    const size_t row_stride = (size_t)nb * BB;
    const int n_tiles = (n + TR - 1) / TR;
    constexpr int RW = R * NW;

    struct Frag {
        uint4 hdr[RW], q0[RW], q1[RW];
        uint4 h0[Q5 ? RW : 1], h1[Q5 ? RW : 1];   // Q5_K: qh over l 0..15 and 16..31 (every pair's lane reads both)
    };
    // One pass (16 super-block slots) of R rows per lane group of every matrix into registers. A
    // lane past the row end re-reads the row's last block and drops its d / dmin when it consumes
    // it, so it adds nothing (the loaded registers themselves are left alone: touching them here
    // would make the wave wait for the load).
    auto load = [&](Frag& f, int tile, int it) {
        const bool valid = it * S + slot < nb;
        const uint32_t back = valid ? 0u : (uint32_t)(it * S + slot - (nb - 1)) * BB;
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = min(tile * TR + rp * R + r, n - 1);
                const uint8_t* bp = (const uint8_t*)(job.vx[w] + row * row_stride + (size_t)it * (S * BB));
                Frag& g = f;
                g.hdr[w * R + r] = *(const uint4*)(bp + (hdr_off - back));
                g.q0[w * R + r] = *(const uint4*)(bp + (qs_off - back));
                g.q1[w * R + r] = *(const uint4*)(bp + (qs_off - back + 16));
                if (Q5) {
                    g.h0[w * R + r] = *(const uint4*)(bp + (hdr_off - back + 16));
                    g.h1[w * R + r] = *(const uint4*)(bp + (hdr_off - back + 32));
                }
            }
    };

    float acc[RW][B];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

    auto compute = [&](const Frag& f, int tile, int it) {
        const int block = it * S + slot;   // the lane's super-block of its row
        float d[RW], dmin[RW], scl[RW], sch[RW], ml[RW], mh[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            uint32_t sc, mn;
            sel.unpack(f.hdr[r].y, f.hdr[r].z, f.hdr[r].w, sc, mn);
            const uint32_t dd = block < nb ? f.hdr[r].x : 0u;
            d[r] = f16_bits_to_f32(dd & 0xFFFFu);
            dmin[r] = f16_bits_to_f32(dd >> 16);
            scl[r] = (float)(sc & 0xFFu);
            sch[r] = (float)(sc >> 8);
            ml[r] = (float)(mn & 0xFFu);
            mh[r] = (float)(mn >> 8);
        }
#pragma unroll
        for (int c = 0; c < B; ++c) {
            const uint8_t* rowl = lds + c * row_bytes;
            const uint8_t* codes = rowl + (block >> 4) * 4096 + ((block & 15) * 4 + p) * 16;
            const uint4 a00 = *(const uint4*)(codes);
            const uint4 a01 = *(const uint4*)(codes + 1024);
            const uint4 a10 = *(const uint4*)(codes + 2048);
            const uint4 a11 = *(const uint4*)(codes + 3072);
            const float4 s4 = *(const float4*)(rowl + n_iter_lds * 4096 + (size_t)(block * 8 + 2 * p) * 8);
#pragma unroll
            for (int r = 0; r < RW; ++r) {
                int d_lo = 0, d_hi = 0;
                if (Q5) {
                    q5k_dots(f.q0[r], shr4(f.h0[r], 2 * p), a00, a10, d_lo, d_hi);
                    q5k_dots(f.q1[r], shr4(f.h1[r], 2 * p), a01, a11, d_lo, d_hi);
                } else {
                    q4k_dots(f.q0[r], a00, a10, d_lo, d_hi);
                    q4k_dots(f.q1[r], a01, a11, d_lo, d_hi);
                }
                acc[r][c] += q4k_pair_share(d[r], dmin[r], scl[r], sch[r], ml[r], mh[r], s4.x, s4.z, s4.y,
                                            s4.w, (float)d_lo, (float)d_hi);
            }
        }
        if (it == n_iter - 1) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int c = 0; c < B; ++c) {
                    float q[NW][4];
#pragma unroll
                    for (int w = 0; w < NW; ++w) {
                        row16_sums(acc[w * R + r][c], q[w]);
                        acc[w * R + r][c] = 0.f;
                    }
                    if (lane == 0) {
                        float tot[NW];
                        const int row0 = tile * TR + r;
                        if (RP == 1) {
#pragma unroll
                            for (int w = 0; w < NW; ++w) tot[w] = (q[w][0] + q[w][1]) + (q[w][2] + q[w][3]);
                            if (row0 < n) epi(row0, c, tot);
                        } else if (RP == 2) {
#pragma unroll
                            for (int g = 0; g < 2; ++g) {
#pragma unroll
                                for (int w = 0; w < NW; ++w) tot[w] = q[w][2 * g] + q[w][2 * g + 1];
                                if (row0 + g * R < n) epi(row0 + g * R, c, tot);
                            }
                        } else {
#pragma unroll
                            for (int g = 0; g < 4; ++g) {
#pragma unroll
                                for (int w = 0; w < NW; ++w) tot[w] = q[w][g];
                                if (row0 + g * R < n) epi(row0 + g * R, c, tot);
                            }
                        }
                    }
                }
            done(tile);
        }
    };

    // The first weight loads go out between the two halves of the staging, so the two memory
    // latencies overlap instead of adding up (most of a small matrix's run time).
    int tile = job.tile_first + wave * job.wave_stride, it = 0;
    Frag fa, fb;
    // (a wave without a tile loads the last one rather than nothing: a load under a branch would
    // blur the count of loads ahead of the weights and the staging would wait for some of them)
    stage_around<FmtQ4K, B>(lds, job, nb * 8, n_iter_lds, [&] { load(fa, min(tile, n_tiles - 1), 0); });
    __syncthreads();
    if (tile >= n_tiles) return;
    // Steps are (tile, pass) pairs in order; the loads of step i+1 are issued before step i is
    // consumed, ping-ponging between two register fragments.
    for (;;) {
        int nt = tile, ni = it + 1;
        if (ni == n_iter) { ni = 0; nt = next_tile(job, nt); }
        if (nt < n_tiles) load(fb, nt, ni);
        compute(fa, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
        nt = tile; ni = it + 1;
        if (ni == n_iter) { ni = 0; nt = next_tile(job, nt); }
        if (nt < n_tiles) load(fa, nt, ni);
        compute(fb, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
    }
}

// ---------------------------------------------------------------------------------------------
// The step loop the Q6_K and Q8_0 engines share. Steps are (row tile, pass) pairs in order; the
// loads of step i+1 are issued before step i is consumed, ping-ponging between two register
// fragments, and the very first loads go out between the two halves of the activation staging so
// that the two memory latencies overlap.
// ---------------------------------------------------------------------------------------------
template <class Frag, int NW, class Stage, class Load, class Compute>
static __device__ __forceinline__ void step_loop(const RowJob<NW>& job, int tile, int n_tiles, int n_iter, Stage&& stage,
                                                 Load&& load, Compute&& compute) {
    int it = 0;
    Frag fa, fb;
    // (a wave without a tile loads the last one rather than nothing: a load under a branch would
    // blur the count of loads ahead of the weights and the staging would wait for some of them)
    stage([&] { load(fa, min(tile, n_tiles - 1), 0); });
    __syncthreads();
    if (tile >= n_tiles) return;
    for (;;) {
        int nt = tile, ni = it + 1;
        if (ni == n_iter) { ni = 0; nt = next_tile(job, nt); }
        if (nt < n_tiles) load(fb, nt, ni);
        compute(fa, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
        nt = tile; ni = it + 1;
        if (ni == n_iter) { ni = 0; nt = next_tile(job, nt); }
        if (nt < n_tiles) load(fa, nt, ni);
        compute(fb, tile, it);
        tile = nt; it = ni;
        if (tile >= n_tiles) break;
    }
}

// ---------------------------------------------------------------------------------------------
// Q6_K: 4 lanes per super-block, 16 super-blocks per wave pass. Lane (half h, run lh) takes the
// 16 bytes of both ql half-rows and the 16 bytes of qh at l = 16 * lh, which is 16 codes of each
// of the half's four groups and reads no byte of ql / qh twice across the wave (the load unit's
// cycles, not HBM, bound this format). The codes stay unsigned; the -32 offset comes in through
// the staged per-run activation sums.
// ---------------------------------------------------------------------------------------------
// PACK: rows of at most 8 (4) super-blocks share a pass two (four) at a time, each in its own 32 (16)
// lanes, as the short Q4_K rows do.
template <int B, int R, int NW, bool PACK, class Epi, class Done>
static __device__ __forceinline__ void rows_q6k(const RowJob<NW>& job, uint8_t* lds, Epi&& epi, Done&& done) {
    const int nb = job.nb, n = job.n;
    const int n_iter_lds = (nb + 15) >> 4;   // passes of the staged activation (its layout)
    const int row_bytes = lds_bytes_per_row<FmtQ6K>(n_iter_lds);
    const int total = n_iter_lds * 128;   // Q8_1 blocks the staged row is padded to
    const int RP = (!PACK || job.run_len > 1) ? 1 : q4k_rows_per_pass(nb);
    const int S = PACK ? 16 / RP : 16;       // super-block slots of one row in a pass
    const int n_iter = (nb + S - 1) / S;     // passes per tile (1 whenever RP > 1)
    const int TR = R * RP;                   // rows per tile

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lb = lane >> 2, h = (lane >> 1) & 1, lh = lane & 1;
    const int slot = lb & (S - 1), rp = lb / S;
    const uint32_t ql_off = 64 * h + 16 * lh, qh_off = 128 + 32 * h + 16 * lh, sc_off = 192 + 8 * h;
    const size_t row_stride = (size_t)nb * Q6K_BYTES;
    const int n_tiles = (n + TR - 1) / TR;
    constexpr int RW = R * NW;

    struct Frag {
        uint4 ql0[RW], ql1[RW], qh[RW];
        uint2 sc[RW];     // the half's 8 scale bytes
        uint32_t d[RW];   // f16 bits
    };
    // A lane past the row end re-reads the row's last block and drops its d when it consumes it.
    auto load = [&](Frag& f, int tile, int it) {
        const int blk_c = min(it * S + slot, nb - 1);
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = min(tile * TR + rp * R + r, n - 1);
                const uint8_t* bp = (const uint8_t*)(job.vx[w] + row * row_stride + (size_t)blk_c * Q6K_BYTES);
                f.ql0[w * R + r] = *(const uint4_a2*)(bp + ql_off);
                f.ql1[w * R + r] = *(const uint4_a2*)(bp + ql_off + 32);
                f.qh[w * R + r] = *(const uint4_a2*)(bp + qh_off);
                f.sc[w * R + r] = *(const uint2_a2*)(bp + sc_off);
                f.d[w * R + r] = *(const uint16_t*)(bp + 208);
            }
    };

    float acc[RW][B];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

    auto compute = [&](const Frag& f, int tile, int it) {
        const int block = it * S + slot;   // the lane's super-block of its row
        float ds[RW][4];
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            const float d = block < nb ? f16_bits_to_f32(f.d[r]) : 0.f;
            q6k_run_scales(d, f.sc[r], lh, ds[r]);
        }
#pragma unroll
        for (int c = 0; c < B; ++c) {
            const uint8_t* rowl = lds + c * row_bytes;
            const int blk_l = min(block, n_iter_lds * 16 - 1);   // (a lane past a packed row's end: any staged block)
            const uint8_t* codes = rowl + (blk_l >> 4) * 4096 + ((blk_l & 15) * 4 + (lane & 3)) * 16;
            uint4 a[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) a[g] = *(const uint4*)(codes + g * 1024);
            const uint8_t* sc = rowl + n_iter_lds * 4096;
            const int j0 = blk_l * 8 + 4 * h;   // the half's four Q8_1 blocks
            const float4 d8 = *(const float4*)(sc + 4 * j0);
            const int4 bias = *(const int4*)(sc + 4 * (total * (1 + lh) + j0));
#pragma unroll
            for (int r = 0; r < RW; ++r) {
                int dot[4] = {bias.x, bias.y, bias.z, bias.w};
                q6k_dots_biased(f.ql0[r], f.ql1[r], f.qh[r], a, dot);
                q6k_half_share(acc[r][c], ds[r], d8, dot);
            }
        }
        if (it == n_iter - 1) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int c = 0; c < B; ++c) {
                    float tot[NW];
                    if (RP == 1) {
#pragma unroll
                        for (int w = 0; w < NW; ++w) {
                            tot[w] = wave_sum(acc[w * R + r][c]);
                            acc[w * R + r][c] = 0.f;
                        }
                        if (lane == 0 && tile * R + r < n) epi(tile * R + r, c, tot);
                    } else {
                        float q[NW][4];
#pragma unroll
                        for (int w = 0; w < NW; ++w) {
                            row16_sums(acc[w * R + r][c], q[w]);
                            acc[w * R + r][c] = 0.f;
                        }
                        if (lane == 0) {
                            const int row0 = tile * TR + r;
                            if (RP == 2) {
#pragma unroll
                                for (int g = 0; g < 2; ++g) {
#pragma unroll
                                    for (int w = 0; w < NW; ++w) tot[w] = q[w][2 * g] + q[w][2 * g + 1];
                                    if (row0 + g * R < n) epi(row0 + g * R, c, tot);
                                }
                            } else {
#pragma unroll
                                for (int g = 0; g < 4; ++g) {
#pragma unroll
                                    for (int w = 0; w < NW; ++w) tot[w] = q[w][g];
                                    if (row0 + g * R < n) epi(row0 + g * R, c, tot);
                                }
                            }
                        }
                    }
                }
            done(tile);
        }
    };
    step_loop<Frag>(job, job.tile_first + wave * job.wave_stride, n_tiles, n_iter,
                    [&](auto&& mid) { stage_around<FmtQ6K, B>(lds, job, nb * 8, n_iter_lds, mid); }, load, compute);
}

// ---------------------------------------------------------------------------------------------
// Q8_0: 2 lanes per 32-value block, 32 blocks per wave pass.
// ---------------------------------------------------------------------------------------------
template <int B, int R, int NW, class Epi, class Done>
static __device__ __forceinline__ void rows_q80(const RowJob<NW>& job, uint8_t* lds, Epi&& epi, Done&& done) {
    const int nb = job.nb, n = job.n;
    const int n_iter = (nb + 31) >> 5;
    const int row_bytes = lds_bytes_per_row<FmtQ80>(n_iter);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lb = lane >> 1, lh = lane & 1;
    const size_t row_stride = (size_t)nb * Q80_BYTES;
    const int n_tiles = (n + R - 1) / R;
    constexpr int RW = R * NW;

    struct Frag {
        Run16 q[RW];
        uint32_t d[RW];       // f16 bits
        uint32_t shift[RW];   // bits to shift q by
    };
    // A lane past the row end re-reads the row's last block and drops its d when it consumes it.
    auto load = [&](Frag& f, int tile, int it) {
        const int blk_c = min(it * 32 + lb, nb - 1);
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = min(tile * R + r, n - 1);
                const uint8_t* bp = (const uint8_t*)(job.vx[w] + row * row_stride + (size_t)blk_c * Q80_BYTES);
                f.q[w * R + r] = load_run16(bp + 2 + 16 * lh);
                f.shift[w * R + r] = ((uint32_t)(uintptr_t)(bp + 2) & 2u) * 8u;
                f.d[w * R + r] = *(const uint16_t*)bp;
            }
    };

    float acc[RW][B];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int c = 0; c < B; ++c) acc[r][c] = 0.f;

    auto compute = [&](const Frag& f, int tile, int it) {
        const int blk = it * 32 + lb;
        uint4 q[RW];
        float d[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            q[r] = run16_value(f.q[r], f.shift[r]);
            d[r] = blk < nb ? f16_bits_to_f32(f.d[r]) : 0.f;
        }
#pragma unroll
        for (int c = 0; c < B; ++c) {
            const uint8_t* rowl = lds + c * row_bytes;
            const uint4 a = *(const uint4*)(rowl + it * 1024 + lane * 16);
            const float d8 = ((const float*)(rowl + n_iter * 1024))[blk];
#pragma unroll
            for (int r = 0; r < RW; ++r) acc[r][c] += (d[r] * d8) * (float)dot16(q[r], a, 0);
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
            done(tile);
        }
    };
    step_loop<Frag>(job, job.tile_first + wave * job.wave_stride, n_tiles, n_iter,
                    [&](auto&& mid) { stage_around<FmtQ80, B>(lds, job, nb, n_iter, mid); }, load, compute);
}


// Format tags: which engine serves a ggml type, and its LDS footprint.
struct EngQ4K {
    using Fmt = FmtQ4K;
    static constexpr bool ONE_ROW_TILES = false;   // one row per wave tile at one activation row
    static constexpr int WGS_PER_CU_ONE_ROW = 8;
    static __host__ __device__ int rows_per_pass(int) { return 1; }
    template <int B, int R, int NW, class Epi, class Done = NoTileHook>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e, Done&& d = Done()) {
        rows_q4k<B, R, NW, false, false>(j, lds, e, d);
    }
};
// Q4_K rows of at most 8 super-blocks (k <= 2048): 2 or 4 rows share a pass.
struct EngQ4KShort {
    using Fmt = FmtQ4K;
    static constexpr bool ONE_ROW_TILES = false;   // one row per wave tile at one activation row
    static constexpr int WGS_PER_CU_ONE_ROW = 8;
    static __host__ __device__ int rows_per_pass(int nb) { return q4k_rows_per_pass(nb); }
    template <int B, int R, int NW, class Epi, class Done = NoTileHook>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e, Done&& d = Done()) {
        rows_q4k<B, R, NW, true, false>(j, lds, e, d);
    }
};
// Q5_K: the Q4_K engine with the fifth-bit plane (long and short rows alike).
struct EngQ5K {
    using Fmt = FmtQ5K;
    static constexpr bool ONE_ROW_TILES = false;   // one row per wave tile at one activation row
    static constexpr int WGS_PER_CU_ONE_ROW = 8;
    static __host__ __device__ int rows_per_pass(int) { return 1; }
    template <int B, int R, int NW, class Epi, class Done = NoTileHook>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e, Done&& d = Done()) {
        rows_q4k<B, R, NW, false, true>(j, lds, e, d);
    }
};
struct EngQ5KShort {
    using Fmt = FmtQ5K;
    static constexpr bool ONE_ROW_TILES = false;   // one row per wave tile at one activation row
    static constexpr int WGS_PER_CU_ONE_ROW = 8;
    static __host__ __device__ int rows_per_pass(int nb) { return q4k_rows_per_pass(nb); }
    template <int B, int R, int NW, class Epi, class Done = NoTileHook>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e, Done&& d = Done()) {
        rows_q4k<B, R, NW, true, true>(j, lds, e, d);
    }
};
struct EngQ6K {
    using Fmt = FmtQ6K;
    static constexpr bool ONE_ROW_TILES = true;   // one row per wave tile at one activation row
    static constexpr int WGS_PER_CU_ONE_ROW = 3;
    static __host__ __device__ int rows_per_pass(int) { return 1; }
    template <int B, int R, int NW, class Epi, class Done = NoTileHook>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e, Done&& d = Done()) {
        rows_q6k<B, R, NW, false>(j, lds, e, d);
    }
};
// Q6_K rows of at most 8 super-blocks: 2 or 4 rows share a pass.
struct EngQ6KShort {
    using Fmt = FmtQ6K;
    static constexpr bool ONE_ROW_TILES = false;   // one row per wave tile at one activation row
    static constexpr int WGS_PER_CU_ONE_ROW = 8;
    static __host__ __device__ int rows_per_pass(int nb) { return q4k_rows_per_pass(nb); }
    template <int B, int R, int NW, class Epi, class Done = NoTileHook>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e, Done&& d = Done()) {
        rows_q6k<B, R, NW, true>(j, lds, e, d);
    }
};
struct EngQ80 {
    using Fmt = FmtQ80;
    static constexpr bool ONE_ROW_TILES = false;   // one row per wave tile at one activation row
    static constexpr int WGS_PER_CU_ONE_ROW = 8;
    static __host__ __device__ int rows_per_pass(int) { return 1; }
    template <int B, int R, int NW, class Epi, class Done = NoTileHook>
    static __device__ __forceinline__ void run(const RowJob<NW>& j, uint8_t* lds, Epi&& e, Done&& d = Done()) {
        rows_q80<B, R, NW>(j, lds, e, d);
    }
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

static inline int lds_bytes_of(int wtype, int nb, int batch) {
    switch (wtype) {
        case LK_TYPE_Q4_K: case LK_TYPE_Q5_K: return lds_bytes_for<FmtQ4K>(nb, batch);
        case LK_TYPE_Q6_K: return lds_bytes_for<FmtQ6K>(nb, batch);
        default: return lds_bytes_for<FmtQ80>(nb, batch);
    }
}

static inline int block_len_of(int wtype) {
    switch (wtype) {
        case LK_TYPE_Q4_K: case LK_TYPE_Q5_K: case LK_TYPE_Q6_K: return 256;
        case LK_TYPE_Q8_0: return 32;
        default: return 0;
    }
}
static inline int block_bytes_of(int wtype) {
    switch (wtype) {
        case LK_TYPE_Q4_K: return Q4K_BYTES;
        case LK_TYPE_Q5_K: return Q5K_BYTES;
        case LK_TYPE_Q6_K: return Q6K_BYTES;
        case LK_TYPE_Q8_0: return Q80_BYTES;
        default: return 0;
    }
}

}  // namespace mmvq

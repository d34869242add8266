// Prefill / batched matmul on int8 MFMA: GGUF weight rows against Q8_1-quantized token rows.
//
//   out[token, n] = sum over 32-value sub-blocks s of  wscale_s[n] * d8_s[token] * D_s[n, token]
//                   (Q4_K: minus sum_s (dmin*m_s)[n] * (d8_s*S_s)[token])
// where D_s is the exact integer dot of a sub-block (v_mfma_i32_32x32x32_i8, K = 32 = one
// sub-block) and S_s the integer sum of the activation codes. The integer part is what loken's
// CPU path forms (src/tensor/quant_cpu/format/q4_k.rs:138-153, q6_k.rs:137-160, q8_0.rs:88-95);
// the f32 combine is the Q8_1-side one (cuda/moe/gguf.cuh:664-713, 782-816, 486-495). This file
// stands in for cuda/mmq_gguf/{mmq_quantize.cu, mmq_launch.cuh, mmq_gguf.cuh} of the reference
// and shares nothing with them but the entry-point names and the workspace size contract.
//
// Workspace ("y", written by launch_mmq_quantize_q8_1_*): per (256-value block kb, row) one
// record of 288 bytes = 2 x 144, block-major: record (kb * rows + row) holds
//   [256 int8 codes][8 x f16 d8][8 x int16 sum of codes]   (one d8 / sum per 32 codes).
// Same bytes per row as the reference's block_q8_1_mmq tiles (144 per 128 values), so the
// host-side sizing rows * (k_padded/128) * 144 (+ slack) of src/tensor/quantized/kernel_matmul/
// mmq.rs:38-41 holds unchanged. The quantization rule is the decode quantizer's (d = amax/127,
// codes = round_half_away(x * (1/d))), so a tiled product is M mat-vec products to the integer.
//
// Kernel shape: workgroup tile 128 weight rows x TM tokens, K walked one 256-value block at a
// time. Per step the workgroup expands the weight nibbles to int8 in LDS laid out
// [sub-block][row][32 bytes] (so an MFMA operand is one conflict-free ds_read_b128 per lane),
// copies the token codes likewise, and tables the per-sub-block scales as f32. A wave owns a
// 32*JT x 32*IT patch of the tile: lanes <-> weight rows (coalesced stores), accumulator
// registers <-> tokens. The Q4_K min term is a rank-8 update per block and runs on the f32
// MFMA (v_mfma_f32_32x32x2_f32) straight into the accumulators, costing no per-element VALU.

#include "mmq_problem.h"
#include "legacy_blocks.h"
#include "codebook_blocks.h"

#include <cstdlib>

namespace {

constexpr int MMQ_WG = 256;
constexpr int TN = 128;            // weight rows per workgroup tile
constexpr int REC_BYTES = MMQ_REC_BYTES;

// --------------------------------------------------------------------------------------------
// Activation quantizer -> workspace records
// --------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void mmq_quantize_kernel(const T* __restrict__ x,
                                                           const int32_t* __restrict__ ids,
                                                           uint8_t* __restrict__ vy, int64_t ne00,
                                                           int64_t s01, int64_t s02, int64_t s03,
                                                           int64_t ne0, int ne1, int ne2) {
#pragma clang fp contract(off)
    const int64_t i0 = ((int64_t)blockIdx.y * 256 + threadIdx.x) * 4;
    if (i0 >= ne0) return;
    const int row = blockIdx.x;
    const int64_t channel = blockIdx.z % ne2, sample = blockIdx.z / ne2;
    const int64_t src_row = ids ? ids[row] : row;
    const T* xr = x + sample * s03 + channel * s02 + src_row * s01;

    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i0 + 0 < ne00) v.x = to_f32<T>(xr[i0 + 0]);
    if (i0 + 1 < ne00) v.y = to_f32<T>(xr[i0 + 1]);
    if (i0 + 2 < ne00) v.z = to_f32<T>(xr[i0 + 2]);
    if (i0 + 3 < ne00) v.w = to_f32<T>(xr[i0 + 3]);

    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = max8(amax);
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const int q0 = (int)roundf(v.x * inv), q1 = (int)roundf(v.y * inv);
    const int q2 = (int)roundf(v.z * inv), q3 = (int)roundf(v.w * inv);
    int quad_sum;
    const int sum = sum8(q0 + q1 + q2 + q3, quad_sum);

    const int64_t kb = i0 / 256;
    const int64_t blocks_per_channel = (ne0 / 256) * ne1;
    uint8_t* rec = vy + ((int64_t)blockIdx.z * blocks_per_channel + kb * ne1 + row) * REC_BYTES;
    const int in_rec = (int)(i0 % 256);
    *(uint32_t*)(rec + in_rec) = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) |
                                 ((uint32_t)(q2 & 0xFF) << 16) | ((uint32_t)(q3 & 0xFF) << 24);
    if ((in_rec & 31) == 0) {
        const int s = in_rec >> 5;
        *(uint16_t*)(rec + 256 + 2 * s) = __half_as_ushort(__float2half_rn(d));
        *(int16_t*)(rec + 272 + 2 * s) = (int16_t)sum;
    }
}

static void launch_quantize(const void* x, const int32_t* ids, void* vy, int type_x, int64_t ne00,
                            int64_t s01, int64_t s02, int64_t s03, int64_t ne0, int64_t ne1,
                            int64_t ne2, int64_t ne3, void* stream) {
    if (!x || !vy || ne1 <= 0 || ne0 <= 0 || ne0 % 256 != 0 || ne2 <= 0 || ne3 <= 0) return;
    const dim3 grid((unsigned)ne1, (unsigned)((ne0 + 1023) / 1024), (unsigned)(ne2 * ne3));
    hipStream_t s = (hipStream_t)stream;
    if (type_x == LK_TYPE_F16) {
        hipLaunchKernelGGL(mmq_quantize_kernel<__half>, grid, dim3(256), 0, s, (const __half*)x, ids,
                           (uint8_t*)vy, ne00, s01, s02, s03, ne0, (int)ne1, (int)ne2);
    } else if (type_x == LK_TYPE_BF16) {
        hipLaunchKernelGGL(mmq_quantize_kernel<__hip_bfloat16>, grid, dim3(256), 0, s, (const __hip_bfloat16*)x, ids,
                           (uint8_t*)vy, ne00, s01, s02, s03, ne0, (int)ne1, (int)ne2);
    } else {
        hipLaunchKernelGGL(mmq_quantize_kernel<float>, grid, dim3(256), 0, s, (const float*)x, ids,
                           (uint8_t*)vy, ne00, s01, s02, s03, ne0, (int)ne1, (int)ne2);
    }
    (void)hipGetLastError();
}

// --------------------------------------------------------------------------------------------
// Weight formats: how one 256-value block of TN rows becomes int8 sub-block tiles + scales.
// LDS per step:  wq[8][TN][32] int8, aq[8][TM][32] int8, wsc[NS][TN] f32, wmn[8][TN] f32 (Q4_K),
//                ad8[8][TM] f32, ads[8][TM] f32 (Q4_K).   NS = weight scales per block (8 or 16).
// Staging is split in two so a step's global loads fly while the previous step is multiplied:
// fetch() issues the loads into a register fragment, commit() expands the fragment into LDS.
// --------------------------------------------------------------------------------------------
// Q5 = false: Q4_K. Q5 = true: Q5_K, the same header followed by 32 bytes of fifth bits (bit s of
// byte l belongs to value l of sub-block s, worth 16: src/tensor/quant_cpu/format/q5_k.rs:66-71) and
// then the nibbles; the int8 tiles take codes 0..31 as they take 0..15.
template <bool Q5>
struct MmqQ45K {
    static constexpr int ALIGN = 4;   // whole-header reads
    static constexpr int BLOCK_BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES;
    static constexpr int QS0 = Q5 ? 48 : 16;
    static constexpr bool F16_TILES = !Q5;   // Q4_K above 32 tokens (dense) or 64 (expert-batched): the f16 tile kernels
    static constexpr int WIDE_FROM = 384;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int NS = 8;          // one weight scale per 32 values
    static constexpr bool HAS_MIN = true;
    static constexpr int MIN_RANK = 8;   // one minimum per 32 values
    static constexpr int BLOCKS_PER_STEP = 1;
    static constexpr int QCH = TN * 8 / MMQ_WG;   // 16-byte qs chunks per thread per step

    struct Frag {
        uint4 q[QCH];
        uint4 qh[Q5 ? QCH : 1];
        uint4 hdr;
    };
    // nb: Q4_K blocks between consecutive rows
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, c = idx & 7;
            const int gn = min(n0 + row, n - 1);
            const uint8_t* block = w + ((int64_t)gn * nb + kb) * BLOCK_BYTES;
            f.q[i] = *(const uint4*)(block + QS0 + 16 * c);
            if (Q5) f.qh[i] = *(const uint4*)(block + 16 + 16 * (c & 1));
        }
        if (threadIdx.x < TN) {
            const int gn = min(n0 + (int)threadIdx.x, n - 1);
            f.hdr = *(const uint4*)(w + ((int64_t)gn * nb + kb) * BLOCK_BYTES);
        }
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, c = idx & 7;
            const uint4 q = f.q[i];
            uint4 lo, hi;
            lo.x = q.x & 0x0F0F0F0Fu; hi.x = (q.x >> 4) & 0x0F0F0F0Fu;
            lo.y = q.y & 0x0F0F0F0Fu; hi.y = (q.y >> 4) & 0x0F0F0F0Fu;
            lo.z = q.z & 0x0F0F0F0Fu; hi.z = (q.z >> 4) & 0x0F0F0F0Fu;
            lo.w = q.w & 0x0F0F0F0Fu; hi.w = (q.w >> 4) & 0x0F0F0F0Fu;
            const int p = c >> 1, h = c & 1;
            if (Q5) {
                const uint4 b = f.qh[i];
                const int s0 = 2 * p;
                lo.x |= ((b.x >> s0) << 4) & 0x10101010u; hi.x |= ((b.x >> s0) << 3) & 0x10101010u;
                lo.y |= ((b.y >> s0) << 4) & 0x10101010u; hi.y |= ((b.y >> s0) << 3) & 0x10101010u;
                lo.z |= ((b.z >> s0) << 4) & 0x10101010u; hi.z |= ((b.z >> s0) << 3) & 0x10101010u;
                lo.w |= ((b.w >> s0) << 4) & 0x10101010u; hi.w |= ((b.w >> s0) << 3) & 0x10101010u;
            }
            *(uint4*)(wq + ((2 * p) * TN + row) * 32 + 16 * h) = lo;
            *(uint4*)(wq + ((2 * p + 1) * TN + row) * 32 + 16 * h) = hi;
        }
        if (threadIdx.x < TN) {
            const int row = threadIdx.x;
            const bool live = n0 + row < n;
            const float d = live ? f16_bits_to_f32(f.hdr.x & 0xFFFFu) : 0.f;
            const float dmin = live ? f16_bits_to_f32(f.hdr.x >> 16) : 0.f;
            const uint32_t w1 = f.hdr.y, w2 = f.hdr.z, w3 = f.hdr.w;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                uint32_t sc, mn;
                if (j < 4) {
                    sc = (w1 >> (8 * j)) & 63u;
                    mn = (w2 >> (8 * j)) & 63u;
                } else {
                    const int t = j - 4;
                    sc = ((w3 >> (8 * t)) & 0xFu) | ((((w1 >> (8 * t)) >> 6) & 3u) << 4);
                    mn = ((w3 >> (8 * t + 4)) & 0xFu) | ((((w2 >> (8 * t)) >> 6) & 3u) << 4);
                }
                wsc[j * TN + row] = d * (float)sc;
                wmn[j * TN + row] = -(dmin * (float)mn);
            }
        }
    }
};
using MmqQ4K = MmqQ45K<false>;
using MmqQ5K = MmqQ45K<true>;

// Q6_K: sixteen int8 scales per block, one per 16 values, so one MFMA K (32) spans two of them;
// the tile loop runs each 32-group as two MFMAs over half-masked weight operands.
struct MmqQ6K {
    static constexpr int ALIGN = 2;
    static constexpr int BLOCK_BYTES = Q6K_BYTES;
    static constexpr int NS = 16;
    static constexpr bool HAS_MIN = false;
    static constexpr int MIN_RANK = 0;
    static constexpr bool F16_TILES = false;
    static constexpr int WIDE_FROM = 384;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int BLOCKS_PER_STEP = 1;
    static constexpr int QCH = TN * 8 / MMQ_WG;

    struct Frag {
        uint4 ql[QCH], qh[QCH];
        uint4 sc;       // the sixteen scale bytes of this thread's row
        uint32_t d;     // its f16 d
    };
    static __device__ __forceinline__ uint32_t word(uint32_t ql, uint32_t qh, int nib_shift, int hi_shift) {
        const uint32_t code = ((ql >> nib_shift) & 0x0F0F0F0Fu) | (((qh >> hi_shift) & 0x03030303u) << 4);
        return (code + 0x60606060u) ^ 0x80808080u;  // per byte: code - 32, signed
    }
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, c = idx & 7;
            const int h = c >> 2, lh = c & 1;
            const int gn = min(n0 + row, n - 1);
            const uint8_t* bp = w + ((int64_t)gn * nb + kb) * Q6K_BYTES;
            f.ql[i] = *(const uint4_a2*)(bp + 16 * c);
            f.qh[i] = *(const uint4_a2*)(bp + 128 + 16 * (2 * h + lh));
        }
        if (threadIdx.x < TN) {
            const int gn = min(n0 + (int)threadIdx.x, n - 1);
            const uint8_t* bp = w + ((int64_t)gn * nb + kb) * Q6K_BYTES;
            f.sc = *(const uint4_a2*)(bp + 192);
            f.d = *(const uint16_t*)(bp + 208);
        }
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
        (void)wmn;
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, c = idx & 7;
            const int h = c >> 2, g0 = (c >> 1) & 1, lh = c & 1;
            const uint4 ql = f.ql[i], qh = f.qh[i];
            uint4 ca, cb;
            const int sh = 2 * g0;
            ca.x = word(ql.x, qh.x, 0, sh); cb.x = word(ql.x, qh.x, 4, sh + 4);
            ca.y = word(ql.y, qh.y, 0, sh); cb.y = word(ql.y, qh.y, 4, sh + 4);
            ca.z = word(ql.z, qh.z, 0, sh); cb.z = word(ql.z, qh.z, 4, sh + 4);
            ca.w = word(ql.w, qh.w, 0, sh); cb.w = word(ql.w, qh.w, 4, sh + 4);
            *(uint4*)(wq + ((4 * h + g0) * TN + row) * 32 + 16 * lh) = ca;
            *(uint4*)(wq + ((4 * h + g0 + 2) * TN + row) * 32 + 16 * lh) = cb;
        }
        if (threadIdx.x < TN) {
            const int row = threadIdx.x;
            const float d = n0 + row < n ? f16_bits_to_f32(f.d) : 0.f;
            const uint32_t w[4] = {f.sc.x, f.sc.y, f.sc.z, f.sc.w};
#pragma unroll
            for (int j = 0; j < 16; ++j)
                wsc[j * TN + row] = d * (float)(int8_t)((w[j >> 2] >> (8 * (j & 3))) & 0xFFu);
        }
    }
};

// Q8_0: eight 34-byte blocks per 256-value step, codes copied as they are.
struct MmqQ80 {
    static constexpr int BLOCK_BYTES = Q80_BYTES;
    static constexpr int ALIGN = 2;
    static constexpr int NS = 8;
    static constexpr bool HAS_MIN = false;
    static constexpr int MIN_RANK = 0;
    static constexpr bool F16_TILES = false;
    static constexpr int WIDE_FROM = 96;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int BLOCKS_PER_STEP = 8;
    static constexpr int QCH = TN * 16 / MMQ_WG, DCH = TN * 8 / MMQ_WG;

    struct Frag {
        uint4 q[QCH];
        uint32_t d[DCH];
    };
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 4, c = idx & 15, blk = c >> 1, h = c & 1;
            const int gn = min(n0 + row, n - 1);
            f.q[i] = *(const uint4_a2*)(w + ((int64_t)gn * nb + (int64_t)kb * 8 + blk) * Q80_BYTES + 2 + 16 * h);
        }
#pragma unroll
        for (int i = 0; i < DCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, blk = idx & 7;
            const int gn = min(n0 + row, n - 1);
            f.d[i] = *(const uint16_t*)(w + ((int64_t)gn * nb + (int64_t)kb * 8 + blk) * Q80_BYTES);
        }
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
        (void)wmn;
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 4, c = idx & 15, blk = c >> 1, h = c & 1;
            *(uint4*)(wq + (blk * TN + row) * 32 + 16 * h) = f.q[i];
        }
#pragma unroll
        for (int i = 0; i < DCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, blk = idx & 7;
            wsc[blk * TN + row] = n0 + row < n ? f16_bits_to_f32(f.d[i]) : 0.f;
        }
    }
};

// The 32-value nibble formats (Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, MXFP4): eight blocks per 256-value step,
// one scale each, so the tile is Q8_0's with the codes expanded on the way into LDS. Codes leave as
// int8 less the format's bias (a table format's as its levels); Q4_1 / Q5_1 keep unsigned codes and
// table the block minimum, which rides the rank-8 update that serves Q4_K's: + m * (d8 * sum of codes).
// A thread takes whole blocks (row = idx / 8, block = idx % 8: a row's eight blocks are one
// contiguous run of 136..192 bytes).
template <int ID>
struct MmqLegacy {
    using L = Legacy<ID>;
    static constexpr int BLOCK_BYTES = L::BYTES;
    static constexpr int NS = 8;
    static constexpr bool HAS_MIN = L::M_AT >= 0;
    static constexpr int MIN_RANK = HAS_MIN ? 8 : 0;
    static constexpr bool F16_TILES = false;
    static constexpr int WIDE_FROM = 300;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int BLOCKS_PER_STEP = 8;
    static constexpr int ALIGN = L::BYTES % 2 ? 1 : 2;
    static constexpr int PER = TN * 8 / MMQ_WG;

    struct Frag {
        uint4 q[PER];
        uint32_t qh[PER];
        float d[PER], m[PER];
    };
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, blk = idx & 7;
            const int gn = min(n0 + row, n - 1);
            const uint8_t* bp = w + ((int64_t)gn * nb + (int64_t)kb * 8 + blk) * L::BYTES;
            f.q[i] = block_code_bytes<L>(bp);
            f.qh[i] = block_fifth_word<L>(bp);
            f.d[i] = block_scale<L>(bp);
            f.m[i] = HAS_MIN ? f16_bits_to_f32(*(const uint16_t*)(bp + (HAS_MIN ? L::M_AT : 0))) : 0.f;
        }
    }
    static __device__ __forceinline__ uint32_t less_bias(uint32_t codes) {
        // per byte code - BIAS as int8: code + (0x80 - BIAS) never carries (code <= 31), and flipping
        // bit 7 takes the 0x80 off again in two's complement
        if (L::BIAS == 0) return codes;
        return (codes + 0x01010101u * (uint32_t)(0x80 - L::BIAS)) ^ 0x80808080u;
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, blk = idx & 7;
            uint4 lo, hi;
            expand_codes<L>(f.q[i], f.qh[i], lo, hi);
            lo = make_uint4(less_bias(lo.x), less_bias(lo.y), less_bias(lo.z), less_bias(lo.w));
            hi = make_uint4(less_bias(hi.x), less_bias(hi.y), less_bias(hi.z), less_bias(hi.w));
            *(uint4*)(wq + (blk * TN + row) * 32) = lo;
            *(uint4*)(wq + (blk * TN + row) * 32 + 16) = hi;
            const bool live = n0 + row < n;
            wsc[blk * TN + row] = live ? f.d[i] : 0.f;
            if (HAS_MIN) wmn[blk * TN + row] = live ? f.m[i] : 0.f;
        }
    }
};
using MmqQ40 = MmqLegacy<LK_TYPE_Q4_0>;
using MmqQ41 = MmqLegacy<LK_TYPE_Q4_1>;
using MmqQ50 = MmqLegacy<LK_TYPE_Q5_0>;
using MmqQ51 = MmqLegacy<LK_TYPE_Q5_1>;
using MmqIq4Nl = MmqLegacy<LK_TYPE_IQ4_NL>;
using MmqMxfp4 = MmqLegacy<LK_TYPE_MXFP4>;

// Q3_K {hmask[32], qs[64], scales[12], d} (110 bytes; src/tensor/quant_cpu/format/q3_k.rs:10-37, 127-146):
// sixteen six-bit scales (less 32), one per 16 values, over codes (two bits, less four where the hmask
// bit is clear) in -4..3: Q6_K's tile shape, two scales per 32-value sub-block. A thread takes one half
// (128 values) of a row's super-block: its four sub-blocks share the same 32 code bytes at four shifts.
struct MmqQ3K {
    static constexpr int ALIGN = 2;
    static constexpr int BLOCK_BYTES = 110;
    static constexpr int NS = 16;
    static constexpr bool HAS_MIN = false;
    static constexpr int MIN_RANK = 0;
    static constexpr bool F16_TILES = false;
    static constexpr int WIDE_FROM = 384;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int BLOCKS_PER_STEP = 1;
    static_assert(TN * 2 == MMQ_WG, "one (row, half) per thread");

    struct Frag {
        uint4 q0, q1, h0, h1;
        uint32_t s0, s1, s2, d;
    };
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
        const int row = threadIdx.x >> 1, half = threadIdx.x & 1;
        const int gn = min(n0 + row, n - 1);
        const uint8_t* bp = w + ((int64_t)gn * nb + kb) * BLOCK_BYTES;
        f.q0 = *(const uint4_a2*)(bp + 32 + 32 * half);
        f.q1 = *(const uint4_a2*)(bp + 48 + 32 * half);
        f.h0 = *(const uint4_a2*)bp;
        f.h1 = *(const uint4_a2*)(bp + 16);
        f.s0 = *(const uint32_a2*)(bp + 96);
        f.s1 = *(const uint32_a2*)(bp + 100);
        f.s2 = *(const uint32_a2*)(bp + 104);
        f.d = *(const uint16_t*)(bp + 108);
    }
    // two-bit codes less four where `clear` holds a 1, as int8: 0x80 + q - 4 never borrows
    static __device__ __forceinline__ uint32_t signed_codes(uint32_t q, uint32_t clear) {
        return ((q | 0x80808080u) - (clear << 2)) ^ 0x80808080u;
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
        (void)wmn;
        const int row = threadIdx.x >> 1, half = threadIdx.x & 1;
        const float d = n0 + row < n ? f16_bits_to_f32(f.d) : 0.f;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int j = 4 * half + jj, shift = 2 * jj;
            const uint32_t m2 = 0x03030303u, m1 = 0x01010101u;
            uint4 lo, hi;
            lo.x = signed_codes((f.q0.x >> shift) & m2, (~f.h0.x >> j) & m1);
            lo.y = signed_codes((f.q0.y >> shift) & m2, (~f.h0.y >> j) & m1);
            lo.z = signed_codes((f.q0.z >> shift) & m2, (~f.h0.z >> j) & m1);
            lo.w = signed_codes((f.q0.w >> shift) & m2, (~f.h0.w >> j) & m1);
            hi.x = signed_codes((f.q1.x >> shift) & m2, (~f.h1.x >> j) & m1);
            hi.y = signed_codes((f.q1.y >> shift) & m2, (~f.h1.y >> j) & m1);
            hi.z = signed_codes((f.q1.z >> shift) & m2, (~f.h1.z >> j) & m1);
            hi.w = signed_codes((f.q1.w >> shift) & m2, (~f.h1.w >> j) & m1);
            *(uint4*)(wq + (j * TN + row) * 32) = lo;
            *(uint4*)(wq + (j * TN + row) * 32 + 16) = hi;
            // scales 2 j and 2 j + 1 of the sixteen packed in twelve bytes (scale i: low four bits =
            // nibble i / 8 of byte i % 8, top two = bits 2 (i / 4) of byte 8 + i % 4)
            const int group = j >> 1, at = 2 * (j & 1);
            const uint32_t low = ((group & 1) ? f.s1 : f.s0) >> (8 * at + (group < 2 ? 0 : 4));
            const uint32_t top = f.s2 >> (8 * at + 2 * group);
            const int sc0 = (int)((low & 15u) | ((top & 3u) << 4)) - 32;
            const int sc1 = (int)(((low >> 8) & 15u) | (((top >> 8) & 3u) << 4)) - 32;
            wsc[(2 * j) * TN + row] = d * (float)sc0;
            wsc[(2 * j + 1) * TN + row] = d * (float)sc1;
        }
    }
};

// Q2_K {scales[16], qs[64], d, dmin} (84 bytes; src/tensor/quant_cpu/format/q2_k.rs:15-33): sixteen groups of
// sixteen two-bit codes, byte g of scales = scale (low nibble) and minimum (high nibble) of group g:
// d * scale * q - dmin * minimum. Q3_K's tile shape with unsigned codes, and the minimum as a rank-16
// update against the token's sums per 16 codes (cuda/moe/gguf.cuh:524-546 combines per group likewise).
struct MmqQ2K {
    static constexpr int ALIGN = 4;
    static constexpr int BLOCK_BYTES = 84;
    static constexpr int NS = 16;
    static constexpr bool HAS_MIN = true;
    static constexpr int MIN_RANK = 16;
    static constexpr bool F16_TILES = false;
    static constexpr int WIDE_FROM = 384;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int BLOCKS_PER_STEP = 1;
    static_assert(TN * 2 == MMQ_WG, "one (row, half) per thread");

    struct Frag {
        uint4 q0, q1;
        uint2 sm;       // the half's eight scale | minimum bytes
        uint32_t dm;    // d | dmin << 16
    };
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
        const int row = threadIdx.x >> 1, half = threadIdx.x & 1;
        const int gn = min(n0 + row, n - 1);
        const uint8_t* bp = w + ((int64_t)gn * nb + kb) * BLOCK_BYTES;
        f.q0 = *(const uint4_a4*)(bp + 16 + 32 * half);
        f.q1 = *(const uint4_a4*)(bp + 32 + 32 * half);
        f.sm = make_uint2(*(const uint32_t*)(bp + 8 * half), *(const uint32_t*)(bp + 8 * half + 4));
        f.dm = *(const uint32_t*)(bp + 80);
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
        const int row = threadIdx.x >> 1, half = threadIdx.x & 1;
        const bool live = n0 + row < n;
        const float d = live ? f16_bits_to_f32(f.dm & 0xFFFFu) : 0.f;
        const float dmin = live ? f16_bits_to_f32(f.dm >> 16) : 0.f;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int j = 4 * half + jj, shift = 2 * jj;
            const uint32_t m2 = 0x03030303u;
            *(uint4*)(wq + (j * TN + row) * 32) =
                make_uint4((f.q0.x >> shift) & m2, (f.q0.y >> shift) & m2, (f.q0.z >> shift) & m2, (f.q0.w >> shift) & m2);
            *(uint4*)(wq + (j * TN + row) * 32 + 16) =
                make_uint4((f.q1.x >> shift) & m2, (f.q1.y >> shift) & m2, (f.q1.z >> shift) & m2, (f.q1.w >> shift) & m2);
            const uint32_t pair = ((jj < 2 ? f.sm.x : f.sm.y) >> (16 * (jj & 1))) & 0xFFFFu;   // bytes 2 j, 2 j + 1
            wsc[(2 * j) * TN + row] = d * (float)(pair & 15u);
            wsc[(2 * j + 1) * TN + row] = d * (float)((pair >> 8) & 15u);
            wmn[(2 * j) * TN + row] = -(dmin * (float)((pair >> 4) & 15u));
            wmn[(2 * j + 1) * TN + row] = -(dmin * (float)(pair >> 12));
        }
    }
};

// IQ4_XS {d, scales_h, scales_l[4], qs[128]} (136 bytes; src/tensor/quant_cpu/format/iq4_xs.rs:5-37): eight
// runs of 32 values, each IQ4_NL levels under one six-bit scale less 32: the Q4_K tile shape without a
// minimum. A thread takes (row, run) items.
struct MmqIq4Xs {
    static constexpr int ALIGN = 4;
    static constexpr int BLOCK_BYTES = 136;
    static constexpr int NS = 8;
    static constexpr bool HAS_MIN = false;
    static constexpr int MIN_RANK = 0;
    static constexpr bool F16_TILES = false;
    static constexpr int WIDE_FROM = 300;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int BLOCKS_PER_STEP = 1;
    static constexpr int PER = TN * 8 / MMQ_WG;

    struct Frag {
        uint4 q[PER];
        uint2 head[PER];
    };
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, j = idx & 7;
            const int gn = min(n0 + row, n - 1);
            const uint8_t* bp = w + ((int64_t)gn * nb + kb) * BLOCK_BYTES;
            f.q[i] = *(const uint4_a4*)(bp + 8 + 16 * j);
            f.head[i] = *(const uint2_a2*)bp;   // d, scales_h | scales_l[4]
        }
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
        (void)wmn;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, j = idx & 7;
            const uint4 q = f.q[i];
            const uint4 lo = make_uint4(levels_of<1>(q.x & 0x0F0F0F0Fu), levels_of<1>(q.y & 0x0F0F0F0Fu),
                                        levels_of<1>(q.z & 0x0F0F0F0Fu), levels_of<1>(q.w & 0x0F0F0F0Fu));
            const uint4 hi = make_uint4(levels_of<1>((q.x >> 4) & 0x0F0F0F0Fu), levels_of<1>((q.y >> 4) & 0x0F0F0F0Fu),
                                        levels_of<1>((q.z >> 4) & 0x0F0F0F0Fu), levels_of<1>((q.w >> 4) & 0x0F0F0F0Fu));
            *(uint4*)(wq + (j * TN + row) * 32) = lo;
            *(uint4*)(wq + (j * TN + row) * 32 + 16) = hi;
            const uint32_t low = (f.head[i].y >> (4 * j)) & 15u, high = (f.head[i].x >> (16 + 2 * j)) & 3u;
            const int sc = (int)(low | (high << 4)) - 32;
            wsc[j * TN + row] = n0 + row < n ? f16_bits_to_f32(f.head[i].x & 0xFFFFu) * (float)sc : 0.f;
        }
    }
};

// The codebook formats of the expert tables (IQ3_XXS, IQ3_S, IQ2_S, Q2_0; codebook_blocks.h): a run of 32
// values decodes to int8 weights under an odd integer scale times the block's float, so the tiles take them
// as they take IQ4_XS; IQ2_S scales its halves apart and takes Q6_K's shape of two scales per sub-block. A
// thread takes (row, run) items; Q2_0's blocks of 64 values go four to a step.
template <int ID>
struct MmqCodebook {
    using C = codebook::Fmt<ID>;
    static constexpr int ALIGN = 2;
    static constexpr int BLOCK_BYTES = C::BYTES;
    static constexpr int NS = ID == 22 ? 16 : 8;
    static constexpr bool HAS_MIN = false;
    static constexpr int MIN_RANK = 0;
    static constexpr bool F16_TILES = false;
    static constexpr int WIDE_FROM = 300;   // 128-token tiles from this many of them (launch_dense)
    static constexpr int BLOCKS_PER_STEP = 8 / C::RUNS;
    static constexpr int PER = TN * 8 / MMQ_WG;

    struct Frag {
        codebook::Raw raw[PER];
    };
    static __device__ __forceinline__ void fetch(Frag& f, const uint8_t* __restrict__ w, int64_t nb, int kb,
                                                 int n0, int n) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, j = idx & 7;
            const int gn = min(n0 + row, n - 1);
            const uint8_t* bp = w + ((int64_t)gn * nb + (int64_t)kb * BLOCKS_PER_STEP + j / C::RUNS) * BLOCK_BYTES;
            f.raw[i] = codebook::fetch<ID>(bp, j % C::RUNS);
        }
    }
    static __device__ __forceinline__ void commit(const Frag& f, int n0, int n, int8_t* wq, float* wsc, float* wmn) {
        (void)wmn;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, row = idx >> 3, j = idx & 7;
            const codebook::Run r = codebook::decode<ID>(f.raw[i], j % C::RUNS);
            *(uint4*)(wq + (j * TN + row) * 32) = r.lo;
            *(uint4*)(wq + (j * TN + row) * 32 + 16) = r.hi;
            const float d = n0 + row < n ? r.d : 0.f;
            if (NS == 16) {
                wsc[(2 * j) * TN + row] = d * (float)r.sc0;
                wsc[(2 * j + 1) * TN + row] = d * (float)r.sc1;
            } else {
                wsc[j * TN + row] = d * (float)r.sc0;
            }
        }
    }
};
using MmqIq3Xxs = MmqCodebook<18>;
using MmqIq3S = MmqCodebook<21>;
using MmqIq2S = MmqCodebook<22>;
using MmqQ2_0 = MmqCodebook<42>;

// Token rows [m0, m0+TM) of block kb (record layout above). Rows at or past m_end read as zeros.
// S16: the weight format has a minimum per 16 values (Q2_K), so the sums are formed per chunk of 16
// codes from the codes themselves (the record holds them per 32) and each chunk's thread reads its scale.
template <int TM, bool S16 = false>
struct TokenFrag {
    static constexpr int CCH = (TM * 16 + MMQ_WG - 1) / MMQ_WG;   // code chunks per thread
    uint4 codes[CCH];
    uint32_t chunk_d8[S16 ? CCH : 1];
    uint4 d8, sums;   // thread r < TM: the scales and sums of row r

    __device__ __forceinline__ void fetch(const uint8_t* __restrict__ y, int64_t rows_total, int kb, int m0, int m_end) {
#pragma unroll
        for (int i = 0; i < CCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, r = idx >> 4, c = idx & 15;
            codes[i] = make_uint4(0, 0, 0, 0);
            if (S16) chunk_d8[i] = 0;
            if (idx < TM * 16 && m0 + r < m_end) {
                const uint8_t* rec = y + ((int64_t)kb * rows_total + m0 + r) * REC_BYTES;
                codes[i] = *(const uint4*)(rec + 16 * c);
                if (S16) chunk_d8[i] = *(const uint16_t*)(rec + 256 + 2 * (c >> 1));
            }
        }
        d8 = sums = make_uint4(0, 0, 0, 0);
        if ((int)threadIdx.x < TM && m0 + (int)threadIdx.x < m_end) {
            const uint8_t* rec = y + ((int64_t)kb * rows_total + m0 + threadIdx.x) * REC_BYTES;
            d8 = *(const uint4*)(rec + 256);
            sums = *(const uint4*)(rec + 272);
        }
    }
    template <bool WITH_SUMS>
    __device__ __forceinline__ void commit(int8_t* aq, float* ad8, float* ads) const {
#pragma unroll
        for (int i = 0; i < CCH; ++i) {
            const int idx = threadIdx.x + i * MMQ_WG, r = idx >> 4, c = idx & 15;
            if (idx < TM * 16) {
                *(uint4*)(aq + ((c >> 1) * TM + r) * 32 + 16 * (c & 1)) = codes[i];
                if (S16) {
                    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
                    ads[c * TM + r] = f16_bits_to_f32(chunk_d8[i]) * (float)dot16(ones, codes[i], 0);
                }
            }
        }
        if ((int)threadIdx.x < TM) {
            const int r = threadIdx.x;
            const uint32_t dw[4] = {d8.x, d8.y, d8.z, d8.w}, sw[4] = {sums.x, sums.y, sums.z, sums.w};
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const float d = f16_bits_to_f32((dw[s >> 1] >> (16 * (s & 1))) & 0xFFFFu);
                ad8[s * TM + r] = d;
                if (WITH_SUMS && !S16) ads[s * TM + r] = d * (float)(int)(int16_t)((sw[s >> 1] >> (16 * (s & 1))) & 0xFFFFu);
            }
        }
    }
};

template <class F, int TM, int WAVES_M>
static __device__ __forceinline__ void mmq_tile(const MmqProblem& pb, int n0, int m0, uint8_t* lds, int kb0, int kb1) {
    constexpr int WAVES_N = 4 / WAVES_M;
    constexpr int JT = TN / (32 * WAVES_N), IT = TM / (32 * WAVES_M);
    static_assert(JT >= 1 && IT >= 1, "tile does not split over four waves");
    // Which operand's index lands on the accumulator registers. A wave with more token tiles than
    // weight tiles puts the weight rows there (matrix instruction called as weights x tokens);
    // not for two scales per sub-block (Q6_K), whose second set of 16 registers spills.
    constexpr bool SWAP = IT > JT && F::NS != 16;

    int8_t* wq = (int8_t*)lds;                       // [8][TN][32]
    int8_t* aq = wq + 8 * TN * 32;                   // [8][TM][32]
    float* wsc = (float*)(aq + 8 * TM * 32);         // [NS][TN]
    float* wmn = wsc + F::NS * TN;                   // [MIN_RANK][TN]
    float* ad8 = wmn + F::MIN_RANK * TN;             // [8][TM]
    float* ads = ad8 + 8 * TM;                       // [MIN_RANK][TM]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave % WAVES_N, wm = wave / WAVES_N;
    const int l32 = lane & 31, lh = lane >> 5;

    v16f acc[IT][JT];
#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
        for (int jt = 0; jt < JT; ++jt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[it][jt][v] = 0.f;

    typename F::Frag wf;
    TokenFrag<TM, F::MIN_RANK == 16> tf;
    F::fetch(wf, pb.w, pb.row_blocks, kb0, n0, pb.n);
    tf.fetch(pb.y, pb.rows_total, kb0, m0, pb.m_end);

    for (int kb = kb0; kb < kb1; ++kb) {
        __syncthreads();  // the previous step's readers are done with the tiles
        F::commit(wf, n0, pb.n, wq, wsc, wmn);
        tf.template commit<F::HAS_MIN>(aq, ad8, ads);
        __syncthreads();
        if (kb + 1 < kb1) {  // next step's loads fly under this step's arithmetic
            F::fetch(wf, pb.w, pb.row_blocks, kb + 1, n0, pb.n);
            tf.fetch(pb.y, pb.rows_total, kb + 1, m0, pb.m_end);
        }

#pragma unroll
        for (int s = 0; s < 8; ++s) {
            v4i a[IT], b[JT];
            float ws[JT], ws2[JT];
#pragma unroll
            for (int it = 0; it < IT; ++it)
                a[it] = *(const v4i*)(aq + (s * TM + (wm * IT + it) * 32 + l32) * 32 + 16 * lh);
#pragma unroll
            for (int jt = 0; jt < JT; ++jt) {
                b[jt] = *(const v4i*)(wq + (s * TN + (wn * JT + jt) * 32 + l32) * 32 + 16 * lh);
                if constexpr (F::NS == 16) {
                    ws[jt] = wsc[(2 * s) * TN + (wn * JT + jt) * 32 + l32];
                    ws2[jt] = wsc[(2 * s + 1) * TN + (wn * JT + jt) * 32 + l32];
                } else {
                    ws[jt] = wsc[s * TN + (wn * JT + jt) * 32 + l32];
                    ws2[jt] = 0.f;
                }
            }
            if constexpr (SWAP) {
                // Weight rows on the accumulator registers, tokens on the lanes: the 16 per-register
                // scales are the weight tile's (read once and shared by the wave's token tiles), the
                // token scale is one value per lane.
                float wsv[JT][16], ws2v[JT][16], wso[JT][16];
#pragma unroll
                for (int jt = 0; jt < JT; ++jt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int at = (wn * JT + jt) * 32 + 8 * g + 4 * lh;
                        const float4 t = *(const float4*)(wsc + (F::NS == 16 ? 2 * s : s) * TN + at);
                        wsv[jt][4 * g + 0] = t.x; wsv[jt][4 * g + 1] = t.y; wsv[jt][4 * g + 2] = t.z; wsv[jt][4 * g + 3] = t.w;
                        if constexpr (F::NS == 16) {
                            const float4 u = *(const float4*)(wsc + (2 * s + 1) * TN + at);
                            ws2v[jt][4 * g + 0] = u.x; ws2v[jt][4 * g + 1] = u.y; ws2v[jt][4 * g + 2] = u.z; ws2v[jt][4 * g + 3] = u.w;
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e) wso[jt][4 * g + e] = -12582912.0f * wsv[jt][4 * g + e];
                    }
#pragma unroll
                for (int it = 0; it < IT; ++it) {
                    const float d8l = ad8[s * TM + (wm * IT + it) * 32 + l32];
#pragma unroll
                    for (int jt = 0; jt < JT; ++jt) {
                        if constexpr (F::NS == 16) {
                            const v4i zero = {0, 0, 0, 0};
                            const v4i b_lo = lh == 0 ? b[jt] : zero, b_hi = lh == 0 ? zero : b[jt];
                            v16i c0 = {0}, c1 = {0};
                            c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(b_lo, a[it], c0, 0, 0, 0);
                            c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(b_hi, a[it], c1, 0, 0, 0);
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                const float t = fmaf(ws2v[jt][v], (float)c1[v], wsv[jt][v] * (float)c0[v]);
                                acc[it][jt][v] = fmaf(t, d8l, acc[it][jt][v]);
                            }
                        } else {
                            if constexpr (F::HAS_MIN) {
                                v16i c = {0};
                                c = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[jt], a[it], c, 0, 0, 0);
#pragma unroll
                                for (int v = 0; v < 16; ++v)
                                    acc[it][jt][v] = fmaf((float)c[v], wsv[jt][v] * d8l, acc[it][jt][v]);
                            } else {
                                // The int32 accumulators start at the bit pattern of 1.5 * 2^23, so the
                                // dots leave the matrix unit as the floats MAGIC + dot; the offset goes
                                // in the first fma, exactly (the weight scale is an f16: MAGIC * scale
                                // does not round), which then rounds dot * scale once, as
                                // convert-then-multiply would. (With a min term to carry as well, the 16
                                // registers of offsets cost more than the conversions they save.)
                                v16i c;
#pragma unroll
                                for (int v = 0; v < 16; ++v) c[v] = 0x4B400000;
                                c = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[jt], a[it], c, 0, 0, 0);
#pragma unroll
                                for (int v = 0; v < 16; ++v)
                                    acc[it][jt][v] = fmaf(fmaf(__int_as_float(c[v]), wsv[jt][v], wso[jt][v]), d8l, acc[it][jt][v]);
                            }
                        }
                    }
                }
            } else {
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                // d8 of the 16 tokens this lane's accumulator registers stand for
                float d8v[16];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float4 t = *(const float4*)(ad8 + s * TM + (wm * IT + it) * 32 + 8 * g + 4 * lh);
                    d8v[4 * g + 0] = t.x; d8v[4 * g + 1] = t.y; d8v[4 * g + 2] = t.z; d8v[4 * g + 3] = t.w;
                }
#pragma unroll
                for (int jt = 0; jt < JT; ++jt) {
                    if constexpr (F::NS == 16) {
                        // lanes 0-31 hold k 0..15 of the operand, lanes 32-63 k 16..31: masking one
                        // half leaves the 16-value group the other weight scale does not govern
                        const v4i zero = {0, 0, 0, 0};
                        const v4i b_lo = lh == 0 ? b[jt] : zero, b_hi = lh == 0 ? zero : b[jt];
                        // The accumulators start at the bit pattern of 1.5 * 2^23, so the dots leave
                        // the matrix unit as the floats MAGIC + dot and no conversion is spent; the
                        // offset comes off inside the fma, exactly (the weight scale is an f16 times
                        // an int8, 18 significant bits: MAGIC * scale does not round).
                        v16i c0, c1;
#pragma unroll
                        for (int v = 0; v < 16; ++v) c0[v] = c1[v] = 0x4B400000;
                        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[it], b_lo, c0, 0, 0, 0);
                        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[it], b_hi, c1, 0, 0, 0);
                        const float off0 = -12582912.0f * ws[jt], off1 = -12582912.0f * ws2[jt];
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const float t = fmaf(__int_as_float(c0[v]), ws[jt], off0) + fmaf(__int_as_float(c1[v]), ws2[jt], off1);
                            acc[it][jt][v] = fmaf(t, d8v[v], acc[it][jt][v]);
                        }
                    } else {
                        v16i c = {0};
                        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[it], b[jt], c, 0, 0, 0);
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            acc[it][jt][v] = fmaf((float)c[v], ws[jt] * d8v[v], acc[it][jt][v]);
                    }
                }
            }
            }
        }
        if (F::HAS_MIN) {
            // acc += (d8*S)[token, s] * (-dmin*m)[s, n], s = 0..MIN_RANK-1: K=2 f32 MFMAs, two s each
#pragma unroll
            for (int kk = 0; kk < F::MIN_RANK / 2; ++kk) {
                float am[IT], bm[JT];
#pragma unroll
                for (int it = 0; it < IT; ++it) am[it] = ads[(2 * kk + lh) * TM + (wm * IT + it) * 32 + l32];
#pragma unroll
                for (int jt = 0; jt < JT; ++jt) bm[jt] = wmn[(2 * kk + lh) * TN + (wn * JT + jt) * 32 + l32];
#pragma unroll
                for (int it = 0; it < IT; ++it)
#pragma unroll
                    for (int jt = 0; jt < JT; ++jt)
                        acc[it][jt] = SWAP ? __builtin_amdgcn_mfma_f32_32x32x2f32(bm[jt], am[it], acc[it][jt], 0, 0, 0)
                                           : __builtin_amdgcn_mfma_f32_32x32x2f32(am[it], bm[jt], acc[it][jt], 0, 0, 0);
            }
        }
    }

#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
        for (int jt = 0; jt < JT; ++jt) {
            if constexpr (SWAP) {
                const int col = m0 + (wm * IT + it) * 32 + l32;
                if (col < pb.m_end) {
                    const int64_t drow = pb.ids_dst ? pb.ids_dst[col] : col;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int gn = n0 + (wn * JT + jt) * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
                        if (gn < pb.n) pb.dst[drow * pb.ldd + gn] = acc[it][jt][v];
                    }
                }
            } else {
                const int gn = n0 + (wn * JT + jt) * 32 + l32;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int col = m0 + (wm * IT + it) * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
                    if (gn < pb.n && col < pb.m_end) {
                        const int64_t drow = pb.ids_dst ? pb.ids_dst[col] : col;
                        pb.dst[drow * pb.ldd + gn] = acc[it][jt][v];
                    }
                }
            }
        }
}

template <class F, int TM>
static constexpr int mmq_lds_bytes() {
    return 8 * TN * 32 + 8 * TM * 32 + (F::NS * TN + F::MIN_RANK * TN + 8 * TM + F::MIN_RANK * TM) * 4;
}

// Dense product. Workgroup id -> (n tile, m tile) so that the m tiles of one n tile (which
// re-read the same weight rows) are issued back to back on the same XCD: ids are dealt round
// robin over the 8 XCDs, so the XCD is id % 8 and its local sequence id / 8.
template <class F, int TM, int WAVES_M>
__global__ __launch_bounds__(MMQ_WG, 2) void mmq_dense_kernel(MmqProblem pb, int n_tiles, int m_tiles) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int id = blockIdx.x;
    const int xcd = id & 7, seq = id >> 3;
    const int m_tile = seq % m_tiles;
    const int n_tile = (seq / m_tiles) * 8 + xcd;
    if (n_tile >= n_tiles) return;
    mmq_tile<F, TM, WAVES_M>(pb, n_tile * TN, pb.m_begin + m_tile * TM, lds, 0, (int)pb.nb);
}

// The dense product with K cut into `splits` ranges of blocks, for shapes whose tiles alone leave most
// of the chip idle (4096 weight rows x 128 token rows are 32 tiles for 256 CUs, each walking all of K).
// A workgroup walks one range and writes its partial tile to part[split] ([token][n] floats, token
// rows n floats apart); mmq_split_sum_kernel then adds the ranges in ascending order, so a result does
// not depend on which workgroup finished when. Ids: the m tiles of one (n tile, range) back to back
// on one XCD, as above.
template <class F, int TM, int WAVES_M>
__global__ __launch_bounds__(MMQ_WG, 2) void mmq_dense_split_kernel(MmqProblem pb, int n_tiles, int m_tiles, int splits,
                                                                   float* part, int64_t part_stride) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int id = blockIdx.x;
    const int xcd = id & 7;
    int seq = id >> 3;
    const int m_tile = seq % m_tiles;
    seq /= m_tiles;
    const int split = seq % splits;
    const int n_tile = (seq / splits) * 8 + xcd;
    if (n_tile >= n_tiles) return;
    const int kb0 = (int)(pb.nb * split / splits), kb1 = (int)(pb.nb * (split + 1) / splits);
    pb.dst = part + split * part_stride;
    pb.ldd = pb.n;
    mmq_tile<F, TM, WAVES_M>(pb, n_tile * TN, pb.m_begin + m_tile * TM, lds, kb0, kb1);
}

// dst[token][c] = part[0][token][c] + part[1][token][c] + ... in that order; four columns a thread.
__global__ __launch_bounds__(256) void mmq_split_sum_kernel(const float* __restrict__ part, int splits, int64_t part_stride,
                                                            float* __restrict__ dst, int64_t count, int n, int64_t ldd) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= count) return;
    float4 a = *(const float4*)(part + i);
    for (int s = 1; s < splits; ++s) {
        const float4 b = *(const float4*)(part + s * part_stride + i);
        a.x += b.x;
        a.y += b.y;
        a.z += b.z;
        a.w += b.w;
    }
    const int64_t row = i / n, col = i - row * n;
    *(float4*)(dst + row * ldd + col) = a;
}

// Expert-batched product: expert e's slab against the sorted rows [bounds[e], bounds[e+1]).
// grid = (n tiles, column tiles sized for the longest run the host expects, stacks * experts);
// a run longer than the grid covers is walked by the same workgroups in further passes.
template <class F, int TM, int WAVES_M>
__global__ __launch_bounds__(MMQ_WG, 2) void mmq_moe_kernel(MmqProblem pb, const uint8_t* w_second,
                                                         int64_t dst_second, const int32_t* __restrict__ bounds,
                                                         int64_t stride_expert, int n_experts) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int stack = blockIdx.z / n_experts, e = blockIdx.z % n_experts;
    pb.m_begin = bounds[e];
    pb.m_end = bounds[e + 1];
    if (pb.m_end <= pb.m_begin) return;
    pb.w = (stack ? w_second : pb.w) + (int64_t)e * stride_expert;
    if (stack) pb.dst += dst_second;
    for (int m0 = pb.m_begin + blockIdx.y * TM; m0 < pb.m_end; m0 += gridDim.y * TM)
        mmq_tile<F, TM, WAVES_M>(pb, blockIdx.x * TN, m0, lds, 0, (int)pb.nb);
}

template <class F, int TM, int WAVES_M>
static int launch_dense_tm(const MmqProblem& pb, hipStream_t s, void* fixup = nullptr) {
    constexpr int lds_bytes = mmq_lds_bytes<F, TM>();
    const int n_tiles = (pb.n + TN - 1) / TN;
    const int m_tiles = (pb.m_end - pb.m_begin + TM - 1) / TM;
    const int n_groups = (n_tiles + 7) / 8;
    const int splits = mmq_splits(pb, (int64_t)n_tiles * m_tiles, 2 * lk_device().cus, fixup);   // two workgroups fit a CU
    if (splits > 1) {
        auto kernel = mmq_dense_split_kernel<F, TM, WAVES_M>;
        if (mmq_prepare_kernel(kernel, lds_bytes) != LK_OK) return 0;
        const int64_t count = (int64_t)pb.m_end * pb.n;
        hipLaunchKernelGGL(kernel, dim3(n_groups * 8 * m_tiles * splits), dim3(MMQ_WG), lds_bytes, s, pb, n_tiles, m_tiles,
                           splits, (float*)fixup, count);
        return lk_mmq_split_sum((const float*)fixup, splits, pb, s) == LK_OK ? TM : 0;
    }
    auto kernel = mmq_dense_kernel<F, TM, WAVES_M>;
    if (mmq_prepare_kernel(kernel, lds_bytes) != LK_OK) return 0;
    const int grid = n_groups * 8 * m_tiles;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(MMQ_WG), lds_bytes, s, pb, n_tiles, m_tiles);
    return hipGetLastError() == hipSuccess ? TM : 0;
}

template <class F>
static int launch_dense(void* fixup, const void* x, const void* y, void* dst, int64_t ncols_x, int64_t nrows_x,
                        int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst, void* stream) {
    if (!x || !y || !dst || ncols_x <= 0 || nrows_x <= 0 || ncols_y <= 0) return 0;
    if ((uintptr_t)x % F::ALIGN != 0) return 0;
    if (ncols_x % 256 != 0 || stride_row_x < ncols_x / 256 * F::BLOCKS_PER_STEP) return 0;
    if (stride_col_dst < nrows_x || nrows_x > INT32_MAX || ncols_y > INT32_MAX) return 0;
    MmqProblem pb{(const uint8_t*)x, (const uint8_t*)y, (float*)dst, nullptr, ncols_x / 256, stride_row_x,
                  ncols_y, stride_col_dst, (int)nrows_x, 0, (int)ncols_y};
    hipStream_t s = (hipStream_t)stream;
    if (ncols_y <= 32) return launch_dense_tm<F, 32, 1>(pb, s, fixup);
    // (Q2_K stays on 64-token tiles: with the rank-16 minimum its 128-token tile spills and runs 512 x
    // 4096 -> 14336 in 344 us against 240, 2048 x 14336 -> 4096 in 1155 against 742; every other format
    // is 3 to 40 % faster on the wide tile)
    // (Q4_K from 33 rows of a matrix of 2048 rows or more goes on to its 64-token f16 tiles: 14336 x 4096 at 64
    // rows 40.5 us against 46.4 on the int8 tiles, 4096 x 14336 43.8 against 49.1, 4096 x 4096 the same 33)
    const bool f16_from_33 = F::F16_TILES && nrows_x >= 2048 && !lk_env_flag("LK_MMQ_I8");
    if ((ncols_y <= 64 && !f16_from_33) || F::MIN_RANK == 16) return launch_dense_tm<F, 64, 2>(pb, s, fixup);
    if constexpr (F::F16_TILES) {   // Q4_K: scales folded into f16 operands
        // (under 2048 weight rows the 256-row f16 tiles are too few even with K cut: 1024 x 4096 at 512 / 1024 /
        // 2048 rows 48 / 63 / 93 us against 38 / 49 / 73 on the int8 tiles)
        if (!lk_env_flag("LK_MMQ_I8") && nrows_x >= 2048) {
            // 128-token tiles with the token side expanded once per call, where they pad the rows at most a
            // tenth more than the 64-token tiles would (512 x 4096 -> 14336: 105 us against 123) and are
            // enough to occupy half the CUs (fewer: the 64-token tiles, which can cut K)
            const int64_t pad128 = (ncols_y + 127) / 128 * 128, pad64 = (ncols_y + 63) / 64 * 64;
            const int64_t wide_tiles = (nrows_x + 255) / 256 * (pad128 / 128);
            if (ncols_y > 128 && 10 * pad128 <= 11 * pad64 && 2 * wide_tiles > lk_device().cus && !lk_env_flag("LK_MMQ_NO_WIDE")) {
                const int tm = lk_mmq_q4k_wide_dense(pb, s);
                if (tm >= 0) return tm;
            }
            const int tm = lk_mmq_q4k_f16_dense(pb, s, fixup);
            if (tm >= 0) return tm;
        }
    }
    // 128-token tiles where there are F::WIDE_FROM of them or more, else 64-token tiles, twice as many and
    // with K cut where those are still few. Quantizer + matmul, 64- against 128-token tiles:
    //   Q6_K  4096 x 14336 at 128 / 512 / 1024 rows (32 / 128 / 256 tiles) 70 / 215 / 393 us against 99 / 307 /
    //         577, at 2048 rows (512) 724 against 639; 14336 x 4096 at 384 rows (336) 182 against 196, at 512
    //         (448) 211 against 197. Q5_K and Q3_K alike.
    //   Q4_0  14336 x 4096 at 256 rows (224) 115 against 120, at 384 (336) 178 against 155
    //   Q8_0  4096 x 4096 at 256 rows (64) 61.5 against 62.1, at 384 (96) 92 against 87, at 2048 (512) 299 against 190
    // LK_TUNE_MMQ_TM = 64 / 128 forces one in measurement runs.
    const int forced_tm = lk_tune_env("LK_TUNE_MMQ_TM");
    const int64_t tiles128 = (nrows_x + TN - 1) / TN * ((ncols_y + 127) / 128);
    if (forced_tm == 64 || (forced_tm != 128 && tiles128 < F::WIDE_FROM)) return launch_dense_tm<F, 64, 2>(pb, s, fixup);
    // 128-token tile: a wave takes all four token tiles of one 32-row weight tile (measured against
    // a 2 x 2 patch per wave: Q4_K 366 against 334 TOP/s at 512 rows, 434 against 364 at 2048;
    // Q6_K 320 against 313; Q8_0 305 against 304)
    constexpr int WAVES_M = 1;
    return launch_dense_tm<F, 128, WAVES_M>(pb, s, fixup);
}

template <class F, int TM, int WAVES_M>
static int launch_moe_tm(const MmqProblem& pb, const uint8_t* w_second, int64_t dst_second,
                         const int32_t* bounds, int64_t stride_expert, int n_experts, int64_t ncols_max,
                         hipStream_t s) {
    auto kernel = mmq_moe_kernel<F, TM, WAVES_M>;
    constexpr int lds_bytes = mmq_lds_bytes<F, TM>();
    if (mmq_prepare_kernel(kernel, lds_bytes) != LK_OK) return 0;
    const int64_t col_tiles = (ncols_max + TM - 1) / TM;
    const dim3 grid((pb.n + TN - 1) / TN, (unsigned)(col_tiles < 1 ? 1 : (col_tiles > 65535 ? 65535 : col_tiles)),
                    (unsigned)((w_second ? 2 : 1) * n_experts));
    hipLaunchKernelGGL(kernel, grid, dim3(MMQ_WG), lds_bytes, s, pb, w_second, dst_second, bounds,
                       stride_expert, n_experts);
    return hipGetLastError() == hipSuccess ? TM : 0;
}

template <class F>
static int launch_moe(const void* x, const void* x_second, int64_t dst_second, const void* y, void* dst,
                      const int* expert_bounds, const int* ids_dst, int64_t stride_expert_x,
                      int64_t ncols_x, int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                      int64_t stride_col_dst, int n_experts, int64_t ncols_max, int64_t ncols_hint,
                      int mmq_x, void* stream) {
    if (!x || !y || !dst || !expert_bounds || ncols_x <= 0 || nrows_x <= 0 || ncols_y <= 0 || n_experts <= 0) return 0;
    if ((uintptr_t)x % F::ALIGN != 0 || (uintptr_t)x_second % F::ALIGN != 0 || stride_expert_x % F::ALIGN != 0) return 0;
    if (ncols_x % 256 != 0 || stride_row_x < ncols_x / 256 * F::BLOCKS_PER_STEP) return 0;
    if (nrows_x > INT32_MAX || ncols_y > INT32_MAX || (int64_t)n_experts * 2 > 65535) return 0;
    MmqProblem pb{(const uint8_t*)x, (const uint8_t*)y, (float*)dst, ids_dst, ncols_x / 256, stride_row_x,
                  ncols_y, stride_col_dst, (int)nrows_x, 0, 0};
    hipStream_t s = (hipStream_t)stream;
    const uint8_t* w2 = (const uint8_t*)x_second;
    // the narrowest tile at or above what was asked for, else one sized for the expected run
    const int64_t want = mmq_x > 0 ? mmq_x : (ncols_hint > 0 ? ncols_hint : ncols_max);
    if (want <= 32) return launch_moe_tm<F, 32, 1>(pb, w2, dst_second, expert_bounds, stride_expert_x, n_experts, ncols_max, s);
    if (want <= 64) return launch_moe_tm<F, 64, 2>(pb, w2, dst_second, expert_bounds, stride_expert_x, n_experts, ncols_max, s);
    // The 128-token tile of this kernel (the routing's bounds and destination map on top of the dense
    // tile's registers) runs out of registers for the formats with a minimum or two scales per sub-block
    // and loses to the 64-token tile: 128 experts of 2048 -> 768 -> 2048, top-8, gate + up and down,
    // 2048 tokens: Q6_K 954 us against 1352, Q5_K 739 against 1231; 4096 tokens: 1608 against 1991, 1297
    // against 1787 (Q8_0 and Q4_0 go either way by a tenth and keep the wide tile).
    if constexpr (!F::F16_TILES && (F::HAS_MIN || F::NS == 16))
        return launch_moe_tm<F, 64, 2>(pb, w2, dst_second, expert_bounds, stride_expert_x, n_experts, ncols_max, s);
    else {
        // Left to choose (no mmq_x), the narrower tile where it pads the expected longest run a fifth
        // less: a run of 150 rows is three tiles of 64 or two of 128, the second nearly empty (2048
        // tokens, as above: Q8_0 1198 us against 1300, Q4_0 742 against 983; at 1024 and 4096 tokens the
        // runs fill the wide tiles and those win by a tenth).
        if (!F::F16_TILES && mmq_x <= 0 && 5 * ((want + 63) / 64 * 64) <= 4 * ((want + 127) / 128 * 128))
            return launch_moe_tm<F, 64, 2>(pb, w2, dst_second, expert_bounds, stride_expert_x, n_experts, ncols_max, s);
        if constexpr (F::F16_TILES) {
            if (!lk_env_flag("LK_MMQ_I8")) {
                const int tm = lk_mmq_q4k_f16_moe(pb, w2, dst_second, expert_bounds, stride_expert_x, n_experts, ncols_max, s);
                if (tm >= 0) return tm;
            }
        }
        constexpr int WAVES_M = 1;
        return launch_moe_tm<F, 128, WAVES_M>(pb, w2, dst_second, expert_bounds, stride_expert_x, n_experts, ncols_max, s);
    }
}

}  // namespace

int lk_mmq_split_sum(const float* part, int splits, const MmqProblem& pb, hipStream_t s) {
    const int64_t count = (int64_t)pb.m_end * pb.n;
    hipLaunchKernelGGL(mmq_split_sum_kernel, dim3((unsigned)((count / 4 + 255) / 256)), dim3(256), 0, s, part, splits, count,
                       pb.dst, count, pb.n, pb.ldd);
    return lk_launch_status();
}

extern "C" void launch_mmq_quantize_q8_1_D4(const void* x, const int32_t* ids, void* vy, int type_x,
                                            int64_t ne00, int64_t s01, int64_t s02, int64_t s03,
                                            int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3, void* stream) {
    launch_quantize(x, ids, vy, type_x, ne00, s01, s02, s03, ne0, ne1, ne2, ne3, stream);
}

extern "C" void launch_mmq_quantize_q8_1_DS4(const void* x, const int32_t* ids, void* vy, int type_x,
                                             int64_t ne00, int64_t s01, int64_t s02, int64_t s03,
                                             int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3, void* stream) {
    launch_quantize(x, ids, vy, type_x, ne00, s01, s02, s03, ne0, ne1, ne2, ne3, stream);
}

extern "C" void launch_mmq_quantize_q8_1_D2S6(const void* x, const int32_t* ids, void* vy, int type_x,
                                              int64_t ne00, int64_t s01, int64_t s02, int64_t s03,
                                              int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3, void* stream) {
    launch_quantize(x, ids, vy, type_x, ne00, s01, s02, s03, ne0, ne1, ne2, ne3, stream);
}

extern "C" int launch_mmq_gguf_q4_k(void* tmp_fixup, const void* x, const void* y, void* dst,
                                    int64_t ncols_x, int64_t nrows_x, int64_t ncols_y,
                                    int64_t stride_row_x, int64_t stride_col_dst, int cc, int nsm,
                                    int64_t smpbo, int warp_size, void* stream) {
    (void)cc; (void)nsm; (void)smpbo; (void)warp_size;
    return launch_dense<MmqQ4K>(tmp_fixup, x, y, dst, ncols_x, nrows_x, ncols_y, stride_row_x, stride_col_dst, stream);
}

extern "C" int launch_mmq_gguf_q5_k(void* tmp_fixup, const void* x, const void* y, void* dst,
                                    int64_t ncols_x, int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x,
                                    int64_t stride_col_dst, int cc, int nsm, int64_t smpbo, int warp_size,
                                    void* stream) {
    (void)cc; (void)nsm; (void)smpbo; (void)warp_size;
    return launch_dense<MmqQ5K>(tmp_fixup, x, y, dst, ncols_x, nrows_x, ncols_y, stride_row_x, stride_col_dst, stream);
}

extern "C" int launch_mmq_gguf_q6_k(void* tmp_fixup, const void* x, const void* y, void* dst,
                                    int64_t ncols_x, int64_t nrows_x, int64_t ncols_y,
                                    int64_t stride_row_x, int64_t stride_col_dst, int cc, int nsm,
                                    int64_t smpbo, int warp_size, void* stream) {
    (void)cc; (void)nsm; (void)smpbo; (void)warp_size;
    return launch_dense<MmqQ6K>(tmp_fixup, x, y, dst, ncols_x, nrows_x, ncols_y, stride_row_x, stride_col_dst, stream);
}

extern "C" int launch_mmq_gguf_q8_0(void* tmp_fixup, const void* x, const void* y, void* dst,
                                    int64_t ncols_x, int64_t nrows_x, int64_t ncols_y,
                                    int64_t stride_row_x, int64_t stride_col_dst, int cc, int nsm,
                                    int64_t smpbo, int warp_size, void* stream) {
    (void)cc; (void)nsm; (void)smpbo; (void)warp_size;
    return launch_dense<MmqQ80>(tmp_fixup, x, y, dst, ncols_x, nrows_x, ncols_y, stride_row_x, stride_col_dst, stream);
}

#define LK_MMQ_DENSE_ENTRY(NAME, FMT)                                                                   \
    extern "C" int NAME(void* tmp_fixup, const void* x, const void* y, void* dst, int64_t ncols_x,     \
                        int64_t nrows_x, int64_t ncols_y, int64_t stride_row_x, int64_t stride_col_dst, \
                        int cc, int nsm, int64_t smpbo, int warp_size, void* stream) {                 \
        (void)cc; (void)nsm; (void)smpbo; (void)warp_size;                            \
        return launch_dense<FMT>(tmp_fixup, x, y, dst, ncols_x, nrows_x, ncols_y, stride_row_x, stride_col_dst, stream); \
    }

LK_MMQ_DENSE_ENTRY(launch_mmq_gguf_q4_0, MmqQ40)
LK_MMQ_DENSE_ENTRY(launch_mmq_gguf_q4_1, MmqQ41)
LK_MMQ_DENSE_ENTRY(launch_mmq_gguf_q5_0, MmqQ50)
LK_MMQ_DENSE_ENTRY(launch_mmq_gguf_q5_1, MmqQ51)
LK_MMQ_DENSE_ENTRY(launch_mmq_gguf_q3_k, MmqQ3K)
LK_MMQ_DENSE_ENTRY(launch_mmq_gguf_q2_k, MmqQ2K)

#define LK_MMQ_MOE_ENTRY(NAME, FMT)                                                                     \
    extern "C" int NAME(const void* x, const void* x_second, int64_t dst_second, const void* y,        \
                        void* dst, const int* expert_bounds, const int* ids_dst,                       \
                        int64_t stride_expert_x, int64_t ncols_x, int64_t nrows_x, int64_t ncols_y,    \
                        int64_t stride_row_x, int64_t stride_col_dst, int n_experts, int64_t ncols_max, \
                        int64_t ncols_hint, int mmq_x, int cc, int64_t smpbo, int warp_size,           \
                        void* stream) {                                                                \
        (void)cc; (void)smpbo; (void)warp_size;                                                        \
        return launch_moe<FMT>(x, x_second, dst_second, y, dst, expert_bounds, ids_dst, stride_expert_x, \
                               ncols_x, nrows_x, ncols_y, stride_row_x, stride_col_dst, n_experts,     \
                               ncols_max, ncols_hint, mmq_x, stream);                                  \
    }

LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q4_k, MmqQ4K)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q5_k, MmqQ5K)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q6_k, MmqQ6K)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q8_0, MmqQ80)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q4_0, MmqQ40)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q4_1, MmqQ41)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q5_0, MmqQ50)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q5_1, MmqQ51)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_iq4_nl, MmqIq4Nl)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_mxfp4, MmqMxfp4)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q3_k, MmqQ3K)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_iq4_xs, MmqIq4Xs)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q2_k, MmqQ2K)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_iq3_xxs, MmqIq3Xxs)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_iq3_s, MmqIq3S)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_iq2_s, MmqIq2S)
LK_MMQ_MOE_ENTRY(launch_mmq_moe_gguf_q2_0, MmqQ2_0)

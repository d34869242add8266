// Q4_K weight rows against 129 or more Q8_1 token rows: the f16-operand tiles of mmq_q4k_f16.hip
// with four token tiles per wave and every byte delivered to LDS without passing through registers.
//
//   out[token, n] = sum over 256-value blocks of
//        d[n] * sum_s d8_s[token] * D_s[n, token]  -  dmin[n] * sum_s m_s[n] * (d8_s * S_s)[token]
//   D_s[n, token] = sum over the 32 values of sub-block s of (sc_s[n] * q[n, k]) * a[token, k]
//
// The arithmetic is that of mmq_q4k_f16.hip, operation for operation (sc * q and the int8 codes are
// exact in f16, D_s is an exact integer in the f32 accumulator, one fma by the token's d8 per element
// and sub-block in ascending s, the block's d and dmin applied once per 256 values with the minimum
// term as a rank-8 update on the bf16 matrix unit), so both kernels return the same bits: the integer
// sub-block dots of loken's BlockQ4K::dot_scalar (src/tensor/quant_cpu/format/q4_k.rs:62-88, 138-153)
// combined as cuda/moe/gguf.cuh:664-713 combines them.
//
// What differs is where the vector unit's time goes. That unit issues both the matrix instructions
// and everything else, and the per-sub-block fma is 16 vector instructions against two matrix
// instructions, so the kernel is bound by vector issue and every other vector instruction counts:
//   * the token side is expanded ONCE per call by `q4k_tokens_f16_kernel` into operand order (f16
//     codes, f32 scales, the bf16 pieces of d8 * S): 74 KiB per (128-token tile, block), in memory
//     the library keeps per stream. The tile kernel then spends nothing on tokens.
//   * a wave owns 32 weight rows x 128 tokens (four tiles of v_mfma_f32_32x32x16_f16, registers <->
//     weight rows, lanes <-> tokens), so the nibble expansion of its rows is shared by four token
//     tiles instead of two.
//   * token quarters (two sub-blocks), the weight nibbles (four planes of 32 bytes per row), the
//     block headers and the per-block token tables reach LDS through global_load_lds_dwordx4: no
//     staging registers, no address arithmetic per byte, no ds_write. A ring of four quarters keeps
//     loads three quarters ahead of their use; a wave waits only for loads issued before the quarter
//     it is in, then the workgroup meets at one barrier per quarter.
//   * the 32 items (sub-block, token tile) of a block run as one software pipeline that does not
//     stop at block or quarter boundaries: LDS reads of item i + 1, the two matrix instructions of
//     item i, the 16 fmas of item i - 1 between and after them, the next sub-block's operand
//     expansion and the previous block's d / dmin update spread over the slots.

#include "mmq_problem.h"

#include <mutex>
#include <utility>
#include <vector>

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

static __device__ __forceinline__ h2 as_h2(uint32_t bits) { return __builtin_bit_cast(h2, bits); }
static __device__ __forceinline__ uint32_t h2_bits(h2 v) { return __builtin_bit_cast(uint32_t, v); }

struct Wd {
    static constexpr int WAVES = 8, THREADS = 64 * WAVES;
    static constexpr int TN = 32 * WAVES, TM = 128, TT = 4;
    static constexpr int TCH = 16 / WAVES;                   // 1 KiB chunks of a token quarter per wave
    static constexpr int RCH = (10 + WAVES - 1) / WAVES;      // of the per-block tables
    static constexpr int HW = WAVES / 2;                      // waves that cover the headers once
    static constexpr int QB = 2 * 4 * TM * 16;              // one quarter: two sub-blocks of f16 codes
    static constexpr int D8B = 8 * TM * 4;                  // d8 [s][token] f32
    static constexpr int REGION = D8B + 3 * TM * 16;        // + hi | mid | lo planes of d8 * S
    static constexpr int UNIT = 4 * QB + REGION;            // one (token tile, block)
    static constexpr int WPB = TN * 32;                     // one nibble plane
    static constexpr int T_AT = 0;                          // ring of four quarters: quarter q lives in slot q
    static constexpr int WP_AT = T_AT + 4 * QB;
    static constexpr int H_AT = WP_AT + 4 * WPB;
    static constexpr int R_AT = H_AT + TN * 16;             // two regions (block parity)
    static constexpr int WD_AT = R_AT + 2 * REGION;         // per wave and block parity: d, -dmin of its 32 rows
    static constexpr int LDS = WD_AT + WAVES * 2 * 256;
};
static_assert(Wd::LDS <= 160 * 1024, "LDS of one CU");
static_assert(Wd::QB == 16 * 1024 && Wd::REGION == 10 * 1024, "chunks of 1 KiB per wave load");

// ------------------------------------------------------------------ token side, once per call
// grid (blocks, token tiles), 256 threads: thread = (token, half of the block's sub-blocks).
__global__ __launch_bounds__(256) void q4k_tokens_f16_kernel(const uint8_t* __restrict__ y, uint8_t* __restrict__ out,
                                                            int64_t rows_total, int m_begin, int m_end, int nb) {
    const int kb = blockIdx.x, tile = blockIdx.y;
    const int token = threadIdx.x & 127, hh = threadIdx.x >> 7;
    const int row = m_begin + tile * Wd::TM + token;
    const bool live = row < m_end;
    uint8_t* unit = out + ((int64_t)tile * nb + kb) * Wd::UNIT;
    const uint8_t* rec = y + ((int64_t)kb * rows_total + (live ? row : m_begin)) * MMQ_REC_BYTES;
    const uint4 dw = *(const uint4*)(rec + 256);   // eight f16 scales
    const uint32_t dbits[4] = {dw.x, dw.y, dw.z, dw.w};
    const h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
#pragma unroll
    for (int si = 0; si < 4; ++si) {
        const int s = 4 * hh + si;
        uint8_t* quarter = unit + (s >> 1) * Wd::QB + (s & 1) * 4 * Wd::TM * 16;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint4 c = *(const uint4*)(rec + 32 * s + 16 * h);
            if (!live) c = make_uint4(0, 0, 0, 0);
            const uint32_t cw[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                // four int8 codes -> f16 as the byte pairs (0, 2) and (1, 3), the order the weight side
                // unpacks its nibbles in: byte ^ 0x80 = code + 128, OR-ed into the mantissa of 1024.0
                uint32_t o[4];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const uint32_t u = cw[2 * hf + e];
                    o[2 * e] = h2_bits(as_h2((u & 0x00FF00FFu) ^ 0x64806480u) - bias);
                    o[2 * e + 1] = h2_bits(as_h2(((u >> 8) & 0x00FF00FFu) ^ 0x64806480u) - bias);
                }
                *(uint4*)(quarter + ((hf * 2 + h) * Wd::TM + token) * 16) = make_uint4(o[0], o[1], o[2], o[3]);
            }
        }
        const float d8 = live ? f16_bits_to_f32((dbits[s >> 1] >> (16 * (s & 1))) & 0xFFFFu) : 0.f;
        *(float*)(unit + 4 * Wd::QB + (s * Wd::TM + token) * 4) = d8;
    }
    if (hh == 0) {
        // d8 * S as three bf16 (truncations of the running remainder: 8 bits each, nothing lost)
        const uint4 sw = *(const uint4*)(rec + 272);
        const uint32_t sbits[4] = {sw.x, sw.y, sw.z, sw.w};
        uint16_t piece[3][8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const float d8 = live ? f16_bits_to_f32((dbits[s >> 1] >> (16 * (s & 1))) & 0xFFFFu) : 0.f;
            const int sum = (int)(int16_t)((sbits[s >> 1] >> (16 * (s & 1))) & 0xFFFFu);
            const float p0 = d8 * (float)sum;
            const uint32_t b0 = __float_as_uint(p0) & 0xFFFF0000u;
            const float p1 = p0 - __uint_as_float(b0);
            const uint32_t b1 = __float_as_uint(p1) & 0xFFFF0000u;
            const float p2 = p1 - __uint_as_float(b1);
            piece[0][s] = (uint16_t)(b0 >> 16);
            piece[1][s] = (uint16_t)(b1 >> 16);
            piece[2][s] = (uint16_t)(__float_as_uint(p2) >> 16);
        }
        uint8_t* planes = unit + 4 * Wd::QB + Wd::D8B + token * 16;
#pragma unroll
        for (int pc = 0; pc < 3; ++pc)
            *(uint4*)(planes + pc * Wd::TM * 16) =
                make_uint4(piece[pc][0] | (uint32_t)piece[pc][1] << 16, piece[pc][2] | (uint32_t)piece[pc][3] << 16,
                           piece[pc][4] | (uint32_t)piece[pc][5] << 16, piece[pc][6] | (uint32_t)piece[pc][7] << 16);
    }
}

// ------------------------------------------------------------------ weight side
// 64 lanes x 16 bytes from global memory straight into LDS: uniform base + the lane's 32-bit
// offset on the global side; lane i's bytes land at wave_base + 16 i.
static __device__ __forceinline__ void to_lds16(const uint8_t* base, uint32_t lane_off, uint8_t* wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + lane_off),
                                     (__attribute__((address_space(3))) void*)wave_base, 16, 0, 0);
}

// This wave's LDS reads are done and every load it issued before its latest `KEEP` has landed; then
// the workgroup's barrier. The memory clobber keeps the compiler from moving LDS accesses across it.
template <int KEEP>
static __device__ __forceinline__ void meet() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(KEEP) : "memory");
}

// 6-bit scale / min of sub-block S from the header's packed words (get_scale_min_k4 of the format)
template <int S>
static __device__ __forceinline__ uint32_t q4k_scale(uint32_t w1, uint32_t w3) {
    if constexpr (S < 4) return (w1 >> (8 * S)) & 63u;
    else return ((w3 >> (8 * (S - 4))) & 0xFu) | (((w1 >> (8 * (S - 4) + 6)) & 3u) << 4);
}
template <int S>
static __device__ __forceinline__ uint32_t q4k_min(uint32_t w2, uint32_t w3) {
    if constexpr (S < 4) return (w2 >> (8 * S)) & 63u;
    else return ((w3 >> (8 * (S - 4) + 4)) & 0xFu) | (((w2 >> (8 * (S - 4) + 6)) & 3u) << 4);
}

// A operand `HF` of sub-block S from the lane's 16 nibble bytes of the pair: (1024 + q) * sc - 1024 * sc
// for the low nibbles; the high nibbles sit four bits up, (1024 + 16 q) * (sc / 16) - 64 * sc. Exact in f16.
template <int S, int HF>
static __device__ __forceinline__ v8h weight_operand(const uint4& q, uint32_t w1, uint32_t w3, uint32_t h1024) {
    constexpr bool HIGH = (S & 1) != 0;
    const float sc = (float)q4k_scale<S>(w1, w3);
    const _Float16 scale = (_Float16)(sc * (HIGH ? 0.0625f : 1.0f));
    const _Float16 offset = (_Float16)(sc * (HIGH ? -64.0f : -1024.0f));
    const h2 scale2 = {scale, scale}, offset2 = {offset, offset};
    constexpr uint32_t mask = HIGH ? 0x00F000F0u : 0x000F000Fu;
    const uint32_t u[4] = {q.x, q.y, q.z, q.w};
    uint32_t ab[4];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const uint32_t x = u[2 * HF + e];
        ab[2 * e] = h2_bits(__builtin_elementwise_fma(as_h2((x & mask) | h1024), scale2, offset2));
        ab[2 * e + 1] = h2_bits(__builtin_elementwise_fma(as_h2(((x >> 8) & mask) | h1024), scale2, offset2));
    }
    return __builtin_bit_cast(v8h, make_uint4(ab[0], ab[1], ab[2], ab[3]));
}

// What a wave carries through the pipeline. Every index into the arrays below is a compile-time
// constant (the slots are template instances), so all of it lives in registers.
struct WideWave {
    // global -> LDS: uniform bases that move with the block, lane offsets that do not
    const uint8_t* tok_base;      // + block * UNIT + quarter * QB (+ 1024)
    const uint8_t* region_base;   // + block * UNIT + chunk * 1024
    const uint8_t* w_base;        // + block * 144 (+ 16 + 32 * plane)
    uint32_t lane16, nib_off, hdr_off;
    int wave;
    uint8_t* lds;
    // LDS addresses of this lane
    const uint8_t* wp;   // its 16 nibble bytes in plane 0 (+ plane * WPB)
    const uint8_t* hp;   // its row's header
    const uint8_t* tb;   // its atom of token tile 0 (+ quarter * QB + sub-block, K half, tile)
    const uint8_t* rp;   // its token's d8 (+ parity * REGION + (s * TM + 32 tt) * 4)
    const uint8_t* mp;   // its token's d8 * S pieces (+ parity * REGION + plane * 2048 + tt * 512)
    float* wd;           // the wave's table (+ parity * 64): [0, 32) d, [32, 64) -dmin of its rows
    int h, j;

    v16f acc[4], part[4], dot[2];
    v8h a[2], b[2][2];
    float d8v[4];
    uint4 nib;
    uint32_t w1, w2, w3, w1n, w2n, w3n;   // header words: this block's scales and mins; the next block's
    v8bf m_op;                            // the mins of the block being folded, as a bf16 operand
    uint32_t h1024;

    __device__ __forceinline__ void load_quarter(int kb, int q) const {
        const uint8_t* from = tok_base + (int64_t)kb * Wd::UNIT + q * Wd::QB;
        uint8_t* to = lds + Wd::T_AT + wave * (Wd::TCH * 1024) + q * Wd::QB;
#pragma unroll
        for (int c = 0; c < Wd::TCH; ++c) to_lds16(from + c * 1024, lane16, to + c * 1024);
    }
    __device__ __forceinline__ void load_plane(int kb, int plane) const {
        to_lds16(w_base + (int64_t)kb * Q4K_BYTES + 32 * plane, nib_off, lds + Wd::WP_AT + wave * 1024 + plane * Wd::WPB);
    }
    __device__ __forceinline__ void load_headers(int kb) const {
        to_lds16(w_base + (int64_t)kb * Q4K_BYTES, hdr_off, lds + Wd::H_AT + (wave % Wd::HW) * 1024);
    }
    __device__ __forceinline__ void load_region(int kb) const {
        const uint8_t* from = region_base + (int64_t)kb * Wd::UNIT;
        uint8_t* to = lds + Wd::R_AT + (kb & 1) * Wd::REGION;
#pragma unroll
        for (int c = 0; c < Wd::RCH; ++c) {
            const int chunk = min(wave + c * Wd::WAVES, 9);
            to_lds16(from + chunk * 1024, lane16, to + chunk * 1024);
        }
    }

    // Item I of a block: sub-block I / 4, token tile I % 4.
    template <int I>
    __device__ __forceinline__ void load_item(int parity) {
        constexpr int s = I / 4, tt = I % 4;
        const uint8_t* at = tb + (s >> 1) * Wd::QB + (s & 1) * (4 * Wd::TM * 16) + tt * 512;
        b[I & 1][0] = *(const v8h*)(at);
        b[I & 1][1] = *(const v8h*)(at + 2 * Wd::TM * 16);
        d8v[I & 3] = *(const float*)(rp + parity * Wd::REGION + (s * Wd::TM + 32 * tt) * 4);
    }
    static __device__ __forceinline__ v8bf mins_operand(uint32_t x2, uint32_t x3) {
        const float m0f = (float)q4k_min<0>(x2, x3), m1f = (float)q4k_min<1>(x2, x3), m2f = (float)q4k_min<2>(x2, x3),
                    m3f = (float)q4k_min<3>(x2, x3), m4f = (float)q4k_min<4>(x2, x3), m5f = (float)q4k_min<5>(x2, x3),
                    m6f = (float)q4k_min<6>(x2, x3), m7f = (float)q4k_min<7>(x2, x3);
        // small integers as bf16: the top half of their f32
        return __builtin_bit_cast(v8bf, make_uint4((__float_as_uint(m0f) >> 16) | (__float_as_uint(m1f) & 0xFFFF0000u),
                                                   (__float_as_uint(m2f) >> 16) | (__float_as_uint(m3f) & 0xFFFF0000u),
                                                   (__float_as_uint(m4f) >> 16) | (__float_as_uint(m5f) & 0xFFFF0000u),
                                                   (__float_as_uint(m6f) >> 16) | (__float_as_uint(m7f) & 0xFFFF0000u)));
    }
    // acc += d * part - dmin * (m . d8 S) for token tile TTU of the block whose tables sit at `parity`
    template <int TTU>
    __device__ __forceinline__ void fold_block(int parity) {
        const uint8_t* planes = mp + parity * Wd::REGION + TTU * 512;
        const uint4 hm = *(const uint4*)(planes + h * 2048);   // K slots 0..7 hi, 8..15 mid
        uint4 lz = *(const uint4*)(planes + 2 * 2048);         // K slots 0..7 lo, the rest nothing
        if (h) lz = make_uint4(0, 0, 0, 0);
        v16f mins = {0.f};
        mins = __builtin_amdgcn_mfma_f32_32x32x16_bf16(m_op, __builtin_bit_cast(v8bf, hm), mins, 0, 0, 0);
        mins = __builtin_amdgcn_mfma_f32_32x32x16_bf16(m_op, __builtin_bit_cast(v8bf, lz), mins, 0, 0, 0);
        const float* tab = wd + parity * 64 + 4 * h;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 dv = *(const float4*)(tab + 8 * g);
            const float4 nd = *(const float4*)(tab + 32 + 8 * g);
            acc[TTU][4 * g + 0] = fmaf(nd.x, mins[4 * g + 0], fmaf(dv.x, part[TTU][4 * g + 0], acc[TTU][4 * g + 0]));
            acc[TTU][4 * g + 1] = fmaf(nd.y, mins[4 * g + 1], fmaf(dv.y, part[TTU][4 * g + 1], acc[TTU][4 * g + 1]));
            acc[TTU][4 * g + 2] = fmaf(nd.z, mins[4 * g + 2], fmaf(dv.z, part[TTU][4 * g + 2], acc[TTU][4 * g + 2]));
            acc[TTU][4 * g + 3] = fmaf(nd.w, mins[4 * g + 3], fmaf(dv.w, part[TTU][4 * g + 3], acc[TTU][4 * g + 3]));
            // one pair of table rows at a time, used where it is read (left to itself the instruction
            // selector reads all of them ahead and sinks the fmas to the block's end, through spills)
            asm volatile("" : "+v"(acc[TTU][4 * g]), "+v"(acc[TTU][4 * g + 1]), "+v"(acc[TTU][4 * g + 2]), "+v"(acc[TTU][4 * g + 3]));
        }
    }
    __device__ __forceinline__ void read_header(uint32_t& x1, uint32_t& x2, uint32_t& x3, int parity) {
        const uint4 t = *(const uint4*)hp;
        x1 = t.y; x2 = t.z; x3 = t.w;
        if (h == 0) {
            wd[parity * 64 + j] = f16_bits_to_f32(t.x & 0xFFFFu);
            wd[parity * 64 + 32 + j] = -f16_bits_to_f32(t.x >> 16);
        }
    }

    template <int Q>
    static constexpr int loads_in() { return Wd::TCH + 1 + (Q == 0 ? 1 : Q == 1 ? Wd::RCH : 0); }

    // Slot I of block kb. A wave's vector instructions issue under its own matrix instruction only when
    // they do not wait for it, so the 16 fmas of item I - 1 sit behind the two matrix instructions of
    // item I (the second takes the first one's result as its accumulator and cannot issue before that
    // is written: eight fmas fill exactly that gap), with this slot's share of the other work.
    template <int I>
    __device__ __forceinline__ void slot(int kb, int next) {
        constexpr int s = I / 4, tt = I % 4, q = I / 8;
        constexpr int P = (I + 31) & 31, pt = P % 4, ps = P / 4;   // the item before (the previous block's last for I = 0)
        const int par = kb & 1;
        if constexpr (I % 8 == 7) {
            // everything issued before the previous quarter has landed (nothing is read sooner than three
            // quarters after its load was issued); the last two quarters' loads stay in flight
            meet<loads_in<q>() + loads_in<(q + 3) & 3>()>();
        }
        if constexpr (I % 8 == 0) {
            // the quarter three ahead into the ring slot the last barrier released, the plane the
            // previous quarter read for the last time, and once per block the next headers and tables
            load_quarter(q == 0 ? kb : next, (q + 3) & 3);
            load_plane(next, q);
            if constexpr (q == 0) load_headers(next);
            if constexpr (q == 1) load_region(next);
        }
        if constexpr (I == 24) read_header(w1n, w2n, w3n, par ^ 1);
        // the next item's operands: a slot ahead of their use, which is what an LDS read takes here
        if constexpr (I < 31) load_item<I + 1>(par);
        else load_item<0>(par ^ 1);
        // the pair after this one, into the nibble registers whose last use was the expansion a sub-block ago
        if constexpr (tt == 1 && (s & 1)) nib = *(const uint4*)(wp + (((s + 1) >> 1) & 3) * Wd::WPB);
        {
            const v16f zero = {0.f};
            dot[I & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[0], b[I & 1][0], zero, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        {
            const float d8p = d8v[P & 3];
#pragma unroll
            for (int v = 0; v < 8; ++v) part[pt][v] = ps == 0 ? dot[P & 1][v] * d8p : fmaf(dot[P & 1][v], d8p, part[pt][v]);
        }
        __builtin_amdgcn_sched_barrier(0);
        dot[I & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[1], b[I & 1][1], dot[I & 1], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        {
            const float d8p = d8v[P & 3];
#pragma unroll
            for (int v = 8; v < 16; ++v) part[pt][v] = ps == 0 ? dot[P & 1][v] * d8p : fmaf(dot[P & 1][v], d8p, part[pt][v]);
        }
        // the next sub-block's operands, over the ones its last item has just used
        if constexpr (tt == 3) {
            const uint32_t x1 = s == 7 ? w1n : w1, x3 = s == 7 ? w3n : w3;
            a[0] = weight_operand<(s + 1) & 7, 0>(nib, x1, x3, h1024);
            a[1] = weight_operand<(s + 1) & 7, 1>(nib, x1, x3, h1024);
        }
        // the previous block's factors, one token tile per slot: tile I's sums were complete by slot 0
        // and slot I + 1 re-starts them (before the first block: tables of zeros)
        if constexpr (I < 4) fold_block<I>(par ^ 1);
        if constexpr (I == 5) m_op = mins_operand(w2, w3);
        if constexpr (I == 31) { w1 = w1n; w2 = w2n; w3 = w3n; }
        // Pins the slot's end for the instruction selector, which orders only what has side effects:
        // the previous item's sums are complete here and the next slot's matrix instructions start from
        // here, so no third set of results is ever alive.
        asm volatile("" : "+v"(part[pt]), "+v"(a[0]));
        __builtin_amdgcn_sched_barrier(0);
    }
    template <int... I>
    __device__ __forceinline__ void block(int kb, int next, std::integer_sequence<int, I...>) {
        (slot<I>(kb, next), ...);
    }
};

static __device__ __forceinline__ void wide_tile(const MmqProblem& pb, const uint8_t* __restrict__ units, int n0, int m0,
                                                 uint8_t* lds) {
    using C = Wd;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, h = lane >> 5;
    const int last = (int)pb.nb - 1;
    const int64_t row_bytes = pb.row_blocks * Q4K_BYTES;

    WideWave w;
    w.tok_base = units + wave * (C::TCH * 1024);
    w.region_base = units + 4 * C::QB;
    w.w_base = pb.w + (int64_t)n0 * row_bytes;
    w.lane16 = lane * 16;
    w.nib_off = (uint32_t)(min(32 * wave + (lane >> 1), pb.n - 1 - n0) * (int)row_bytes + 16 + 16 * (lane & 1));
    w.hdr_off = (uint32_t)(min(64 * (wave % C::HW) + lane, pb.n - 1 - n0) * (int)row_bytes);
    w.wave = wave;
    w.lds = lds;
    w.wp = lds + C::WP_AT + ((32 * wave + j) * 32 + 16 * h);
    w.hp = lds + C::H_AT + (32 * wave + j) * 16;
    w.tb = lds + C::T_AT + h * (C::TM * 16) + j * 16;
    w.rp = lds + C::R_AT + j * 4;
    w.mp = lds + C::R_AT + C::D8B + j * 16;
    w.wd = (float*)(lds + C::WD_AT) + wave * 128;
    w.h = h; w.j = j;
    w.w1n = w.w2n = w.w3n = 0;
#pragma unroll
    for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int v = 0; v < 16; ++v) { w.acc[tt][v] = 0.f; w.part[tt][v] = 0.f; }
    // the first block folds a block that was never there: its tables (parity 1) read as zeros
    for (int i = tid; i < 3 * C::TM; i += C::THREADS) *(uint4*)(lds + C::R_AT + C::REGION + C::D8B + i * 16) = make_uint4(0, 0, 0, 0);
    if (lane < 64) w.wd[64 + lane] = 0.f;
    w.h1024 = 0x64006400u;   // in a vector register: (x & mask) | h1024 is then one v_and_or_b32 with the mask as its literal
    asm volatile("" : "+v"(w.h1024));

    // prologue: three quarters, the four planes, the headers and the tables of block 0
    w.load_quarter(0, 0);
    w.load_quarter(0, 1);
    w.load_quarter(0, 2);
#pragma unroll
    for (int p = 0; p < 4; ++p) w.load_plane(0, p);
    w.load_headers(0);
    w.load_region(0);
    meet<0>();
    w.read_header(w.w1, w.w2, w.w3, 0);
    w.m_op = WideWave::mins_operand(w.w2, w.w3);
    w.nib = *(const uint4*)w.wp;
    w.load_item<0>(0);
    w.a[0] = weight_operand<0, 0>(w.nib, w.w1, w.w3, w.h1024);
    w.a[1] = weight_operand<0, 1>(w.nib, w.w1, w.w3, w.h1024);
#pragma unroll
    for (int v = 0; v < 16; ++v) w.dot[1][v] = 0.f;   // "the item before the first": zeros times zero
    w.d8v[3] = 0.f;
    meet<0>();   // the headers and plane 0 are reloaded from the first slot on

    for (int kb = 0; kb <= last; ++kb) w.block(kb, min(kb + 1, last), std::make_integer_sequence<int, 32>{});

    {
        const float d8p = w.d8v[3];
#pragma unroll
        for (int v = 0; v < 16; ++v) w.part[3][v] = fmaf(w.dot[1][v], d8p, w.part[3][v]);
    }
    w.fold_block<0>(last & 1);
    w.fold_block<1>(last & 1);
    w.fold_block<2>(last & 1);
    w.fold_block<3>(last & 1);

    const bool vec_ok = ((uintptr_t)pb.dst % 16 == 0) && (pb.ldd % 4 == 0);
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
        const int col = m0 + 32 * tt + j;
        if (col >= pb.m_end) continue;
        const int64_t drow = pb.ids_dst ? pb.ids_dst[col] : col;
        float* out = pb.dst + drow * pb.ldd;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int gn0 = n0 + 32 * wave + 8 * g + 4 * h;
            if (vec_ok && gn0 + 3 < pb.n) {
                *(float4*)(out + gn0) = make_float4(w.acc[tt][4 * g], w.acc[tt][4 * g + 1], w.acc[tt][4 * g + 2], w.acc[tt][4 * g + 3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (gn0 + e < pb.n) out[gn0 + e] = w.acc[tt][4 * g + e];
            }
        }
    }
}

// Workgroup id -> (m tile, n tile). Ids are dealt round robin over the 8 XCDs; an XCD's workgroups
// walk one contiguous eighth of the m-major tile list, so the CUs of an XCD share a token tile (about a
// megabyte of operand atoms at k = 4096: what its L2 holds) and stream the weights.
__global__ __launch_bounds__(Wd::THREADS, 1) void q4k_wide_dense_kernel(MmqProblem pb, const uint8_t* __restrict__ units,
                                                                       int n_tiles, int m_tiles, int per_xcd) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int id = blockIdx.x;
    const int t = (id & 7) * per_xcd + (id >> 3);
    if ((id >> 3) >= per_xcd || t >= n_tiles * m_tiles) return;
    const int m_tile = t / n_tiles, n_tile = t % n_tiles;
    wide_tile(pb, units + (int64_t)m_tile * pb.nb * Wd::UNIT, n_tile * Wd::TN, pb.m_begin + m_tile * Wd::TM, lds);
}

// ------------------------------------------------------------------ the units' memory
// Grow-only, one buffer per (device, stream), as the MoE decode launchers keep theirs; released by
// loken_stream_scratch_release. A call whose tokens need more than the cap runs in several passes
// of token tiles over the same buffer (stream order keeps them apart).
struct UnitSlot {
    int device;
    hipStream_t stream;
    void* ptr = nullptr;
    size_t size = 0;
    std::vector<void*> kept;   // outgrown buffers: queued kernels may still read them
};
std::mutex g_units_mu;
std::vector<UnitSlot> g_units;
constexpr size_t UNITS_CAP = (size_t)256 << 20;

void* reserve_units(size_t bytes, hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    UnitSlot* slot = nullptr;
    for (auto& s : g_units)
        if (s.device == dev && s.stream == stream) slot = &s;
    if (!slot) {
        g_units.push_back(UnitSlot{dev, stream});
        slot = &g_units.back();
    }
    if (slot->size >= bytes) return slot->ptr;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;   // growing allocates, which a recording stream may not do
    if (hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) return nullptr;
    (void)hipGetLastError();
    void* fresh = nullptr;
    const size_t want = (bytes + 255) & ~(size_t)255;
    if (hipMalloc(&fresh, want) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    if (slot->ptr) slot->kept.push_back(slot->ptr);
    slot->ptr = fresh;
    slot->size = want;
    return fresh;
}

}  // namespace

void lk_mmq_q4k_wide_release(int device) {
    std::lock_guard<std::mutex> lock(g_units_mu);
    for (auto it = g_units.begin(); it != g_units.end();) {
        if (it->device != device) { ++it; continue; }
        if (it->ptr) (void)hipFree(it->ptr);
        for (void* p : it->kept) (void)hipFree(p);
        it = g_units.erase(it);
    }
}

int lk_mmq_q4k_wide_dense(const MmqProblem& pb, hipStream_t s) {
    using C = Wd;
    if (((uintptr_t)pb.w | (uintptr_t)pb.y) % 16 != 0 || pb.nb < 1 || pb.nb > (1 << 20)) return -1;
    if (pb.row_blocks * Q4K_BYTES * 256 > (int64_t)INT32_MAX) return -1;   // lane offsets inside a tile are 32-bit
    if (mmq_prepare_kernel(q4k_wide_dense_kernel, C::LDS) != LK_OK) return -1;
    const int m = pb.m_end - pb.m_begin;
    const int m_tiles = (m + C::TM - 1) / C::TM;
    const int n_tiles = (pb.n + C::TN - 1) / C::TN;
    const size_t tile_bytes = (size_t)pb.nb * C::UNIT;
    if (tile_bytes > UNITS_CAP) return -1;
    const int tiles_per_pass = (int)std::min<size_t>((size_t)m_tiles, UNITS_CAP / tile_bytes);
    std::lock_guard<std::mutex> lock(g_units_mu);   // the buffer is the stream's from here until the launches are queued
    uint8_t* units = (uint8_t*)reserve_units(tile_bytes * tiles_per_pass, s);
    if (!units) return -1;
    for (int t0 = 0; t0 < m_tiles; t0 += tiles_per_pass) {
        const int tiles = std::min(tiles_per_pass, m_tiles - t0);
        MmqProblem part = pb;
        part.m_begin = pb.m_begin + t0 * C::TM;
        part.m_end = std::min(pb.m_end, part.m_begin + tiles * C::TM);
        hipLaunchKernelGGL(q4k_tokens_f16_kernel, dim3((unsigned)pb.nb, (unsigned)tiles), dim3(256), 0, s, pb.y, units,
                           pb.rows_total, part.m_begin, part.m_end, (int)pb.nb);
        const int total = tiles * n_tiles, per_xcd = (total + 7) / 8;
        hipLaunchKernelGGL(q4k_wide_dense_kernel, dim3(per_xcd * 8), dim3(C::THREADS), C::LDS, s, part, (const uint8_t*)units,
                           n_tiles, tiles, per_xcd);
        if (hipGetLastError() != hipSuccess) return 0;
    }
    return C::TM;
}

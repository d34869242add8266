// The 32-value nibble formats Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL and MXFP4 as the kernels read them: block
// layouts (src/tensor/quant_cpu/format/q4_0.rs, q4_1.rs, q5_0.rs, q5_1.rs), code expansion four codes to
// the dword, the table formats' levels, and the block scale. Shared by the mat-vec and the tile kernels.
#pragma once

#include "lk_common.h"

namespace {

// TABLE: 0 = the code is the value (less BIAS); 1 = IQ4_NL's levels; 2 = MXFP4's levels, E8M0 scale.
template <int ID> struct Legacy;
template <> struct Legacy<2> { static constexpr int BYTES = 18, M_AT = -1, QH_AT = -1, QS_AT = 2, BIAS = 8, TABLE = 0; };
template <> struct Legacy<3> { static constexpr int BYTES = 20, M_AT = 2, QH_AT = -1, QS_AT = 4, BIAS = 0, TABLE = 0; };
template <> struct Legacy<6> { static constexpr int BYTES = 22, M_AT = -1, QH_AT = 2, QS_AT = 6, BIAS = 16, TABLE = 0; };
template <> struct Legacy<7> { static constexpr int BYTES = 24, M_AT = 2, QH_AT = 4, QS_AT = 8, BIAS = 0, TABLE = 0; };
template <> struct Legacy<20> { static constexpr int BYTES = 18, M_AT = -1, QH_AT = -1, QS_AT = 2, BIAS = 0, TABLE = 1; };
template <> struct Legacy<39> { static constexpr int BYTES = 17, M_AT = -1, QH_AT = -1, QS_AT = 1, BIAS = 0, TABLE = 2; };

typedef uint4 __attribute__((aligned(1))) uint4_a1;

// The levels of four codes (one per byte of `codes`, 0..15) from a 16-entry int8 table held as
// four dwords: a byte permute picks among eight entries, so two of them and the code's bit 3.
template <int TABLE>
static __device__ __forceinline__ uint32_t levels_of(uint32_t codes) {
    // IQ4_NL: -127 -104 -83 -65 | -49 -35 -22 -10 | 1 13 25 38 | 53 69 89 113
    // MXFP4:  0 1 2 3 | 4 6 8 12 | 0 -1 -2 -3 | -4 -6 -8 -12
    constexpr uint32_t T0 = TABLE == 1 ? 0xBFAD9881u : 0x03020100u, T1 = TABLE == 1 ? 0xF6EADDCFu : 0x0C080604u;
    constexpr uint32_t T2 = TABLE == 1 ? 0x26190D01u : 0xFDFEFF00u, T3 = TABLE == 1 ? 0x71594535u : 0xF4F8FAFCu;
    const uint32_t idx = codes & 0x07070707u;
    const uint32_t low = __builtin_amdgcn_perm(T1, T0, idx), high = __builtin_amdgcn_perm(T3, T2, idx);
    const uint32_t top = ((codes >> 3) & 0x01010101u) * 0xFFu;   // 0xFF in the bytes whose code is 8..15
    return (high & top) | (low & ~top);
}

// The block's scale: an f16, or MXFP4's E8M0 byte as 0.5 * 2^(e - 127) (denormal patterns below 2).
template <class F>
static __device__ __forceinline__ float block_scale(const uint8_t* __restrict__ bp) {
    if (F::TABLE == 2) {
        const uint32_t e = bp[0];
        return __uint_as_float(e < 2 ? (0x00200000u << e) : ((e - 1) << 23));
    }
    return f16_bits_to_f32(*(const uint16_t*)bp);
}

// Four bits of `x` (bits 0..3) to bit 4 of four bytes: byte i receives bit i. The multiplier lays
// the nibble down at shifts 0, 7, 14, 21, which puts bit i at position 8 i; the copies do not overlap.
static __device__ __forceinline__ uint32_t fifth_bits(uint32_t x) {
    return (((x & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
}

// The sixteen code bytes of a block as they lie in memory.
template <class F>
static __device__ __forceinline__ uint4 block_code_bytes(const uint8_t* __restrict__ bp) {
    if (F::BYTES % 2) return *(const uint4_a1*)(bp + F::QS_AT);   // 17-byte blocks start on any byte
    if (F::BYTES % 4) {
        // blocks of 18 and 22 bytes put every other run of codes two bytes off a dword, where a
        // 16-byte load runs at three quarters of its rate: read the enclosing dwords and shift
        // (Q4_0 14336 x 4096: 12.8 -> 11.4 us)
        const uint8_t* qs = bp + F::QS_AT;
        return run16_value(load_run16(qs), 8 * (uint32_t)((uintptr_t)qs & 3));
    }
    return *(const uint4_a2*)(bp + F::QS_AT);   // 20- and 24-byte blocks keep the alignment of the blob
}

// The word of fifth bits (formats that have one; 0 otherwise).
template <class F>
static __device__ __forceinline__ uint32_t block_fifth_word(const uint8_t* __restrict__ bp) {
    if (F::QH_AT < 0) return 0;
    return (uint32_t)*(const uint16_t*)(bp + F::QH_AT) | ((uint32_t)*(const uint16_t*)(bp + F::QH_AT + 2) << 16);
}

// Code bytes + fifth bits -> the block's unsigned codes (a table format's: its levels): lo = values
// 0..15, hi = values 16..31, four per dword.
template <class F>
static __device__ __forceinline__ void expand_codes(const uint4 q, const uint32_t qh, uint4& lo, uint4& hi) {
    lo = make_uint4(q.x & 0x0F0F0F0Fu, q.y & 0x0F0F0F0Fu, q.z & 0x0F0F0F0Fu, q.w & 0x0F0F0F0Fu);
    hi = make_uint4((q.x >> 4) & 0x0F0F0F0Fu, (q.y >> 4) & 0x0F0F0F0Fu, (q.z >> 4) & 0x0F0F0F0Fu, (q.w >> 4) & 0x0F0F0F0Fu);
    if (F::TABLE) {
        lo = make_uint4(levels_of<F::TABLE>(lo.x), levels_of<F::TABLE>(lo.y), levels_of<F::TABLE>(lo.z), levels_of<F::TABLE>(lo.w));
        hi = make_uint4(levels_of<F::TABLE>(hi.x), levels_of<F::TABLE>(hi.y), levels_of<F::TABLE>(hi.z), levels_of<F::TABLE>(hi.w));
    }
    if (F::QH_AT >= 0) {
        lo.x |= fifth_bits(qh);       lo.y |= fifth_bits(qh >> 4);  lo.z |= fifth_bits(qh >> 8);  lo.w |= fifth_bits(qh >> 12);
        hi.x |= fifth_bits(qh >> 16); hi.y |= fifth_bits(qh >> 20); hi.z |= fifth_bits(qh >> 24); hi.w |= fifth_bits(qh >> 28);
    }
}

template <class F>
static __device__ __forceinline__ void block_codes(const uint8_t* __restrict__ bp, uint4& lo, uint4& hi) {
    expand_codes<F>(block_code_bytes<F>(bp), block_fifth_word<F>(bp), lo, hi);
}

}  // namespace

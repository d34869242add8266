// What the 16-row-tile kernels for Q4_K / Q5_K share (rows16_mfma.hip: dense launches, the four waves of a
// tile splitting its super-blocks; rows16_moe.hip: per expert over a sorted routing, a wave per tile):
// the activation staged in LDS in the order the matrix instruction's operand wants it, the lane's
// pointers into it, the weight loads of one super-block, and the arithmetic of one super-block.
//
// Layout of the work (v_mfma_i32_16x16x64_i8). Lane l holds weight row l % 16 and the sixteen K values of
// lane group l / 16: the four lane groups of a row take one 64-byte run of `qs`, which holds two
// sub-block pairs, so the instruction on the low nibbles and the one on the high nibbles each see two
// sub-blocks, s in lane groups 0, 1 and s + 2 in groups 2, 3. Up to eight activation rows: the sixteen
// slots of the activation operand are (which of the two sub-blocks) x (row), each slot zero in the other
// sub-block's lane groups; lane l, register v is (weight row l % 16, activation row 4 ((l / 16) % 2) + v,
// sub-block s + 2 (l / 32)). Up to sixteen rows: the slots are rows and every set of weight codes runs
// twice, against s (the activation live in groups 0, 1) and against s + 2; lane l, register v is (weight
// row l % 16, activation row 4 (l / 16) + v) for both.
#pragma once
#include "lk_common.h"

namespace rows16 {

constexpr int TILE = 16;   // weight rows of a wave's tile
static __host__ __device__ constexpr int zero_bytes(int toks) { return toks * 256; }   // the zero lanes' run
// LDS bytes of the staged activation, `chunks` groups of `toks` rows: codes [chunks][nb * 8][toks][32], zeros,
// d8 and d8 * S [chunks][nb * 8][2][toks] floats
static __host__ __device__ constexpr int staged_bytes(int nb, int toks, int chunks = 1) {
    return chunks * nb * 8 * toks * 32 + zero_bytes(toks) + chunks * nb * 8 * 2 * toks * 4;
}

struct WFrag {
    uint4 hdr, q[2], qh;   // qh: Q5_K only
};

template <bool Q5>
struct Blk {
    static constexpr int BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES;
    static constexpr int QS = Q5 ? 48 : 16;
};

// Where the activation rows of a pass live. Dense: row i is row i. Expert-batched: row i of the pass is
// sorted row first + i of the routing, whose activation is row src[first + i] (a missing map: itself).
struct RowsIn {
    const uint8_t* y;   // Q8_1 rows, stride_y blocks apart
    int stride_y;
    const int32_t* src;
    int first;
    __device__ __forceinline__ const uint8_t* block(int i, int sub) const {
        const int r = src ? src[first + i] : first + i;
        return y + ((size_t)r * stride_y + sub) * Q81_BYTES;
    }
};

template <bool Q5, bool T16>
struct Core {
    static constexpr int TOKS = T16 ? 16 : 8;
    static constexpr int PER = 2;   // staging entries a thread has in flight
    // The minimums as a product over the sub-blocks on v_mfma_f32_16x16x4_f32, (d8 * sum of codes)[row, sub-block]
    // x (-dmin * min)[sub-block, weight row], four sub-blocks an instruction, straight into the sums: a third
    // of the per-result vector work otherwise.
    static constexpr bool MIN_ON_MATRIX_UNIT = true;

    uint8_t *codes, *zeros;
    float* table;
    int lane, l16, grp, half, par;
    const uint8_t *a_lane, *a_lane2;
    int a_step, a_step2;       // bytes per super-block (nothing for the zero lanes)
    int a_chunk, a_chunk2;     // bytes per chunk of rows (nothing for the zero lanes)
    int t_chunk;               // floats per chunk of rows
    const float* t_lane;
    int sh16, sh2;
    // staging registers
    uint32_t head[PER];
    uint4 lo[PER], hi[PER];

    // Sets the pointers for `chunks` groups of TOKS rows of `nb` super-blocks; returns the first LDS byte
    // past the staged activation.
    __device__ __forceinline__ uint8_t* init(uint8_t* lds, int nb, int chunks = 1) {
        codes = lds;                                             // [chunks][nb * 8][TOKS][32]
        zeros = codes + (size_t)chunks * nb * 8 * TOKS * 32;     // zero_bytes(TOKS)
        table = (float*)(zeros + zero_bytes(TOKS));              // [chunks][nb * 8][2][TOKS]: d8, d8 * S
        lane = threadIdx.x & 63;
        l16 = lane & 15;
        grp = lane >> 4;
        half = grp & 1;   // which sixteen values of a sub-block (operands), which four rows (results)
        par = grp >> 1;   // which of an instruction's two sub-blocks
        // The lane's piece of the activation operand. Up to eight rows: slot l16 is (sub-block l16 / 8 of
        // the two, row l16 % 8); the lane's K group belongs to sub-block par; where the two differ the
        // piece is zeros: those lanes read the run of zeros, at a stride of nothing. Up to sixteen rows:
        // slot l16 is row l16, and there are two pieces, one per run of the instruction: live for the
        // lanes of sub-block 0 (groups 0, 1) in the first, for those of sub-block 1 in the second.
        const bool live = T16 ? par == 0 : (l16 >> 3) == par;
        const bool live2 = T16 && par == 1;
        a_lane = live ? codes + (T16 ? l16 : 2 * par * TOKS + (l16 & 7)) * 32 + 16 * half : zeros;
        a_lane2 = live2 ? codes + (2 * TOKS + l16) * 32 + 16 * half : zeros;
        a_step = live ? 8 * TOKS * 32 : 0;
        a_step2 = live2 ? 8 * TOKS * 32 : 0;
        a_chunk = live ? nb * 8 * TOKS * 32 : 0;
        a_chunk2 = live2 ? nb * 8 * TOKS * 32 : 0;
        t_chunk = nb * 8 * 2 * TOKS;
        // the lane's results: up to eight rows: sub-blocks 2 par + {0, 1, 4, 5}, rows 4 half .. 4 half + 3;
        // up to sixteen: every sub-block, rows 4 grp .. 4 grp + 3
        t_lane = T16 ? table + 4 * grp : table + 2 * par * 2 * TOKS + 4 * half;
        sh16 = T16 ? 0 : 16 * par;
        sh2 = 2 * par;
        return (uint8_t*)(table + chunks * nb * 8 * 2 * TOKS);
    }

    // The activation: entry (chunk, sub-block, row of the chunk) is one Q8_1 block; `per_chunk` entries to a
    // chunk. `issue` puts the loads of the entries base + u * threads in flight, `place` writes them to LDS
    // (rows past m_count: zeros).
    __device__ __forceinline__ void issue(const RowsIn& rows, int m_count, int entries, int per_chunk, int base, int threads) {
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = min(base + u * threads, entries - 1);
            const int chunk = idx / per_chunk, in_chunk = idx % per_chunk;
            const int sub = in_chunk / TOKS, tok = min(chunk * TOKS + in_chunk % TOKS, m_count - 1);
            const uint8_t* b = rows.block(tok, sub);
            head[u] = *(const uint32_t*)b;
            lo[u] = *(const uint4_a4*)(b + 4);
            hi[u] = *(const uint4_a4*)(b + 20);
        }
    }
    __device__ __forceinline__ void place(int m_count, int entries, int per_chunk, int base, int threads) {
        const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = base + u * threads;
            if (idx < entries) {
                const int chunk = idx / per_chunk, in_chunk = idx % per_chunk;
                const int sub = in_chunk / TOKS, tok = in_chunk % TOKS;
                const bool real = chunk * TOKS + tok < m_count;
                const float d8 = real ? f16_bits_to_f32(head[u] & 0xFFFFu) : 0.f;
                float* t = table + chunk * t_chunk + sub * 2 * TOKS + tok;
                t[0] = d8;
                t[TOKS] = d8 * (float)dot16(ones, hi[u], dot16(ones, lo[u], 0));
                const uint32_t keep = real ? 0xFFFFFFFFu : 0u;   // rows the launch does not have: zeros
                *(uint4*)(codes + (size_t)idx * 32) = make_uint4(lo[u].x & keep, lo[u].y & keep, lo[u].z & keep, lo[u].w & keep);
                *(uint4*)(codes + (size_t)idx * 32 + 16) = make_uint4(hi[u].x & keep, hi[u].y & keep, hi[u].z & keep, hi[u].w & keep);
            }
        }
    }
    // The entries after the first round (whose loads the caller issued ahead of its weight loads), and the
    // run of zeros. The caller's barrier follows.
    __device__ __forceinline__ void finish_staging(const RowsIn& rows, int m_count, int nb, int threads, int chunks = 1) {
        const int per_chunk = nb * 8 * TOKS, entries = chunks * per_chunk;
        place(m_count, entries, per_chunk, threadIdx.x, threads);
        for (int r = threads * PER; r < entries; r += threads * PER) {
            issue(rows, m_count, entries, per_chunk, r + threadIdx.x, threads);
            place(m_count, entries, per_chunk, r + threadIdx.x, threads);
        }
        for (int i = threadIdx.x * 16; i < zero_bytes(TOKS); i += threads * 16) *(uint4*)(zeros + i) = make_uint4(0, 0, 0, 0);
    }

    // The lane's pieces of the super-block at `bp` (its row's): header, fifth bits, the two runs of qs.
    __device__ __forceinline__ void loadw(WFrag& f, const uint8_t* bp) const {
        f.hdr = *(const uint4*)bp;
        if (Q5) f.qh = *(const uint4*)(bp + 16 + 16 * half);
        f.q[0] = *(const uint4*)(bp + Blk<Q5>::QS + 16 * grp);
        f.q[1] = *(const uint4*)(bp + Blk<Q5>::QS + 64 + 16 * grp);
    }

    // Super-block kb of the lane's weight row against the staged activation, into the lane's four sums.
    __device__ __forceinline__ void compute(const WFrag& w, int kb, float (&acc)[4]) const {
        float (&one)[1][4] = reinterpret_cast<float (&)[1][4]>(acc);
        compute_chunks<1>(w, kb, one);
    }
    // The same against CHUNKS groups of rows: the weight codes and scales are unpacked once.
    template <int CHUNKS>
    __device__ __forceinline__ void compute_chunks(const WFrag& w, int kb, float (&acc)[CHUNKS][4]) const {
        // the row's (scale, min) pairs, six bits each (get_scale_min_k4 of the format); up to eight rows:
        // the words shifted to sub-blocks 2 par, 2 par + 1, 4 + 2 par, 5 + 2 par
        const uint32_t w1 = w.hdr.y, w2 = w.hdr.z, w3 = w.hdr.w;
        const uint32_t sc_lo = (w1 & 0x3F3F3F3Fu) >> sh16, mn_lo = (w2 & 0x3F3F3F3Fu) >> sh16;
        const uint32_t sc_hi = ((w3 & 0x0F0F0F0Fu) | ((w1 >> 2) & 0x30303030u)) >> sh16;
        const uint32_t mn_hi = (((w3 >> 4) & 0x0F0F0F0Fu) | ((w2 >> 2) & 0x30303030u)) >> sh16;
        const float d = f16_bits_to_f32(w.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(w.hdr.x >> 16);
        uint32_t hp[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
        if (Q5) {
#pragma unroll
            for (int e = 0; e < 4; ++e) hp[e] >>= sh2;
        }
        const uint8_t* a_blk = a_lane + (size_t)kb * a_step;
        const uint8_t* a_blk2 = a_lane2 + (size_t)kb * a_step2;
        const float* t_blk = t_lane + kb * 8 * 2 * TOKS;
        // The accumulators start at the bit pattern of 1.5 * 2^23: adding an integer of magnitude below
        // 2^22 to that pattern yields the float 1.5 * 2^23 + integer, so the dots leave the matrix unit
        // as floats. The offset goes in the first fused multiply-add, exactly: d * sc is an f16 times a
        // six-bit integer (17 significant bits), MAGIC * d * sc has 19, neither product rounds, and the
        // fma rounds dot * d * sc once, as convert-then-multiply would.
        constexpr int MAGIC_BITS = 0x4B400000;
        constexpr float MAGIC = 12582912.0f;
        const v4i magic = {MAGIC_BITS, MAGIC_BITS, MAGIC_BITS, MAGIC_BITS};
        // one instruction's four results into the sums of chunk ch: sub-block `sub` of the super-block
        auto fold = [&](int ch, const v4i& c, float dsc, float dmm, int sub) {
            const float off = -MAGIC * dsc;
            const float4 t = *(const float4*)(t_blk + ch * t_chunk + sub * 2 * TOKS);
            if constexpr (MIN_ON_MATRIX_UNIT) {   // (the minimums: below)
                acc[ch][0] = fmaf(fmaf(__int_as_float(c[0]), dsc, off), t.x, acc[ch][0]);
                acc[ch][1] = fmaf(fmaf(__int_as_float(c[1]), dsc, off), t.y, acc[ch][1]);
                acc[ch][2] = fmaf(fmaf(__int_as_float(c[2]), dsc, off), t.z, acc[ch][2]);
                acc[ch][3] = fmaf(fmaf(__int_as_float(c[3]), dsc, off), t.w, acc[ch][3]);
                return;
            }
            const float4 s = *(const float4*)(t_blk + ch * t_chunk + sub * 2 * TOKS + TOKS);
            acc[ch][0] = fmaf(fmaf(__int_as_float(c[0]), dsc, off), t.x, fmaf(dmm, s.x, acc[ch][0]));
            acc[ch][1] = fmaf(fmaf(__int_as_float(c[1]), dsc, off), t.y, fmaf(dmm, s.y, acc[ch][1]));
            acc[ch][2] = fmaf(fmaf(__int_as_float(c[2]), dsc, off), t.z, fmaf(dmm, s.z, acc[ch][2]));
            acc[ch][3] = fmaf(fmaf(__int_as_float(c[3]), dsc, off), t.w, fmaf(dmm, s.w, acc[ch][3]));
        };
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
            const uint32_t u[4] = {w.q[c2].x, w.q[c2].y, w.q[c2].z, w.q[c2].w};
#pragma unroll
            for (int nib = 0; nib < 2; ++nib) {
                v4i b;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    uint32_t x = (nib ? u[e] >> 4 : u[e]) & 0x0F0F0F0Fu;
                    if (Q5) x |= ((hp[e] >> (4 * c2 + nib)) & 0x01010101u) << 4;
                    b[e] = (int)x;
                }
                const uint32_t scw = c2 ? sc_hi : sc_lo, mnw = c2 ? mn_hi : mn_lo;
                const float dsc0 = d * (float)((scw >> (8 * nib)) & 0xFFu), dmm0 = -(dmin * (float)((mnw >> (8 * nib)) & 0xFFu));
#pragma unroll
                for (int ch = 0; ch < CHUNKS; ++ch) {
                    if constexpr (T16) {
                        // sub-blocks 4 c2 + nib (lane groups 0, 1) and 4 c2 + 2 + nib (groups 2, 3)
                        const v4i a0 = *(const v4i*)(a_blk + ch * a_chunk + (4 * c2 + nib) * TOKS * 32);
                        const v4i a1 = *(const v4i*)(a_blk2 + ch * a_chunk2 + (4 * c2 + nib) * TOKS * 32);
                        const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b, magic, 0, 0, 0);
                        const v4i c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b, magic, 0, 0, 0);
                        fold(ch, c0, dsc0, dmm0, 4 * c2 + nib);
                        fold(ch, c1, d * (float)((scw >> (8 * nib + 16)) & 0xFFu), -(dmin * (float)((mnw >> (8 * nib + 16)) & 0xFFu)),
                             4 * c2 + 2 + nib);
                    } else {
                        // this lane's sub-block: 4 c2 + 2 par + nib (its scale words are shifted to it)
                        const v4i a = *(const v4i*)(a_blk + ch * a_chunk + (4 * c2 + nib) * TOKS * 32);
                        const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, magic, 0, 0, 0);
                        fold(ch, c, dsc0, dmm0, 4 * c2 + nib);
                    }
                }
            }
        }
        if constexpr (MIN_ON_MATRIX_UNIT) {
            // lane (row l16 of the activation, sub-block 4 h + grp) of d8 * S against lane (weight row l16,
            // sub-block 4 h + grp) of -dmin * min. Up to eight rows: rows 8..15 of the product are nobody's
            // (their lanes' sums join those of rows 0..7 in the end): their operand is zero.
            const uint32_t mins_lo = w2 & 0x3F3F3F3Fu, mins_hi = ((w3 >> 4) & 0x0F0F0F0Fu) | ((w2 >> 2) & 0x30303030u);
            const float* s_blk = table + kb * 8 * 2 * TOKS + TOKS + (l16 & (TOKS - 1));
            const bool real = T16 || l16 < TOKS;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float bmin = -(dmin * (float)(((h ? mins_hi : mins_lo) >> (8 * grp)) & 0xFFu));
#pragma unroll
                for (int ch = 0; ch < CHUNKS; ++ch) {
                    const float at = s_blk[ch * t_chunk + (4 * h + grp) * 2 * TOKS];
                    const float amin = real ? at : 0.f;
                    v4f c = {acc[ch][0], acc[ch][1], acc[ch][2], acc[ch][3]};
                    c = __builtin_amdgcn_mfma_f32_16x16x4f32(amin, bmin, c, 0, 0, 0);
                    acc[ch][0] = c[0];
                    acc[ch][1] = c[1];
                    acc[ch][2] = c[2];
                    acc[ch][3] = c[3];
                }
            }
        }
    }
};

}  // namespace rows16

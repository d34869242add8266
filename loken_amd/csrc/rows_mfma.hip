// Q4_K weights x a handful of Q8_1 activation rows on the int8 matrix unit: the mid-batch path
// between the mat-vec kernels (whose dot work grows with every activation row) and the tiled
// matmul (which stages weights through LDS and needs hundreds of rows to pay for it).
//
// Replaces loken_dense_q4k_imma_m8_plain of the reference (declared src/inference/moe_cuda/
// mod.rs:456-458, called from dense_q4k_imma_m8_matmul, src/inference/moe_cuda/dense/imma.rs:
// 82-135; kernels cuda/q4k_mmvq_imma.cu, cuda/imma_amd.cu:472-545): plain block_q8_1 rows in,
// `out += dsc * d8 * C - dmm * d8 * S` per sub-block. Here S is the integer sum of the codes,
// as everywhere else in this library, not the rounded `s` field of the Q8_1 block.
//
// Shape of the work. A wave owns 32 weight rows and up to 32 activation rows: one
// v_mfma_i32_32x32x32_i8 is one Q4_K sub-block (32 values) of those rows against those
// activations. Weights never touch LDS: lane l holds row l % 32 and reads, per super-block, its
// 16-byte header and the four 16-byte runs of `qs` at 32 * p + 16 * (l / 32), which are exactly
// its half of the B operand for sub-blocks 2p (low nibbles) and 2p + 1 (high nibbles). The
// activation codes come the same way (lane l: row l % 32, 16 codes at 16 * (l / 32), straight
// from the Q8_1 block), so the only LDS traffic is the table of activation scales, staged once
// per workgroup, from which a lane fetches the 16 scales its accumulator registers stand for.
// The four waves of a workgroup split the super-blocks of the same 32 rows between them and
// add their partial tiles through LDS, which keeps small matrices spread over the chip.
//
// Registers stand for activation rows (register v = row (v / 4) * 8 + 4 * (l / 32) + v % 4) and lanes
// for weight rows, so a launch of at most 8 (16) activation rows only ever needs registers 0..3
// (0..7) of each tile: the kernel is compiled for G = 1, 2 or 4 groups of eight rows and spends the
// per-sub-block fix-up on those registers alone. That fix-up is most of the kernel's vector work,
// and with it cut to a quarter the weights stream near the memory rate.
//
// The min term -dmin * m[s] * d8 * S[s] is rank one per sub-block. With G < 4 it is vector work on
// the live registers: d8 * S of every (sub-block, activation row) is tabled in LDS beside d8 when
// the workgroup starts (S summed from the codes there), and a register's row reads it as a
// broadcast. With G = 4 it goes through
// v_mfma_f32_32x32x2_f32 with K = the two halves of the sub-block: A = d8 * (sum of the lane's
// own 16 codes), B = -dmin * m[s] in both halves. No lane exchange is needed for the sum.

#include "lk_common.h"
#include "rows16.h"

#include <mutex>
#include <unordered_map>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int WG = 256, WAVES = 4;
constexpr int TOK = 32;   // activation rows per pass (the matrix instruction's M)

struct Args {
    const uint8_t* w;
    const uint8_t* y;     // Q8_1 rows
    float* dst;
    int nb;               // super-blocks per weight row
    int n;                // weight rows
    int m;                // activation rows in all
    int stride_y;         // Q8_1 blocks between activation rows
    int ldd;              // floats between output rows
    const uint8_t* w2;    // DUAL: the second matrix (same shape); the output is act(w . x) * (w2 . x)
    int gelu;             // DUAL: 0 SiLU, 1 tanh-form GELU
    // MULTI (the dense launch only): up to two more matrices over the same activation rows, each with its
    // own output; their row tiles follow the first matrix's in the launch's tile order
    const uint8_t* w_b = nullptr;
    const uint8_t* w_c = nullptr;
    float* dst_b = nullptr;
    float* dst_c = nullptr;
    int n_b = 0, n_c = 0, ldd_b = 0, ldd_c = 0;
    // DUAL, the dense launch only, when given: the result leaves as Q8_1 rows (a row tile's 32 rows are one
    // block; q81_stride blocks between activation rows) instead of f32 in `dst`; n a multiple of 32
    uint8_t* q81_dst = nullptr;
    int q81_stride = 0;
};

// Row tile `t` of a launch: which matrix it belongs to, and which of that matrix's tiles it is.
struct MatRef {
    const uint8_t* w;
    float* dst;
    int n, ldd, tile;
};
template <bool MULTI>
static __device__ __forceinline__ MatRef mat_of(const Args& p, float* dst, int ldd, int t) {
    if (!MULTI) return {p.w, dst, p.n, ldd, t};
    const int ta = (p.n + 31) >> 5, tb = (p.n_b + 31) >> 5;
    if (t < ta) return {p.w, dst, p.n, ldd, t};
    if (t < ta + tb) return {p.w_b, p.dst_b, p.n_b, p.ldd_b, t - ta};
    return {p.w_c, p.dst_c, p.n_c, p.ldd_c, t - ta - tb};
}

// With DUAL a workgroup walks "virtual" tiles: 2 t is row tile t of the first matrix, 2 t + 1 the same
// rows of the second. The first's reduced sums wait in registers for the second's.
template <bool DUAL>
static __device__ __forceinline__ int first_tile(int wg) { return DUAL ? 2 * wg : wg; }
template <bool DUAL>
static __device__ __forceinline__ int next_tile(int vt, int wgs) {
    return DUAL ? ((vt & 1) ? vt - 1 + 2 * wgs : vt + 1) : vt + wgs;
}

struct Frag {
    uint4 hdr, q[4], qh;   // qh: Q5_K only, the lane's 16 bytes of fifth bits (bit s = sub-block s)
    v4i a[8];
};

// Q5_K is Q4_K with a plane of fifth bits between the header and the nibbles
// (block_q5_K: d, dmin, scales[12], qh[32], qs[128]).
template <bool Q5>
struct Blk {
    static constexpr int BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES;
    static constexpr int QS = Q5 ? 48 : 16;
};

// The B operand of sub-block s from the lane's 16 bytes of its pair's nibbles (and fifth bits).
template <bool Q5>
static __device__ __forceinline__ v4i codes_of(const uint4& q, const uint4& qh, int s) {
    const uint32_t u[4] = {q.x, q.y, q.z, q.w}, h[4] = {qh.x, qh.y, qh.z, qh.w};
    v4i b;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        uint32_t x = ((s & 1) ? u[e] >> 4 : u[e]) & 0x0F0F0F0Fu;
        if (Q5) x |= ((h[e] >> s) & 0x01010101u) << 4;
        b[e] = (int)x;
    }
    return b;
}

// Floats of the scale tables: d8 [nb * 8][8 G], and with G < 4 also d8 * S in the same shape.
template <int G>
static __host__ __device__ constexpr int lds_floats_table(int nb) { return nb * 8 * 8 * G * (G < 4 ? 2 : 1); }

// Where the activation rows of a pass live and where their results go. Dense: consecutive rows.
// Expert-batched: row i of the pass is sorted row first + i of the routing; its activation is row
// src[first + i] of the Q8_1 rows (the token), its result goes to row dst_map[first + i] (or
// first + i) of the output.
struct PassRows {
    const uint8_t* y;        // Q8_1 rows
    float* dst;
    const int32_t* src;      // nullable: activation row of a sorted row
    const int32_t* dst_map;  // nullable: output row of a sorted row
    int first;               // first row of the pass
    int stride_y, ldd;
    __device__ __forceinline__ const uint8_t* y_row(int i) const {
        const int r = src ? src[first + i] : first + i;
        return y + (size_t)r * stride_y * Q81_BYTES;
    }
    __device__ __forceinline__ float* out_row(int i) const {
        const int r = dst_map ? dst_map[first + i] : first + i;
        return dst + (size_t)r * ldd;
    }
};

// One pass: every row tile of this workgroup's share of matrix `p.w` (and `p.w2`) against the
// `m_count` activation rows of `rows` (at most 8 G). Every wave of the workgroup must call it, and
// all leave it past the same barriers, so passes can follow one another.
// KSPLIT: the four waves of the workgroup share each row tile and split its super-blocks (long rows:
// every wave has blocks to stream, and the partial tiles meet in LDS). Without it a wave owns whole
// row tiles, all of a row's super-blocks in turn, and nothing crosses waves but the tables: rows of
// at most eight super-blocks, where a four-way split leaves a wave one or two blocks per tile and
// most of its time in the reduction's barriers.
template <int G, bool DUAL, bool Q5, bool KSPLIT = true, bool MULTI = false>
static __device__ __forceinline__ void q4k_rows_pass(const Args& p, const PassRows& rows, int m_count, uint8_t* lds) {
    static_assert(!MULTI || (!DUAL && KSPLIT), "several matrices: the dense launch with the super-blocks split over the waves");
    constexpr int TW = 8 * G;   // activation rows a table row holds
    constexpr int NV = 4 * G;   // live accumulator registers
    float* d8_table = (float*)lds;                                   // [nb * 8][TW]
    float* ds_table = d8_table + p.nb * 8 * TW;                      // [nb * 8][TW], G < 4 only
    float* reduce = d8_table + lds_floats_table<G>(p.nb);            // [WAVES][NV][64]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int n_tiles = ((p.n + 31) >> 5) + (MULTI ? ((p.n_b + 31) >> 5) + ((p.n_c + 31) >> 5) : 0);
    const size_t row_bytes = (size_t)p.nb * Blk<Q5>::BYTES;

    // Activation scales of this pass, zero for the rows the pass does not have. Eight loads are
    // issued before the first is used: one at a time, each would cost a memory latency.
    const int entries = p.nb * 8 * TW;
    if constexpr (G == 4) {
        for (int base = threadIdx.x; base < entries; base += WG * 8) {
            uint32_t bits[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = min(base + u * WG, entries - 1);
                const int sub = idx >> 5, tok = min(idx & 31, m_count - 1);
                bits[u] = *(const uint16_t*)(rows.y_row(tok) + (size_t)sub * Q81_BYTES);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = base + u * WG;
                if (idx < entries) d8_table[idx] = (idx & 31) < m_count ? f16_bits_to_f32(bits[u]) : 0.f;
            }
        }
    } else {
        // whole blocks: the scale and the integer sum of the 32 codes (four entries in flight)
        for (int base = threadIdx.x; base < entries; base += WG * 4) {
            uint32_t head[4];
            uint4 lo[4], hi[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = min(base + u * WG, entries - 1);
                const int sub = idx / TW, tok = min(idx % TW, m_count - 1);
                const uint8_t* b = rows.y_row(tok) + (size_t)sub * Q81_BYTES;
                head[u] = *(const uint32_t*)b;
                lo[u] = *(const uint4_a4*)(b + 4);
                hi[u] = *(const uint4_a4*)(b + 20);
            }
            const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * WG;
                if (idx < entries) {
                    const bool real = idx % TW < m_count;
                    const float d8 = real ? f16_bits_to_f32(head[u] & 0xFFFFu) : 0.f;
                    d8_table[idx] = d8;
                    ds_table[idx] = d8 * (float)dot16(ones, hi[u], dot16(ones, lo[u], 0));
                }
            }
        }
    }

    // The lane's activation row (a row past the end re-reads the last one; its scales are zero).
    const uint8_t* y_lane = rows.y_row(min(l32, m_count - 1)) + 4 + 16 * lh;

    auto load = [&](Frag& f, int tile, int kb) {
        const MatRef mr = mat_of<MULTI>(p, rows.dst, rows.ldd, DUAL ? tile >> 1 : tile);
        const int row = min(mr.tile * 32 + l32, mr.n - 1);
        const uint8_t* mat = DUAL && (tile & 1) ? p.w2 : mr.w;
        const uint8_t* bp = (const uint8_t*)(to_gbytes(mat) + row * row_bytes + (size_t)kb * Blk<Q5>::BYTES);
        f.hdr = *(const uint4*)bp;
        if (Q5) f.qh = *(const uint4*)(bp + 16 + 16 * lh);
#pragma unroll
        for (int c = 0; c < 4; ++c) f.q[c] = *(const uint4*)(bp + Blk<Q5>::QS + 32 * c + 16 * lh);
        const uint8_t* ap = y_lane + (size_t)kb * 8 * Q81_BYTES;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint4 t = *(const uint4_a4*)(ap + s * Q81_BYTES);
            f.a[s] = v4i{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
        }
    };

    // Two accumulators: the scale term is vector arithmetic on `acc`, the min term a chain of
    // matrix instructions on `acc_min`; kept apart, neither waits for the other's latency.
    // (With G < 4 both are vector arithmetic on the live registers.)
    v16f acc, acc_min;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = acc_min[v] = 0.f;

    auto compute = [&](const Frag& f, int kb) {
        // the row's eight (scale, min) pairs, six bits each (get_scale_min_k4 of the format)
        const uint32_t w1 = f.hdr.y, w2 = f.hdr.z, w3 = f.hdr.w;
        const uint32_t sc_lo = w1 & 0x3F3F3F3Fu, mn_lo = w2 & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (w3 & 0x0F0F0F0Fu) | ((w1 >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((w3 >> 4) & 0x0F0F0F0Fu) | ((w2 >> 2) & 0x30303030u);
        const float d = f16_bits_to_f32(f.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(f.hdr.x >> 16);
        float dsc[8], dmm[8];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            dsc[s] = d * (float)((sc_lo >> (8 * s)) & 0xFFu);
            dsc[s + 4] = d * (float)((sc_hi >> (8 * s)) & 0xFFu);
            dmm[s] = -(dmin * (float)((mn_lo >> (8 * s)) & 0xFFu));
            dmm[s + 4] = -(dmin * (float)((mn_hi >> (8 * s)) & 0xFFu));
        }
        const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const v4i b = codes_of<Q5>(f.q[s >> 1], f.qh, s);
            // The int32 accumulators start at the bit pattern of 1.5 * 2^23: adding an integer of
            // magnitude below 2^22 to that pattern yields the float 1.5 * 2^23 + integer, so the
            // dots leave the matrix unit as floats and no conversion is spent on them. The offset
            // goes in the first fused multiply-add, exactly: d * sc is an f16 times a six-bit
            // integer (17 significant bits), MAGIC * d * sc has 19, so neither product rounds and
            // the fma rounds dot * d * sc once, as convert-then-multiply would.
            constexpr int MAGIC_BITS = 0x4B400000;
            constexpr float MAGIC = 12582912.0f;
            v16i c;
#pragma unroll
            for (int v = 0; v < 16; ++v) c[v] = MAGIC_BITS;
            c = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a[s], b, c, 0, 0, 0);
            const float* d8_sub = d8_table + (kb * 8 + s) * TW;
            if constexpr (G == 4) {
                // min term: this lane's activation row and half of the sub-block
                const uint4 au = make_uint4((uint32_t)f.a[s][0], (uint32_t)f.a[s][1], (uint32_t)f.a[s][2], (uint32_t)f.a[s][3]);
                const float half_sum = d8_sub[l32] * (float)dot16(ones, au, 0);
                acc_min = __builtin_amdgcn_mfma_f32_32x32x2f32(half_sum, dmm[s], acc_min, 0, 0, 0);
            }
            // scale term: register v stands for activation row (v / 4) * 8 + lh * 4 + v % 4
            const float off = -MAGIC * dsc[s];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float4 t = *(const float4*)(d8_sub + 8 * g + 4 * lh);
                acc[4 * g + 0] = fmaf(fmaf(__int_as_float(c[4 * g + 0]), dsc[s], off), t.x, acc[4 * g + 0]);
                acc[4 * g + 1] = fmaf(fmaf(__int_as_float(c[4 * g + 1]), dsc[s], off), t.y, acc[4 * g + 1]);
                acc[4 * g + 2] = fmaf(fmaf(__int_as_float(c[4 * g + 2]), dsc[s], off), t.z, acc[4 * g + 2]);
                acc[4 * g + 3] = fmaf(fmaf(__int_as_float(c[4 * g + 3]), dsc[s], off), t.w, acc[4 * g + 3]);
                if constexpr (G < 4) {
                    const float4 u = *(const float4*)(ds_table + (kb * 8 + s) * TW + 8 * g + 4 * lh);
                    acc_min[4 * g + 0] = fmaf(dmm[s], u.x, acc_min[4 * g + 0]);
                    acc_min[4 * g + 1] = fmaf(dmm[s], u.y, acc_min[4 * g + 1]);
                    acc_min[4 * g + 2] = fmaf(dmm[s], u.z, acc_min[4 * g + 2]);
                    acc_min[4 * g + 3] = fmaf(dmm[s], u.w, acc_min[4 * g + 3]);
                }
            }
        }
    };

    const int n_vt = DUAL ? 2 * n_tiles : n_tiles;
    if constexpr (!KSPLIT) {
        // a wave's own tiles: unit = workgroup * 4 + wave, then every (workgroups * 4)-th
        const int units = (int)gridDim.x * WAVES;
        int tile = first_tile<DUAL>((int)blockIdx.x * WAVES + wave), kb = 0;
        Frag fa, fb;
        if (tile < n_vt) load(fa, tile, 0);
        __syncthreads();   // the scale table is complete
        float gate_keep[NV];
        auto finish_own = [&](int t) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                float sum = acc[v] + acc_min[v];
                acc[v] = acc_min[v] = 0.f;
                if (DUAL && !(t & 1)) { gate_keep[v] = sum; continue; }
                if (DUAL) {
                    LkGateAct act;
                    act.kind = p.gelu ? LK_GATE_GELU : LK_GATE_SILU;
                    sum = lk_gated(act, gate_keep[v], sum, 0);
                }
                const int tok = (v >> 2) * 8 + lh * 4 + (v & 3), row = (DUAL ? t >> 1 : t) * 32 + l32;
                if (tok < m_count && row < p.n) rows.out_row(tok)[row] = sum;
            }
        };
        while (tile < n_vt) {
            int nt = tile, nk = kb + 1;
            const bool last = nk >= p.nb;
            if (last) { nk = 0; nt = next_tile<DUAL>(nt, units); }
            if (nt < n_vt) load(fb, nt, nk);
            compute(fa, kb);
            if (last) finish_own(tile);
            tile = nt; kb = nk;
            if (tile >= n_vt) break;
            nt = tile; nk = kb + 1;
            const bool last2 = nk >= p.nb;
            if (last2) { nk = 0; nt = next_tile<DUAL>(nt, units); }
            if (nt < n_vt) load(fa, nt, nk);
            compute(fb, kb);
            if (last2) finish_own(tile);
            tile = nt; kb = nk;
        }
        __syncthreads();   // every wave is done with the tables: the next pass may rebuild them
        return;
    }

    // Steps are (row tile, super-block) pairs: wave w takes super-blocks w, w + 4, ... of every
    // tile of this workgroup; the loads of the next step fly under the arithmetic of this one.
    const int my_blocks = (p.nb - wave + WAVES - 1) / WAVES;   // may be zero for short rows
    const int wgs = (int)gridDim.x;
    int tile = first_tile<DUAL>(blockIdx.x), kb = wave;
    Frag fa, fb;
    if (tile < n_vt && my_blocks > 0) load(fa, tile, kb);
    __syncthreads();   // the scale table is complete

    float gate_keep[G];
    auto finish_tile = [&](int t) {
        // add the four partial tiles and write the activation rows this pass has
        float* mine = reduce + wave * (NV * 64);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            mine[v * 64 + lane] = acc[v] + acc_min[v];
            acc[v] = acc_min[v] = 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < G; ++r) {
            const int v = wave * G + r;
            float sum = (reduce[v * 64 + lane] + reduce[(NV + v) * 64 + lane]) +
                        (reduce[(2 * NV + v) * 64 + lane] + reduce[(3 * NV + v) * 64 + lane]);
            if (DUAL && !(t & 1)) { gate_keep[r] = sum; continue; }
            if (DUAL) {
                LkGateAct act;
                act.kind = p.gelu ? LK_GATE_GELU : LK_GATE_SILU;
                sum = lk_gated(act, gate_keep[r], sum, 0);
            }
            const int tok = (v >> 2) * 8 + lh * 4 + (v & 3);
            if (DUAL && p.q81_dst) {
                // the 32 lanes of a half wave hold one activation row's results for the tile's 32 rows: a block
                // (every lane takes part in the exchanges; a row the pass does not have stores nothing)
                uint8_t* blk = p.q81_dst + ((size_t)(rows.first + min(tok, m_count - 1)) * p.q81_stride + (t >> 1)) * Q81_BYTES;
                lk_store_q8_1_block_by_lane(sum, l32, blk, tok < m_count);
                continue;
            }
            if (MULTI) {   // (dense rows: the pass's row i is row first + i of every output)
                const MatRef mr = mat_of<MULTI>(p, rows.dst, rows.ldd, t);
                const int row = mr.tile * 32 + l32;
                if (tok < m_count && row < mr.n) mr.dst[(size_t)(rows.first + tok) * mr.ldd + row] = sum;
            } else {
                const int row = (DUAL ? t >> 1 : t) * 32 + l32;
                if (tok < m_count && row < p.n) rows.out_row(tok)[row] = sum;
            }
        }
        __syncthreads();   // the partial tiles may be overwritten (and, past the last tile, the tables)
    };

    while (tile < n_vt) {
        if (my_blocks > 0) {
            for (;;) {
                int nt = tile, nk = kb + WAVES;
                const bool last = nk >= p.nb;
                if (last) { nk = wave; nt = next_tile<DUAL>(nt, wgs); }
                if (nt < n_vt) load(fb, nt, nk);
                compute(fa, kb);
                if (last) { finish_tile(tile); tile = nt; kb = nk; if (tile >= n_vt) return; }
                else kb = nk;
                // second half of the ping-pong
                nt = tile; nk = kb + WAVES;
                const bool last2 = nk >= p.nb;
                if (last2) { nk = wave; nt = next_tile<DUAL>(nt, wgs); }
                if (nt < n_vt) load(fa, nt, nk);
                compute(fb, kb);
                if (last2) { finish_tile(tile); tile = nt; kb = nk; if (tile >= n_vt) return; }
                else kb = nk;
            }
        } else {
            finish_tile(tile);   // nothing of its own to add, but the barriers are the workgroup's
            tile = next_tile<DUAL>(tile, wgs);
        }
    }
}

// Dense: grid y walks the activation in passes of 32 rows.
template <int G, bool DUAL, bool Q5, bool MULTI = false>
__global__ __launch_bounds__(WG, 2) void q4k_rows_mfma_kernel(Args p) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int m0 = blockIdx.y * TOK;
    const PassRows rows{p.y, p.dst, nullptr, nullptr, m0, p.stride_y, p.ldd};
    q4k_rows_pass<G, DUAL, Q5, true, MULTI>(p, rows, min(TOK, p.m - m0), lds);
}

// Expert-batched: grid y is the expert; its sorted rows [bounds[e], bounds[e + 1]) go through in
// passes of 8 G, each a walk over the expert's row tiles (the tables in LDS are rebuilt per pass).
struct MoeRows {
    const int32_t* bounds;    // [experts + 1]
    const int32_t* src;       // sorted row -> activation row; nullable (the sorted row itself)
    const int32_t* dst_map;   // sorted row -> output row; nullable
    int64_t expert_bytes;     // between consecutive experts' matrices (both stacks)
};

template <int G, bool DUAL, bool Q5, bool KSPLIT>
__global__ __launch_bounds__(WG, 2) void q4k_rows_moe_kernel(Args p, MoeRows m) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int e = blockIdx.y;
    const int begin = m.bounds[e], end = m.bounds[e + 1];
    if (end <= begin) return;
    p.w += (int64_t)e * m.expert_bytes;
    if (DUAL) p.w2 += (int64_t)e * m.expert_bytes;
    for (int first = begin; first < end; first += 8 * G) {
        const PassRows rows{p.y, p.dst, m.src, m.dst_map, first, p.stride_y, p.ldd};
        q4k_rows_pass<G, DUAL, Q5, KSPLIT>(p, rows, min(8 * G, end - first), lds);
    }
}

// ---------------------------------------------------------------------------------------------
// At most 16 activation rows whose codes fit in LDS: the workgroup stages the codes once (in the
// order the A operand wants them) beside the two scale tables, so the only global loads of a step
// are the weight row's five 16-byte pieces, and a wave keeps three or four steps of them in flight. With the
// activation read from memory per step as above, two steps in flight left a decode-sized matrix
// (one 32-row tile per workgroup, four steps per wave) waiting on memory latency most of its time.
// ---------------------------------------------------------------------------------------------
struct WFrag {
    uint4 hdr, q[4], qh;
};

template <int G>
static __host__ __device__ constexpr int lds_bytes_staged(int nb) {
    // codes [nb * 8][8 G][32], d8 and d8 * S [nb * 8][8 G] floats each, reduce [WAVES][4 G][64] floats
    return nb * 8 * 8 * G * 32 + 2 * nb * 8 * 8 * G * 4 + WAVES * 4 * G * 64 * 4;
}

template <int G, bool DUAL, bool Q5>
__global__ __launch_bounds__(WG, G == 1 ? 2 : 1) void q4k_rows_staged_kernel(Args p) {
    constexpr int TW = 8 * G, NV = 4 * G;
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* codes = lds;                                            // [nb * 8][TW][32]
    float* d8_table = (float*)(codes + (size_t)p.nb * 8 * TW * 32);  // [nb * 8][TW]
    float* ds_table = d8_table + p.nb * 8 * TW;                      // [nb * 8][TW]
    float* reduce = ds_table + p.nb * 8 * TW;                        // [WAVES][NV][64]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int m_count = p.m;   // one pass: the launcher sends at most TW rows here
    const int n_tiles = (p.n + 31) >> 5;
    const size_t row_bytes = (size_t)p.nb * Blk<Q5>::BYTES;
    const int entries = p.nb * 8 * TW;

    // Steps of this wave: (tile, super-block) pairs, super-blocks wave, wave + 4, ... of each tile
    // of this workgroup in turn.
    const int my_blocks = (p.nb - wave + WAVES - 1) / WAVES;
    // (with DUAL every row tile counts twice: the first matrix's rows, then the second's)
    const int my_tiles = ((int)blockIdx.x < n_tiles ? (n_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0) *
                         (DUAL ? 2 : 1);
    const int total = my_tiles * my_blocks;
    auto tile_of = [&](int ordinal) { return (int)blockIdx.x + (DUAL ? ordinal >> 1 : ordinal) * (int)gridDim.x; };
    auto loadw = [&](WFrag& f, int j) {
        const int ordinal = j / my_blocks, kb = wave + (j % my_blocks) * WAVES;
        const int row = min(tile_of(ordinal) * 32 + l32, p.n - 1);
        const uint8_t* mat = DUAL && (ordinal & 1) ? p.w2 : p.w;
        const uint8_t* bp = (const uint8_t*)(to_gbytes(mat) + row * row_bytes + (size_t)kb * Blk<Q5>::BYTES);
        f.hdr = *(const uint4*)bp;
        if (Q5) f.qh = *(const uint4*)(bp + 16 + 16 * lh);
#pragma unroll
        for (int c = 0; c < 4; ++c) f.q[c] = *(const uint4*)(bp + Blk<Q5>::QS + 32 * c + 16 * lh);
    };

    // The activation: every (sub-block, row) entry is one Q8_1 block; its codes go to LDS as they
    // are, its scale and scale * (sum of codes) into the tables. The first round's loads are issued
    // before the first weight loads and consumed after them (loads return in issue order: asked for
    // after the weights, the activation, which sits in L2, would wait for HBM).
    constexpr int PER = 4;
    uint32_t head[PER];
    uint4 lo[PER], hi[PER];
    auto issue = [&](int base) {
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = min(base + u * WG, entries - 1);
            const int sub = idx / TW, tok = min(idx % TW, m_count - 1);
            const uint8_t* b = p.y + ((size_t)tok * p.stride_y + sub) * Q81_BYTES;
            head[u] = *(const uint32_t*)b;
            lo[u] = *(const uint4_a4*)(b + 4);
            hi[u] = *(const uint4_a4*)(b + 20);
        }
    };
    auto place = [&](int base) {
        const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = base + u * WG;
            if (idx < entries) {
                const bool real = idx % TW < m_count;
                const float d8 = real ? f16_bits_to_f32(head[u] & 0xFFFFu) : 0.f;
                d8_table[idx] = d8;
                ds_table[idx] = d8 * (float)dot16(ones, hi[u], dot16(ones, lo[u], 0));
                *(uint4*)(codes + (size_t)idx * 32) = lo[u];
                *(uint4*)(codes + (size_t)idx * 32 + 16) = hi[u];
            }
        }
    };
    constexpr int DEPTH = G == 1 && !Q5 ? 4 : 3;   // steps of weight loads a wave keeps in flight (registers)
    WFrag f[DEPTH];
    issue(threadIdx.x);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (d < total) loadw(f[d], d);
    place(threadIdx.x);
    for (int r = WG * PER; r < entries; r += WG * PER) {
        issue(r + threadIdx.x);
        place(r + threadIdx.x);
    }
    __syncthreads();

    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.f;

    // the lane's A operand: activation row l32 (rows the launch does not have repeat the live
    // ones; their results sit in registers nobody reads), codes 16 lh .. 16 lh + 15 of the sub-block
    const uint8_t* a_lane = codes + (l32 % TW) * 32 + 16 * lh;

    auto compute = [&](const WFrag& w, int kb) {
        const uint32_t w1 = w.hdr.y, w2 = w.hdr.z, w3 = w.hdr.w;
        const uint32_t sc_lo = w1 & 0x3F3F3F3Fu, mn_lo = w2 & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (w3 & 0x0F0F0F0Fu) | ((w1 >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((w3 >> 4) & 0x0F0F0F0Fu) | ((w2 >> 2) & 0x30303030u);
        const float d = f16_bits_to_f32(w.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(w.hdr.x >> 16);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t scs = ((s < 4 ? sc_lo : sc_hi) >> (8 * (s & 3))) & 0xFFu;
            const uint32_t mns = ((s < 4 ? mn_lo : mn_hi) >> (8 * (s & 3))) & 0xFFu;
            const float dsc = d * (float)scs, dmm = -(dmin * (float)mns);
            const v4i b = codes_of<Q5>(w.q[s >> 1], w.qh, s);
            const int sub = kb * 8 + s;
            const v4i a = *(const v4i*)(a_lane + (size_t)sub * TW * 32);
            // the accumulators start at the bit pattern of 1.5 * 2^23, so the dots leave the matrix
            // unit as floats (see the kernel above)
            constexpr int MAGIC_BITS = 0x4B400000;
            constexpr float MAGIC = 12582912.0f;
            v16i c;
#pragma unroll
            for (int v = 0; v < 16; ++v) c[v] = MAGIC_BITS;
            c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
            const float off = -MAGIC * dsc;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float4 t = *(const float4*)(d8_table + sub * TW + 8 * g + 4 * lh);
                const float4 u = *(const float4*)(ds_table + sub * TW + 8 * g + 4 * lh);
                acc[4 * g + 0] = fmaf(fmaf(__int_as_float(c[4 * g + 0]), dsc, off), t.x, fmaf(dmm, u.x, acc[4 * g + 0]));
                acc[4 * g + 1] = fmaf(fmaf(__int_as_float(c[4 * g + 1]), dsc, off), t.y, fmaf(dmm, u.y, acc[4 * g + 1]));
                acc[4 * g + 2] = fmaf(fmaf(__int_as_float(c[4 * g + 2]), dsc, off), t.z, fmaf(dmm, u.z, acc[4 * g + 2]));
                acc[4 * g + 3] = fmaf(fmaf(__int_as_float(c[4 * g + 3]), dsc, off), t.w, fmaf(dmm, u.w, acc[4 * g + 3]));
            }
            // one sub-block's tile at a time: left free, the scheduler starts all eight matrix
            // instructions of a step first and holds 8 x 16 result registers
            if (s & 1) __builtin_amdgcn_sched_barrier(0);
        }
    };

    float gate_keep[G];
    auto finish_tile = [&](int ordinal) {
        float* mine = reduce + wave * (NV * 64);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            mine[v * 64 + lane] = acc[v];
            acc[v] = 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < G; ++r) {
            const int v = wave * G + r;
            float sum = (reduce[v * 64 + lane] + reduce[(NV + v) * 64 + lane]) +
                        (reduce[(2 * NV + v) * 64 + lane] + reduce[(3 * NV + v) * 64 + lane]);
            if (DUAL && !(ordinal & 1)) { gate_keep[r] = sum; continue; }
            if (DUAL) {
                LkGateAct act;
                act.kind = p.gelu ? LK_GATE_GELU : LK_GATE_SILU;
                sum = lk_gated(act, gate_keep[r], sum, 0);
            }
            const int tok = (v >> 2) * 8 + lh * 4 + (v & 3), row = tile_of(ordinal) * 32 + l32;
            if (tok < m_count && row < p.n) p.dst[(size_t)tok * p.ldd + row] = sum;
        }
        __syncthreads();   // the partial tiles may be overwritten
    };

    if (my_blocks == 0) {   // rows shorter than four super-blocks: this wave only keeps the barriers
        for (int t = 0; t < my_tiles; ++t) finish_tile(t);
        return;
    }
    for (int j0 = 0; j0 < total; j0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int j = j0 + d;
            if (j < total) {
                compute(f[d], wave + (j % my_blocks) * WAVES);
                if (j + DEPTH < total) loadw(f[d], j + DEPTH);
                if ((j + 1) % my_blocks == 0) finish_tile(j / my_blocks);
            }
        }
    }
}

template <int G, bool DUAL, bool Q5, bool MULTI = false>
int resident_cap(int lds_bytes) {
    static std::mutex mu;
    static std::unordered_map<int, int> by_lds;
    std::lock_guard<std::mutex> lock(mu);
    auto it = by_lds.find(lds_bytes);
    if (it != by_lds.end()) return it->second;
    int r = 0;
    if (lds_bytes > lk_device().lds_bytes) {
        r = 0;
    } else if (lds_bytes > 48 * 1024 &&
               hipFuncSetAttribute((const void*)q4k_rows_mfma_kernel<G, DUAL, Q5, MULTI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        r = 0;
    } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q4k_rows_mfma_kernel<G, DUAL, Q5, MULTI>, WG,
                                                            (size_t)lds_bytes) != hipSuccess || r < 1) {
        (void)hipGetLastError();
        r = 1;
    }
    by_lds.emplace(lds_bytes, r);
    return r;
}

template <int G, bool DUAL, bool Q5, bool MULTI = false>
int launch_rows(const Args& a, hipStream_t stream) {
    const int lds_bytes = (lds_floats_table<G>(a.nb) + WAVES * 4 * G * 64) * (int)sizeof(float);
    const int per_cu = resident_cap<G, DUAL, Q5, MULTI>(lds_bytes);
    if (per_cu == 0) return LK_ERR_ARG;   // rows too long for the scale tables
    const int n_tiles = (a.n + 31) / 32 + (MULTI ? (a.n_b + 31) / 32 + (a.n_c + 31) / 32 : 0), groups = (a.m + TOK - 1) / TOK;
    if (groups > 65535) return LK_ERR_ARG;
    int cap = lk_device().cus * per_cu / groups;
    if (cap < 1) cap = 1;
    hipLaunchKernelGGL((q4k_rows_mfma_kernel<G, DUAL, Q5, MULTI>), dim3(n_tiles < cap ? n_tiles : cap, groups), dim3(WG), lds_bytes, stream, a);
    return lk_launch_status();
}

// The staged kernel for `a.m` <= 8 G rows, if its LDS image fits; -1 when it does not.
template <int G, bool DUAL, bool Q5>
int launch_staged(const Args& a, hipStream_t stream) {
    static std::mutex mu;
    static std::unordered_map<int, int> by_lds;
    const int lds_bytes = lds_bytes_staged<G>(a.nb);
    if (lds_bytes > lk_device().lds_bytes) return -1;
    int per_cu;
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = by_lds.find(lds_bytes);
        if (it == by_lds.end()) {
            int r = 0;
            if (lds_bytes > 48 * 1024 &&
                hipFuncSetAttribute((const void*)q4k_rows_staged_kernel<G, DUAL, Q5>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    lds_bytes) != hipSuccess) {
                (void)hipGetLastError();
                r = 0;
            } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q4k_rows_staged_kernel<G, DUAL, Q5>, WG,
                                                                    (size_t)lds_bytes) != hipSuccess || r < 1) {
                (void)hipGetLastError();
                r = 1;
            }
            it = by_lds.emplace(lds_bytes, r).first;
        }
        per_cu = it->second;
    }
    if (per_cu == 0) return -1;
    const int n_tiles = (a.n + 31) / 32, cap = lk_device().cus * per_cu;
    hipLaunchKernelGGL((q4k_rows_staged_kernel<G, DUAL, Q5>), dim3(n_tiles < cap ? n_tiles : cap), dim3(WG), lds_bytes, stream, a);
    return lk_launch_status();
}

// The expert-batched launch: grid (workgroups per expert, experts). A workgroup walks several row
// tiles per pass so that the tables of an expert's rows are staged by a few workgroups, not by one
// per tile.
template <int G, bool DUAL, bool Q5, bool KSPLIT>
int launch_moe(const Args& a, const MoeRows& m, int n_experts, hipStream_t stream) {
    static std::mutex mu;
    static std::unordered_map<int, int> by_lds;
    const int lds_bytes = (lds_floats_table<G>(a.nb) + WAVES * 4 * G * 64) * (int)sizeof(float);
    if (lds_bytes > lk_device().lds_bytes) return LK_ERR_ARG;
    int per_cu;
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = by_lds.find(lds_bytes);
        if (it == by_lds.end()) {
            int r = 0;
            if (lds_bytes > 48 * 1024 &&
                hipFuncSetAttribute((const void*)q4k_rows_moe_kernel<G, DUAL, Q5, KSPLIT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    lds_bytes) != hipSuccess) {
                (void)hipGetLastError();
                r = 0;
            } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q4k_rows_moe_kernel<G, DUAL, Q5, KSPLIT>, WG,
                                                                    (size_t)lds_bytes) != hipSuccess || r < 1) {
                (void)hipGetLastError();
                r = 1;
            }
            it = by_lds.emplace(lds_bytes, r).first;
        }
        per_cu = it->second;
    }
    if (per_cu == 0) return LK_ERR_ARG;
    const int n_tiles = (a.n + 31) / 32, units = KSPLIT ? n_tiles : (n_tiles + WAVES - 1) / WAVES;
    int per_expert = (2 * lk_device().cus * per_cu + n_experts - 1) / n_experts;
    if (per_expert < 2) per_expert = 2;
    if (per_expert > units) per_expert = units;
    hipLaunchKernelGGL((q4k_rows_moe_kernel<G, DUAL, Q5, KSPLIT>), dim3(per_expert, n_experts), dim3(WG), lds_bytes, stream, a, m);
    return lk_launch_status();
}

template <bool DUAL, bool KSPLIT>
int launch_moe_width(const Args& a, const MoeRows& m, int n_experts, int rows_hint, hipStream_t stream) {
    if (rows_hint <= 8) return launch_moe<1, DUAL, false, KSPLIT>(a, m, n_experts, stream);
    if (rows_hint <= 16) return launch_moe<2, DUAL, false, KSPLIT>(a, m, n_experts, stream);
    return launch_moe<4, DUAL, false, KSPLIT>(a, m, n_experts, stream);
}

template <bool DUAL>
int launch_moe_any(const Args& a, const MoeRows& m, int n_experts, int rows_hint, hipStream_t stream) {
    // rows of at most eight super-blocks (the expert matrices of the MoE models: k = 2048, 768): a wave per
    // row tile; longer rows: the four waves split a tile's super-blocks
    return a.nb <= 8 ? launch_moe_width<DUAL, false>(a, m, n_experts, rows_hint, stream)
                     : launch_moe_width<DUAL, true>(a, m, n_experts, rows_hint, stream);
}

template <bool DUAL, bool Q5>
int launch_any(const Args& a, hipStream_t stream) {
    // at most 8 / 16 activation rows in all: the fix-up runs on the registers those rows live in,
    // and the activation is staged in LDS when it fits there
    if (a.m <= 16) {
        // 16-row tiles (rows16_mfma.hip): half the matrix-unit time per weight, twice the tiles
        if (lk_rows16_serves(a.m, a.nb) && lk_tune_env("LK_TUNE_ROWS16_OFF") == 0 &&
            (a.m <= 8 || lk_tune_env("LK_TUNE_ROWS16_MAX8") == 0)) {
            LkRows16 r{};
            r.w[0] = a.w; r.w[1] = a.w2;
            r.dst[0] = a.dst;
            r.n[0] = r.n[1] = a.n;
            r.ldd[0] = a.ldd;
            r.count = DUAL ? 2 : 1;
            r.y = a.y; r.nb = a.nb; r.m = a.m; r.stride_y = a.stride_y; r.gelu = a.gelu;
            return lk_rows16_launch(r, DUAL, Q5, stream);
        }
    }
    if (a.m <= 8) {
        const int rc = launch_staged<1, DUAL, Q5>(a, stream);
        return rc >= 0 ? rc : launch_rows<1, DUAL, Q5>(a, stream);
    }
    if (a.m <= 16) {
        const int rc = launch_staged<2, DUAL, Q5>(a, stream);
        return rc >= 0 ? rc : launch_rows<2, DUAL, Q5>(a, stream);
    }
    return launch_rows<4, DUAL, Q5>(a, stream);
}

bool bad_rows_call(const void* w, const void* q8_1, const float* output, int size_m, int size_n, int size_k) {
    return !w || !q8_1 || !output || size_m < 0 || size_n < 0 || size_k <= 0 || size_k % 256 != 0 ||
           (((uintptr_t)w) & 15) != 0 || (((uintptr_t)q8_1) & 3) != 0;
}

}  // namespace

// Returns LK_OK, or the reason nothing was launched.
static int rows_plain(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k, int stride_y,
                      int ldd, bool q5, hipStream_t stream) {
    if (size_m == 0 || size_n == 0) return LK_OK;
    if (bad_rows_call(w, q8_1, output, size_m, size_n, size_k)) return LK_ERR_ARG;
    if (stride_y < size_k / 32 || ldd < size_n) return LK_ERR_ARG;
    Args a{(const uint8_t*)w, (const uint8_t*)q8_1, output, size_k / 256, size_n, size_m, stride_y, ldd, nullptr, 0};
    return q5 ? launch_any<false, true>(a, stream) : launch_any<false, false>(a, stream);
}

int lk_q4k_rows_mfma(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                     int stride_y, int ldd, hipStream_t stream) {
    return rows_plain(w, q8_1, output, size_m, size_n, size_k, stride_y, ldd, false, stream);
}

extern "C" int lk_dense_q4k_rows(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                                 void* stream) {
    return rows_plain(w, q8_1, output, size_m, size_n, size_k, size_k / 32, size_n, false, (hipStream_t)stream);
}

extern "C" void loken_dense_q4k_imma_m8_plain(const void* w, const void* q8_1, float* output, int size_m, int size_n,
                                              int size_k, void* stream) {
    (void)rows_plain(w, q8_1, output, size_m, size_n, size_k, size_k / 32, size_n, false, (hipStream_t)stream);
}

// Gate and up in one launch: output[m, n] = act(gate[n] . x[m]) * (up[n] . x[m]), act = SiLU or the
// tanh-form GELU. Replaces loken_dense_q4k_imma_m8_actmul (declared src/inference/moe_cuda/mod.rs:452-455,
// launcher cuda/moe/dense_q4k_imma_m8.cu:272-286).
static int rows_actmul(const void* gate, const void* up, const void* q8_1, float* output, int size_m, int size_n,
                       int size_k, int use_gelu, bool q5, hipStream_t stream) {
    if (size_m == 0 || size_n == 0) return LK_OK;
    if (bad_rows_call(gate, q8_1, output, size_m, size_n, size_k) || !up || (((uintptr_t)up) & 15) != 0) return LK_ERR_ARG;
    Args a{(const uint8_t*)gate, (const uint8_t*)q8_1, output, size_k / 256, size_n, size_m, size_k / 32, size_n,
           (const uint8_t*)up, use_gelu ? 1 : 0};
    return q5 ? launch_any<true, true>(a, stream) : launch_any<true, false>(a, stream);
}

extern "C" int lk_dense_q4k_rows_actmul(const void* gate, const void* up, const void* q8_1, float* output, int size_m,
                                        int size_n, int size_k, int use_gelu, void* stream) {
    return rows_actmul(gate, up, q8_1, output, size_m, size_n, size_k, use_gelu, false, (hipStream_t)stream);
}

extern "C" void loken_dense_q4k_imma_m8_actmul(const void* gate, const void* up, const void* q8_1, float* output,
                                               int size_m, int size_n, int size_k, int use_gelu, void* stream) {
    (void)rows_actmul(gate, up, q8_1, output, size_m, size_n, size_k, use_gelu, false, (hipStream_t)stream);
}

// Up to three Q4_K (q5 != 0: Q5_K) matrices over the same plain Q8_1 rows in one launch (q + k + v of a
// decode step): outputs[i] is [size_m, sizes_n[i]] f32. The reference issues one
// loken_dense_q4k_imma_m8_plain per matrix (dense_q4k_imma_m8_matmul, src/inference/moe_cuda/dense/
// imma.rs:82-135); the results equal those launches' bit for bit. One launch at any row count (the 16-row
// tiles up to 16 rows, the 32-row tiles above); rows too long for the kernels' LDS tables fall back to one
// launch per matrix.
extern "C" int lk_dense_q4k_rows_multi(const void* const* weights, float* const* outputs, const int* sizes_n, int count,
                                       const void* q8_1, int size_m, int size_k, int q5, void* stream) {
    if (!weights || !outputs || !sizes_n || count < 1 || count > 3) return LK_ERR_ARG;
    if (size_m == 0) return LK_OK;
    for (int i = 0; i < count; ++i)
        if (sizes_n[i] > 0 && bad_rows_call(weights[i], q8_1, outputs[i], size_m, sizes_n[i], size_k)) return LK_ERR_ARG;
    const int nb = size_k / 256;
    if (lk_rows16_serves(size_m, nb) && lk_tune_env("LK_TUNE_ROWS16_OFF") == 0 &&
        (size_m <= 8 || lk_tune_env("LK_TUNE_ROWS16_MAX8") == 0)) {
        LkRows16 r{};
        for (int i = 0; i < count; ++i) {
            if (sizes_n[i] <= 0) continue;
            r.w[r.count] = (const uint8_t*)weights[i];
            r.dst[r.count] = outputs[i];
            r.n[r.count] = r.ldd[r.count] = sizes_n[i];
            ++r.count;
        }
        if (r.count == 0) return LK_OK;
        r.y = (const uint8_t*)q8_1; r.nb = nb; r.m = size_m; r.stride_y = size_k / 32;
        return lk_rows16_launch(r, false, q5 != 0, (hipStream_t)stream);
    }
    if (size_m > 16 && lk_tune_env("LK_TUNE_ROWS_MULTI_OFF") == 0) {
        // more rows: the 32-row-tile kernel walks the tiles of all the matrices in one launch
        Args a{};
        int live = 0;
        for (int i = 0; i < count; ++i) {
            if (sizes_n[i] <= 0) continue;
            if (live == 0) { a.w = (const uint8_t*)weights[i]; a.dst = outputs[i]; a.n = a.ldd = sizes_n[i]; }
            else if (live == 1) { a.w_b = (const uint8_t*)weights[i]; a.dst_b = outputs[i]; a.n_b = a.ldd_b = sizes_n[i]; }
            else { a.w_c = (const uint8_t*)weights[i]; a.dst_c = outputs[i]; a.n_c = a.ldd_c = sizes_n[i]; }
            ++live;
        }
        if (live == 0) return LK_OK;
        a.y = (const uint8_t*)q8_1; a.nb = nb; a.m = size_m; a.stride_y = size_k / 32;
        if (live > 1) {
            const int rc = q5 ? launch_rows<4, false, true, true>(a, (hipStream_t)stream) : launch_rows<4, false, false, true>(a, (hipStream_t)stream);
            if (rc == LK_OK) return rc;
        }
    }
    for (int i = 0; i < count; ++i) {
        const int rc = rows_plain(weights[i], q8_1, outputs[i], size_m, sizes_n[i], size_k, size_k / 32, sizes_n[i], q5 != 0,
                                  (hipStream_t)stream);
        if (rc != LK_OK) return rc;
    }
    return LK_OK;
}

// Gate and up in one launch with the result handed on as Q8_1: q8_1_out[m][size_n / 32] blocks =
// lk_quantize_q8_1(act(gate . x) * (up . x)), byte for byte, so the down projection of a layer reads it
// without the f32 round trip and the quantizer launch in between (what lk_mmvq_pair_act_q8_1 is to the
// mat-vec pair launch). Up to 16 rows the 16-row-tile kernel at four tiles per workgroup (rows of 2048 or
// 4096 values), above them the 32-row tiles (a tile's rows are one block; any row length its tables hold);
// size_n a multiple of 32; anything else returns LK_ERR_ARG (take the f32 form and the quantizer). q5 != 0: Q5_K. No counterpart in the reference, whose dense_q4k_imma_m8_act_mul writes f32
// (src/inference/moe_cuda/dense/imma.rs:320-400).
extern "C" int lk_dense_q4k_rows_actmul_q8_1(const void* gate, const void* up, const void* q8_1, void* q8_1_out, int size_m,
                                             int size_n, int size_k, int use_gelu, int q5, void* stream) {
    if (size_m == 0 || size_n == 0) return LK_OK;
    if (!gate || !up || !q8_1 || !q8_1_out || size_m < 0 || size_n < 0 || size_n % 32 != 0 || size_k <= 0 ||
        size_k % 256 != 0 || ((((uintptr_t)gate) | ((uintptr_t)up)) & 15) != 0 ||
        ((((uintptr_t)q8_1) | ((uintptr_t)q8_1_out)) & 3) != 0)
        return LK_ERR_ARG;
    const int nb = size_k / 256;
    if (size_m > 16) {   // the 32-row tiles: a tile's rows are one block
        Args a{(const uint8_t*)gate, (const uint8_t*)q8_1, nullptr, nb, size_n, size_m, size_k / 32, size_n,
               (const uint8_t*)up, use_gelu ? 1 : 0};
        a.q81_dst = (uint8_t*)q8_1_out;
        a.q81_stride = size_n / 32;
        return q5 ? launch_rows<4, true, true>(a, (hipStream_t)stream) : launch_rows<4, true, false>(a, (hipStream_t)stream);
    }
    if ((nb != 8 && nb != 16) || !lk_rows16_serves(size_m, nb)) return LK_ERR_ARG;
    LkRows16 r{};
    r.w[0] = (const uint8_t*)gate; r.w[1] = (const uint8_t*)up;
    r.n[0] = r.n[1] = size_n;
    r.count = 2;
    r.y = (const uint8_t*)q8_1; r.nb = nb; r.m = size_m; r.stride_y = size_k / 32; r.gelu = use_gelu ? 1 : 0;
    r.q81_dst = (uint8_t*)q8_1_out; r.q81_stride = size_n / 32;
    return lk_rows16_launch(r, true, q5 != 0, (hipStream_t)stream);
}

// The Q5_K siblings (loken_dense_q5k_imma_m8_plain / _actmul, declared src/inference/moe_cuda/mod.rs:459-466,
// picked by dtype at src/inference/moe_cuda/dense/imma.rs:113-116,362-365): the same kernels with the
// fifth-bit plane folded into the codes.
extern "C" int lk_dense_q5k_rows(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                                 void* stream) {
    return rows_plain(w, q8_1, output, size_m, size_n, size_k, size_k / 32, size_n, true, (hipStream_t)stream);
}

extern "C" void loken_dense_q5k_imma_m8_plain(const void* w, const void* q8_1, float* output, int size_m, int size_n,
                                              int size_k, void* stream) {
    (void)rows_plain(w, q8_1, output, size_m, size_n, size_k, size_k / 32, size_n, true, (hipStream_t)stream);
}

extern "C" int lk_dense_q5k_rows_actmul(const void* gate, const void* up, const void* q8_1, float* output, int size_m,
                                        int size_n, int size_k, int use_gelu, void* stream) {
    return rows_actmul(gate, up, q8_1, output, size_m, size_n, size_k, use_gelu, true, (hipStream_t)stream);
}

extern "C" void loken_dense_q5k_imma_m8_actmul(const void* gate, const void* up, const void* q8_1, float* output,
                                               int size_m, int size_n, int size_k, int use_gelu, void* stream) {
    (void)rows_actmul(gate, up, q8_1, output, size_m, size_n, size_k, use_gelu, true, (hipStream_t)stream);
}

// Expert-batched Q4_K rows on the matrix unit, for routings that give an expert a handful of rows: the
// shape of lk_dense_q4k_rows per expert, every expert's weights read once per 8 / 16 / 32 of its rows.
// The reference reaches these loads through its tiled expert kernel (launch_mmq_moe_gguf_q4_k,
// src/tensor/quantized/mmq.rs:274-286) or one mat-vec per pair; it has no launcher of this shape.
//   weights        [n_experts] matrices of size_n rows, expert_bytes apart
//   weights_second nullable; when given (same layout) the output is act(w . x) * (w2 . x), act 0 SiLU / 1 GELU
//   q8_1           plain Q8_1 rows, stride_blocks blocks apart
//   bounds         [n_experts + 1]: expert e owns sorted rows [bounds[e], bounds[e + 1])
//   src_rows       nullable: sorted row -> row of q8_1 (else the sorted row itself)
//   dst_rows       nullable: sorted row -> row of output (else the sorted row itself)
//   rows_hint      rows an expert is expected to own (picks the pass width; any count is served)
extern "C" int lk_moe_q4k_rows_grouped(const void* weights, const void* weights_second, int act, const void* q8_1,
                                       int stride_blocks, const int32_t* bounds, const int32_t* src_rows,
                                       const int32_t* dst_rows, float* output, int ldd, int n_experts,
                                       int64_t expert_bytes, int size_n, int size_k, int rows_hint, void* stream) {
    if (n_experts == 0 || size_n == 0) return LK_OK;
    if (!weights || !q8_1 || !bounds || !output || n_experts < 0 || n_experts > 65535 || size_n < 0 || size_k <= 0 ||
        size_k % 256 != 0 || stride_blocks < size_k / 32 || ldd < size_n || expert_bytes % 16 != 0)
        return LK_ERR_ARG;
    if ((((uintptr_t)weights) & 15) != 0 || (((uintptr_t)weights_second) & 15) != 0 || (((uintptr_t)q8_1) & 3) != 0)
        return LK_ERR_ARG;
    Args a{(const uint8_t*)weights, (const uint8_t*)q8_1, output, size_k / 256, size_n, 0, stride_blocks, ldd,
           (const uint8_t*)weights_second, act ? 1 : 0};
    const MoeRows m{bounds, src_rows, dst_rows, expert_bytes};
    if (rows_hint < 1) rows_hint = 1;
    {
        // rows of at most eight super-blocks: a wave per 16-row tile, passes of 8 or 16 rows (rows16_moe.hip)
        LkRows16 r{};
        r.w[0] = (const uint8_t*)weights; r.w[1] = (const uint8_t*)weights_second;
        r.dst[0] = output;
        r.n[0] = r.n[1] = size_n;
        r.ldd[0] = ldd;
        r.count = weights_second ? 2 : 1;
        r.y = (const uint8_t*)q8_1; r.nb = size_k / 256; r.stride_y = stride_blocks; r.gelu = act ? 1 : 0;
        const LkRows16Experts ex{bounds, src_rows, dst_rows, expert_bytes};
        const int rc = lk_rows16_launch_experts(r, ex, n_experts, weights_second != nullptr, rows_hint, (hipStream_t)stream);
        if (rc >= 0) return rc;
    }
    return weights_second ? launch_moe_any<true>(a, m, n_experts, rows_hint, (hipStream_t)stream)
                          : launch_moe_any<false>(a, m, n_experts, rows_hint, (hipStream_t)stream);
}

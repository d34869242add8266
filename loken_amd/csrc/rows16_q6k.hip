// Q6_K weights x at most eight Q8_1 activation rows on v_mfma_i32_16x16x64_i8: the Q6_K member of
// the small-batch family in rows16_mfma.hip (`down` and a Q6_K lm_head of a decode step at 2..8
// sequences). The reference has no matrix-unit kernel for this format at these row counts; its
// Q6_K rows go through vec_dot_q6_K_q8_1 (cuda/moe/gguf.cuh:782-816, 1089-1108) one activation row
// at a time. The sums formed here are the same: per 16-value group,
// d * scale[g] * d8 * sum (code - 32) * a.
//
// Shape of the work. A wave owns 16 weight rows; lane l holds row l % 16 and the sixteen K values of
// lane group l / 16. A Q6_K group (16 values, its own int8 scale) is exactly one lane group's share,
// so an instruction's four lane groups hold four groups of a row: the 64 consecutive bytes of `ql`
// at 64 hb (hb: which 128 values of the super-block), low nibbles for one instruction, high nibbles
// for the next, with the two high bits of each code from `qh`. Every byte of ql is loaded once.
// The dots of the four groups must stay apart. With at most FOUR activation rows the sixteen slots
// of the activation operand are (group) x (row): slot i holds row i % 4's codes of group i / 4 in
// that group's lane group and zeros in the other three, and lane l, register v is (weight row
// l % 16, group l / 16, activation row v). With up to EIGHT rows the slots are (one of two groups) x
// (row) and each set of weight registers runs twice, once against groups 0, 1 and once against
// groups 2, 3: lane l, register v is (weight row l % 16, group l / 32 or 2 + l / 32, activation row
// 4 ((l / 16) % 2) + v). The codes go in signed (code - 32 fits int8), so no offset term remains.
//
// Loads. Lane = row loads of this format would be 16 bytes at 2-byte alignment, one cache line per lane,
// and measure at a third of the rate of the same bytes read as aligned consecutive pieces. So a wave
// owns a GRANULE of a row tile: eight consecutive super-blocks, 8 x 210 = 1680 bytes = 105 whole
// 16-byte pieces per row, which start on a 16-byte boundary when the row does (rows are a multiple of
// eight super-blocks: k a multiple of 2048). Super-block i of a granule lies in pieces 13 i .. 13 i + 13
// at byte 2 i of the first: the wave loads those 14 pieces of its 16 rows as consecutive lanes along a
// row (aligned, a few whole lines per load), turns them through its own LDS buffer, and reads each
// operand back as the two pieces that hold it, shifted by the 2 i bytes, which is a constant in the
// eight-fold unrolled step. A workgroup is up to sixteen waves: the granules of one or more row
// tiles, their partial tiles added through LDS. The activation codes are staged in LDS once per
// workgroup (for k = 14336 and eight rows that is 112 KiB of the CU's 160), beside the table of d8
// and a run of zeros that the zero lanes read. Loads run D super-blocks ahead of the arithmetic, across
// the wave's tiles, in a loop body without branches around them, so the counters the compiler waits
// on are exact.

#include "lk_common.h"
#include "rows16.h"

#include <mutex>
#include <type_traits>
#include <unordered_map>

namespace {

constexpr int MAX_WAVES = 16;
constexpr int TILE = 16;
constexpr int GRAN = 8;                 // super-blocks of a wave's granule
constexpr int BLOCK_PIECES = 14;        // 16-byte pieces that hold one super-block of a granule
constexpr int WPITCH = BLOCK_PIECES * 16 + 16;   // bytes between rows of a wave's buffer: 16 rows on 16 bank groups
constexpr int WBUF = TILE * WPITCH;     // bytes of a wave's buffer

struct Args {
    const uint8_t* w;
    const uint8_t* y;     // Q8_1 rows
    float* dst;
    int nb;               // super-blocks per weight row
    int n;                // weight rows
    int m;                // activation rows
    int stride_y;         // Q8_1 blocks between activation rows
    int ldd;              // floats between output rows
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct WFrag {
    u32x4 ql[2];   // [hb]: bytes 64 hb + 16 (l / 16) of ql
    u32x4 qh[2];   // [hb]: bytes 32 hb + 16 ((l / 16) % 2) of qh
    u32x4 sc;      // the 16 group scales
    uint32_t d;    // f16 bits
};

// Sixteen bytes that start PHASE bytes into `lo` and run on into `hi` (PHASE even, below 16).
template <int PHASE>
static __device__ __forceinline__ u32x4 shifted(const u32x4& lo, const u32x4& hi) {
    const uint32_t in[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    constexpr int K = PHASE / 4;
    u32x4 out;
#pragma unroll
    for (int e = 0; e < 4; ++e)
        out[e] = PHASE % 4 ? __builtin_amdgcn_alignbyte(in[e + K + 1], in[e + K], PHASE % 4) : in[e + K];
    return out;
}

template <int TOKS>
static __host__ __device__ constexpr int lds_bytes_for(int nb, int waves) {
    // codes [nb * 8][TOKS][32], zeros, d8 [nb * 8][TOKS] floats, a buffer per wave (which also holds the
    // wave's partial tile of the reduction)
    return nb * 8 * TOKS * 32 + TOKS * 256 + nb * 8 * TOKS * 4 + waves * WBUF;
}

// TOKS: the activation rows a launch serves. 4: one instruction per set of weight registers (slots =
// group x row). 8: two (slots = one of two groups x row). 16: four (slots = rows; the activation live in
// one lane group per instruction; lane l, register v is (weight row l % 16, activation row 4 (l / 16) + v)
// for each of the four groups, so a lane's sums are complete across groups).
// D: super-blocks of loads a wave keeps in flight (4 in workgroups of at most eight waves, else 2).
// tw: row tiles of a workgroup; a tile's nb / 8 granules go to as many waves.
template <int TOKS, int D>
__global__ __launch_bounds__(D == 4 ? 512 : 1024, 1) void q6k_rows16_kernel(Args p, int n_tiles, int tw) {
    constexpr bool T8 = TOKS == 8, T16 = TOKS == 16;
    // grid.y: the activation rows in sets of TOKS, a set per workgroup (the weights are read once per set)
    const int set = (int)blockIdx.y;
    const uint8_t* const act_rows = p.y + (size_t)set * TOKS * p.stride_y * Q81_BYTES;
    float* const out_rows = p.dst + (size_t)set * TOKS * p.ldd;
    const int m_rows = min(TOKS, p.m - set * TOKS);
    constexpr int ZERO_BYTES = TOKS * 256;   // the zero lanes' run: the largest offset a step adds, and 16
    constexpr int BLK = TOKS * 32;       // LDS bytes of one Q8_1 block's codes, all rows
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* codes = lds;                                               // [nb * 8][TOKS][32]
    uint8_t* zeros = codes + (size_t)p.nb * 8 * BLK;                    // ZERO_BYTES
    float* table = (float*)(zeros + ZERO_BYTES);                        // [nb * 8][TOKS]: d8
    uint8_t* wbufs = (uint8_t*)(table + p.nb * 8 * TOKS);               // [waves][16][WPITCH]

    const int WG = (int)blockDim.x;
    const int S = p.nb / GRAN;           // waves that share a tile
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tsel = wave / S, gq = wave % S;
    const int l16 = lane & 15, grp = lane >> 4;
    const size_t row_bytes = (size_t)p.nb * Q6K_BYTES;
    const int entries = p.nb * 8 * TOKS;
    const int n_groups = (n_tiles + tw - 1) / tw;
    const int stride = (int)gridDim.x;
    const int my_passes = (int)blockIdx.x < n_groups ? (n_groups - (int)blockIdx.x + stride - 1) / stride : 0;
    uint8_t* wbuf = wbufs + (size_t)wave * WBUF;

    // ---- the activation: entry (Q8_1 block, row), loads issued before the first weight loads
    constexpr int PER = 4;
    uint32_t head[PER];
    uint4 lo[PER], hi[PER];
    auto issue = [&](int base) {
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = min(base + u * WG, entries - 1);
            const int sub = idx / TOKS, tok = min(idx % TOKS, m_rows - 1);
            const uint8_t* b = act_rows + ((size_t)tok * p.stride_y + sub) * Q81_BYTES;
            head[u] = *(const uint32_t*)b;
            lo[u] = *(const uint4_a4*)(b + 4);
            hi[u] = *(const uint4_a4*)(b + 20);
        }
    };
    auto place = [&](int base) {
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = base + u * WG;
            if (idx < entries) {
                const bool real = idx % TOKS < m_rows;
                table[idx] = real ? f16_bits_to_f32(head[u] & 0xFFFFu) : 0.f;
                const uint32_t keep = real ? 0xFFFFFFFFu : 0u;   // rows the launch does not have: zeros
                *(uint4*)(codes + (size_t)idx * 32) = make_uint4(lo[u].x & keep, lo[u].y & keep, lo[u].z & keep, lo[u].w & keep);
                *(uint4*)(codes + (size_t)idx * 32 + 16) = make_uint4(hi[u].x & keep, hi[u].y & keep, hi[u].z & keep, hi[u].w & keep);
            }
        }
    };

    // ---- the weight loads: load u of a super-block is piece 64 u + lane of its 16 x 14, row after row
    constexpr int LOADS = (TILE * BLOCK_PIECES + 63) / 64;   // 4, the last half used
    uint32_t w_off[LOADS];   // where the piece goes in the wave's buffer
    int w_row[LOADS], w_piece[LOADS];
#pragma unroll
    for (int u = 0; u < LOADS; ++u) {
        const int id = min(64 * u + lane, TILE * BLOCK_PIECES - 1);
        w_row[u] = id / BLOCK_PIECES;
        w_piece[u] = id % BLOCK_PIECES;
        w_off[u] = (uint32_t)(w_row[u] * WPITCH + w_piece[u] * 16);
    }
    // the lane's LOADS addresses of super-block 0 of this wave's granule of the tile of `pass` (past the
    // last tile: the last)
    struct Bases {
        const uint8_t* at[LOADS];
    };
    auto bases_of = [&](int pass) {
        const int tile = min(((int)blockIdx.x + pass * stride) * tw + tsel, n_tiles - 1);
        Bases b;
#pragma unroll
        for (int u = 0; u < LOADS; ++u) {
            const int row = min(tile * TILE + w_row[u], p.n - 1);
            b.at[u] = (const uint8_t*)(to_gbytes(p.w) + row * row_bytes + (size_t)gq * (GRAN * Q6K_BYTES) + w_piece[u] * 16);
        }
        return b;
    };
    struct Pieces {
        u32x4 r[LOADS];
    };
    // super-block I of the granule: pieces 13 I .. 13 I + 13
    auto issue_block = [&](Pieces& f, const Bases& b, int i) {
#pragma unroll
        for (int u = 0; u < LOADS; ++u) f.r[u] = *(const u32x4*)(b.at[u] + i * (13 * 16));
    };
    auto store_block = [&](const Pieces& f) {
#pragma unroll
        for (int u = 0; u < LOADS; ++u)
            if (64 * u + lane < TILE * BLOCK_PIECES) *(u32x4*)(wbuf + w_off[u]) = f.r[u];
    };
    // the lane's operands of the super-block in the buffer, which lies PHASE bytes into its first piece
    const uint8_t* w_lane = wbuf + l16 * WPITCH;
    auto frag_of = [&](auto phase_c) {
        constexpr int PHASE = decltype(phase_c)::value;
        auto piece_at = [&](int c) {   // sixteen bytes at byte c of the super-block
            const u32x4 lo = *(const u32x4*)(w_lane + c);
            if constexpr (PHASE == 0) return lo;
            else return shifted<PHASE>(lo, *(const u32x4*)(w_lane + c + 16));
        };
        WFrag f;
        f.ql[0] = piece_at(16 * grp);
        f.ql[1] = piece_at(64 + 16 * grp);
        f.qh[0] = piece_at(128 + 16 * (grp & 1));
        f.qh[1] = piece_at(160 + 16 * (grp & 1));
        f.sc = piece_at(192);
        f.d = *(const uint16_t*)(w_lane + 208 + PHASE);
        return f;
    };

    // ---- the lane's pieces of the activation operand (zeros where its lane group is not the slot's)
    const uint8_t *pa, *pb = zeros;
    int step_a, step_b = 0;
    if constexpr (T16) {
        // slot l16 is row l16; the lane's group is live in the instruction of that group alone
        pa = codes + (grp >> 1) * BLK + l16 * 32 + 16 * (grp & 1);
        step_a = 8 * BLK;
    } else if constexpr (T8) {
        const int sel = l16 >> 3, tok = l16 & 7;
        const bool live_a = grp < 2 && grp == sel, live_b = grp >= 2 && grp - 2 == sel;
        pa = live_a ? codes + tok * 32 + 16 * grp : zeros;
        pb = live_b ? codes + BLK + tok * 32 + 16 * (grp - 2) : zeros;
        step_a = live_a ? 8 * BLK : 0;
        step_b = live_b ? 8 * BLK : 0;
    } else {
        const int sel = l16 >> 2, tok = l16 & 3;
        const bool live = grp == sel;
        pa = live ? codes + (grp >> 1) * BLK + tok * 32 + 16 * (grp & 1) : zeros;
        step_a = live ? 8 * BLK : 0;
    }
    // the lane's results: 8 rows: groups grp / 2 and 2 + grp / 2, rows 4 (grp % 2) + v; 4 rows: group grp,
    // row v; 16 rows: every group, rows 4 grp + v
    const float* t_lane = T16 ? table + 4 * grp : T8 ? table + 4 * (grp & 1) : table + (grp >> 1) * TOKS;
    const int sh_sc = T16 ? 0 : T8 ? 8 * (grp >> 1) : 8 * grp;
    const int sh_qh = 2 * (grp >> 1);

    float acc[4] = {0.f, 0.f, 0.f, 0.f};

    auto compute = [&](const WFrag& w, int kb, bool live) {
        constexpr int MAGIC_BITS = 0x4B400000;
        constexpr float MAGIC = 12582912.0f;
        const float d = live ? f16_bits_to_f32(w.d) : 0.f;
        const uint8_t* a_blk = pa + (size_t)kb * step_a;
        const uint8_t* b_blk = pb + (size_t)kb * step_b;
        const float* t_blk = t_lane + kb * 8 * TOKS;
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            u32x4 qhp = w.qh[hb] >> (uint32_t)sh_qh;
#pragma unroll
            for (int nb2 = 0; nb2 < 2; ++nb2) {
                // the lane's sixteen signed codes: group 8 hb + 4 nb2 + grp of the row
                v4i b;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t nib = nb2 ? (w.ql[hb][e] >> 4) & 0x0F0F0F0Fu : w.ql[hb][e] & 0x0F0F0F0Fu;
                    const uint32_t up = nb2 ? qhp[e] & 0x30303030u : (qhp[e] << 4) & 0x30303030u;
                    b[e] = (int)(((nib | up) + 0x60606060u) ^ 0x80808080u);
                }
                const int blk = 4 * hb + 2 * nb2;   // the unit's two Q8_1 blocks: blk, blk + 1
                const uint32_t scw = w.sc[2 * hb + nb2] >> (uint32_t)sh_sc;
                // The accumulators start at the bit pattern of 1.5 * 2^23: an integer of magnitude
                // below 2^22 added to that pattern is the float 1.5 * 2^23 + integer, so the dots leave
                // the matrix unit as floats. The offset comes off in the first fused multiply-add,
                // exactly: d * scale is an f16 times an int8 (18 significant bits), MAGIC * d * scale
                // has 20, neither product rounds, and the fma rounds dot * d * scale once.
                const v4i magic = {MAGIC_BITS, MAGIC_BITS, MAGIC_BITS, MAGIC_BITS};
                if constexpr (T16) {
                    // instruction g: the activation of group g alone (zeros in the other lane groups)
                    const v4i a_live = *(const v4i*)(a_blk + blk * BLK);
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        v4i a;
#pragma unroll
                        for (int e = 0; e < 4; ++e) a[e] = grp == g ? a_live[e] : 0;
                        const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, magic, 0, 0, 0);
                        const float dsc = d * (float)(int)__builtin_amdgcn_sbfe(scw, 8 * g, 8);
                        const float off = -MAGIC * dsc;
                        const float4 t = *(const float4*)(t_blk + (blk + (g >> 1)) * TOKS);
                        const float d8[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
                        for (int v = 0; v < 4; ++v) acc[v] = fmaf(fmaf(__int_as_float(c[v]), dsc, off), d8[v], acc[v]);
                    }
                } else if constexpr (T8) {
                    const v4i a0 = *(const v4i*)(a_blk + blk * BLK);
                    const v4i a1 = *(const v4i*)(b_blk + blk * BLK);
                    const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b, magic, 0, 0, 0);
                    const v4i c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b, magic, 0, 0, 0);
                    const float dsc0 = d * (float)(int)__builtin_amdgcn_sbfe(scw, 0, 8);
                    const float dsc1 = d * (float)(int)__builtin_amdgcn_sbfe(scw, 16, 8);
                    const float off0 = -MAGIC * dsc0, off1 = -MAGIC * dsc1;
                    const float4 t0 = *(const float4*)(t_blk + blk * TOKS);
                    const float4 t1 = *(const float4*)(t_blk + (blk + 1) * TOKS);
                    const float d80[4] = {t0.x, t0.y, t0.z, t0.w}, d81[4] = {t1.x, t1.y, t1.z, t1.w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        acc[v] = fmaf(fmaf(__int_as_float(c0[v]), dsc0, off0), d80[v], acc[v]);
                        acc[v] = fmaf(fmaf(__int_as_float(c1[v]), dsc1, off1), d81[v], acc[v]);
                    }
                } else {
                    const v4i a0 = *(const v4i*)(a_blk + blk * BLK);
                    const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b, magic, 0, 0, 0);
                    const float dsc0 = d * (float)(int)__builtin_amdgcn_sbfe(scw, 0, 8);
                    const float off0 = -MAGIC * dsc0;
                    const float4 t0 = *(const float4*)(t_blk + blk * TOKS);
                    const float d80[4] = {t0.x, t0.y, t0.z, t0.w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[v] = fmaf(fmaf(__int_as_float(c0[v]), dsc0, off0), d80[v], acc[v]);
                }
                // One unit at a time: the sums are wanted here, not where they are next read. Left free, the
                // compiler sinks every unit's fix-up to the end of the block, keeps all the result tiles
                // alive and runs out of registers.
#pragma unroll
                for (int v = 0; v < 4; ++v) asm volatile("" : "+v"(acc[v]));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // Adds the partial tiles of the workgroup's row tiles of `pass` and writes them. A wave's partial
    // tile ([4][64] floats) lies at the start of its own buffer: the wave is past its last read of the
    // buffer when it gets here, and stores the next super-block only after the second barrier.
    auto finish = [&](int pass) {
        float* mine = (float*)wbuf;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            mine[v * 64 + lane] = acc[v];
            acc[v] = 0.f;
        }
        __syncthreads();
        // 8 rows: output (tile ts, register v, lane l < 32) adds the S waves' lanes l and l + 32; 4 rows:
        // output (ts, v, l < 16) adds their lanes l, l + 16, l + 32, l + 48; 16 rows: output (ts, v, l < 64)
        // adds their lanes l
        constexpr int LANES = T16 ? 64 : T8 ? 32 : 16, PER_TILE = 4 * LANES;
        for (int o = threadIdx.x; o < PER_TILE * tw; o += WG) {
            const int ts = o / PER_TILE, v = (o / LANES) & 3, l = o % LANES;
            float sum = 0.f;
            for (int sw = 0; sw < S; ++sw) {
                const float* col = (const float*)(wbufs + (size_t)(ts * S + sw) * WBUF) + v * 64 + l;
                if (T16) sum += col[0];
                else if (T8) sum += col[0] + col[32];
                else sum += (col[0] + col[16]) + (col[32] + col[48]);
            }
            const int tile = ((int)blockIdx.x + pass * stride) * tw + ts;
            const int tok = T16 ? 4 * (l >> 4) + v : T8 ? 4 * ((l >> 4) & 1) + v : v, row = tile * TILE + (l & 15);
            if (tile < n_tiles && tok < m_rows && row < p.n) out_rows[(size_t)tok * p.ldd + row] = sum;
        }
        __syncthreads();   // the buffers may be overwritten
    };

    Pieces ring[D];
    issue(threadIdx.x);
    // the load cursor runs D super-blocks ahead of the arithmetic: (pass, super-block of the granule)
    int l_pass = 0;
    Bases l_bases = bases_of(0);
    if (my_passes > 0) {
#pragma unroll
        for (int i = 0; i < D; ++i) issue_block(ring[i], l_bases, i);
    }
    place(threadIdx.x);
    for (int r = WG * PER; r < entries; r += WG * PER) {
        issue(r + threadIdx.x);
        place(r + threadIdx.x);
    }
    for (int i = threadIdx.x * 16; i < ZERO_BYTES; i += WG * 16) *(uint4*)(zeros + i) = make_uint4(0, 0, 0, 0);
    __syncthreads();

    for (int pass = 0; pass < my_passes; ++pass) {
        auto step = [&](auto i_c) {
            constexpr int I = decltype(i_c)::value;
            store_block(ring[I % D]);
            // the super-block D ahead goes out into the registers just stored: this tile's, or the next
            // tile's (past the last tile the last one again: a load nobody waits for)
            if constexpr (I + D == GRAN) {
                l_pass = min(pass + 1, my_passes - 1);
                l_bases = bases_of(l_pass);
            }
            issue_block(ring[I % D], l_bases, (I + D) % GRAN);
            compute(frag_of(std::integral_constant<int, 2 * I>{}), gq * GRAN + I, true);
        };
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 3>{});
        step(std::integral_constant<int, 4>{});
        step(std::integral_constant<int, 5>{});
        step(std::integral_constant<int, 6>{});
        step(std::integral_constant<int, 7>{});
        finish(pass);
    }
}

template <int TOKS, int D>
int launch_shape(const Args& a, int tw, int sets, hipStream_t stream) {
    static std::mutex mu;
    static std::unordered_map<int, int> by_lds;
    const int waves = tw * (a.nb / GRAN);
    const int lds_bytes = lds_bytes_for<TOKS>(a.nb, waves);
    if (lds_bytes > lk_device().lds_bytes) return -1;
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = by_lds.find(lds_bytes);
        if (it == by_lds.end()) {
            int ok = 1;
            if (lds_bytes > 48 * 1024 &&
                hipFuncSetAttribute((const void*)q6k_rows16_kernel<TOKS, D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    lds_bytes) != hipSuccess) {
                (void)hipGetLastError();
                ok = 0;
            }
            it = by_lds.emplace(lds_bytes, ok).first;
        }
        if (!it->second) return -1;
    }
    const int n_tiles = (a.n + TILE - 1) / TILE, groups = (n_tiles + tw - 1) / tw;
    // every workgroup as equal a share of the tile groups as the count allows
    int cap = lk_device().cus * (lds_bytes <= lk_device().lds_bytes / 2 && waves <= 8 ? 2 : 1) / sets;
    const int forced = lk_tune_env("LK_TUNE_ROWS16_WGS");
    if (forced > 0) cap = forced;
    const int passes = (groups + cap - 1) / cap;
    const int wgs = (groups + passes - 1) / passes;
    hipLaunchKernelGGL((q6k_rows16_kernel<TOKS, D>), dim3(wgs, sets), dim3(64 * waves), lds_bytes, stream, a, n_tiles, tw);
    return lk_launch_status();
}

template <int TOKS>
int launch(const Args& a, hipStream_t stream, int sets = 1) {
    // Tiles per workgroup: as many as its sixteen waves and LDS hold while every CU still gets a workgroup.
    const int s = a.nb / GRAN, n_tiles = (a.n + TILE - 1) / TILE, cus = lk_device().cus;
    int tw = 1;
    while (2 * tw * s <= MAX_WAVES && n_tiles * sets >= 2 * tw * cus && lds_bytes_for<TOKS>(a.nb, 2 * tw * s) <= lk_device().lds_bytes) tw *= 2;
    const int forced = lk_tune_env("LK_TUNE_ROWS16_TW");
    if (forced > 0 && forced * s <= MAX_WAVES) tw = forced;
    return tw * s <= 8 ? launch_shape<TOKS, 4>(a, tw, sets, stream) : launch_shape<TOKS, 2>(a, tw, sets, stream);
}

}  // namespace

int lk_rows16_q6k(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k, int stride_y, int ldd,
                  hipStream_t stream) {
    if (size_m < 1 || size_m > 64 || size_n < 1 || size_k < 256) return -1;
    // rows of whole granules, on 16-byte boundaries; a tile's granules within one workgroup
    if (size_k % (256 * GRAN) != 0 || size_k / (256 * GRAN) > MAX_WAVES || (((uintptr_t)w) & 15) != 0) return -1;
    if (lk_tune_env("LK_TUNE_ROWS16_OFF") != 0) return -1;
    const Args a{(const uint8_t*)w, (const uint8_t*)q8_1, output, size_k / 256, size_n, size_m, stride_y, ldd};
    if (size_m > 8 && lk_tune_env("LK_TUNE_ROWS16_MAX8") != 0) return -1;
    if (size_m <= 4) return launch<4>(a, stream);
    const int n_tiles = (size_n + TILE - 1) / TILE;
    // 5..8 rows as two sets of four where that fills the chip sooner than eight at once: so few tiles that a
    // workgroup per tile leaves half the CUs idle (2048 x 6144: 8.9 us against 10.7; 2048 x 14336 12.9 against
    // 16.3), or a matrix small enough for its second reading to come from L2 at no cost (4096 x 4096 9.1 us
    // against 10.3, 8192 x 2048 8.8 against 9.5, 6144 x 4096 11.7 against 12.7; 8192 x 4096, 27.5 MB, 12.2
    // against 11.1 and stays with eight). (Sets: below.)
    const size_t weight_bytes = (size_t)size_n * a.nb * Q6K_BYTES;
    if (size_m <= 8)
        return 2 * n_tiles <= lk_device().cus || weight_bytes <= ((size_t)22 << 20) ? launch<4>(a, stream, 2) : launch<8>(a, stream);
    // 9..32 rows. Sixteen at once when their codes fit LDS and the row tiles are several to the CU; else the
    // rows in sets of eight, a set per workgroup (grid.y), in one launch: rows too long for sixteen in LDS (k =
    // 14336: 229 KB; 4096 x 14336 at 16 rows 25.7 us against 37.4 on the 32-row tiles that would take the
    // call otherwise), up to two tiles to the CU, where twice the workgroups with half the staging each
    // finish sooner (16 rows: 2048 x 6144 11.1 us against 15.9, 4096 x 4096 10.8 against 14.7, 8192 x 2048
    // 10.4 against 13.2, 8192 x 4096 14.5 against 15.7; 11008 x 4096 28.2 against 23.8 and 14336 x 4096 27.2
    // against 25.7 stay with sixteen at once), or 17..32 rows (2048 x 6144 at 32 rows 13.5 us against 22.4 on the 32-row
    // tiles, 4096 x 4096 13.8 against 17.4, 4096 x 14336 42.7 against 47.4, 4096 x 8192 24.8 against 31.1).
    // Every set reads the weights again, from L2 while they fit there, and three or four sets of more than a
    // tile to the CU are too many workgroups: above 16 rows a matrix of more than 64 MB or of more tiles
    // than CUs stays with the 32-row tiles (at 32 rows 151936 x 2048 173 us against 99, 6144 x 4096 25.8
    // against 18.4, 14336 x 4096 39.7 against 32.4).
    if (size_m > 16 && (n_tiles > lk_device().cus || weight_bytes > ((size_t)64 << 20))) return -1;
    // 33..64 rows: only as whole rounds of workgroups that are all resident at two to the CU, one round or
    // exactly two (2048 x 6144 at 64 rows, 128 tiles x 8 sets: 18.7 us against 22.3 on the 32-row tiles; at
    // 40..56 rows, a second round partly filled, 24 against 22.2; 1024 x 2048, 64 tiles, 9.5 against 12.0 at 64
    // rows and 10.3 against 11.8 at 40)
    if (size_m > 32) {
        const int total = n_tiles * ((size_m + 7) / 8), cus = lk_device().cus;
        const bool two_per_cu = lds_bytes_for<8>(a.nb, a.nb / GRAN) <= lk_device().lds_bytes / 2 && a.nb / GRAN <= 8;
        if (!two_per_cu || (total > 2 * cus && total != 4 * cus)) return -1;
    }
    if (size_m <= 16 && n_tiles > 2 * lk_device().cus) {
        const int rc = launch<16>(a, stream);
        if (rc != -1) return rc;
    }
    return launch<8>(a, stream, (size_m + 7) / 8);
}

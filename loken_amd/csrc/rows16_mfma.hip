// Q4_K / Q5_K weights x at most eight Q8_1 activation rows on v_mfma_i32_16x16x64_i8: the decode
// step of a small batch, where the weights should stream at the memory rate and the dot work of the
// mat-vec kernels (which grows with every activation row) no longer fits under that stream.
//
// Serves loken_dense_q4k_imma_m8_plain / _actmul and the Q5_K siblings at size_m <= 8 (declared
// src/inference/moe_cuda/mod.rs:452-466 of the reference, kernels cuda/q4k_mmvq_imma.cu,
// cuda/moe/dense_q4k_imma_m8.cu), and the same launch over up to three matrices that share an
// activation (q + k + v), which the reference issues as separate launches.
//
// Shape of the work. The instruction multiplies a 16 x 64 operand by a 64 x 16 one; lane l holds
// row (column) l % 16 and sixteen K values, group l / 16 of four. Which sixteen is free as long as
// both operands agree, so a lane takes 16 consecutive bytes of its weight row: the four lane groups
// of a row read one 64-byte run of `qs`, two loads cover a super-block's 128 bytes, and every byte
// is loaded once. A run holds the nibbles of two sub-block PAIRS (bytes 0..31: sub-blocks 2 p and
// 2 p + 1 in the low and high nibbles; bytes 32..63: the next pair), so one instruction on the low
// nibbles and one on the high nibbles each see two sub-blocks, s and s + 2, in their K range: lane
// groups 0, 1 hold s, groups 2, 3 hold s + 2. Their dots must stay apart (each sub-block has its own
// scale), so the sixteen slots of the activation operand are (which of the two sub-blocks) x (eight
// activation rows): slot i < 8 holds row i's codes of sub-block s in groups 0, 1 and zeros in groups
// 2, 3; slot i >= 8 holds row i - 8's codes of sub-block s + 2 in groups 2, 3 and zeros below. Half
// the lanes of that operand are zeros; all 16 x 16 results are wanted: lane l, register v is (weight
// row l % 16, activation row 4 ((l / 16) % 2) + v, sub-block s + 2 (l / 32)). The lane's own 16-byte
// header therefore carries the scales its results need: lanes 0..31 unpack sub-blocks 0, 1, 4, 5,
// lanes 32..63 sub-blocks 2, 3, 6, 7. Against the 32 x 32 x 32 form (32 weight rows x 32 slots of
// which 8 are used) this spends half the matrix-unit time per weight and loads nothing twice, and a
// 4096-row matrix is 256 row tiles instead of 128.
//
// Weights never touch LDS. The activation does: a workgroup stages the codes of its (at most) eight
// rows once, in the order the operand wants them, beside a table of d8 and d8 * (sum of codes) per
// (sub-block, row), and a 2 KiB run of zeros that the zero lanes read. A workgroup is eight waves:
// two row tiles at a time (gate and up of the same rows in the dual launch), the four waves of a
// tile splitting its super-blocks and adding their partial tiles through LDS. Rows of 8 or 16
// super-blocks (k = 2048, 4096) take a straight-line path: every load of a wave's share of a tile is
// in flight before its first instruction on the matrix unit, and the next tile's loads go out into
// the same registers when the last has been read, ahead of the reduction.

#include "lk_common.h"
#include "rows16.h"

#include <mutex>
#include <unordered_map>

namespace {

constexpr int KSPLIT = 4;   // waves that share a row tile
constexpr int MAX_TOKS = 16;   // activation rows a launch serves: kernels for up to 8 and up to 16
constexpr int TILE = 16;    // weight rows of a wave's tile
static __host__ __device__ constexpr int zero_bytes(int toks) { return toks * 256; }   // the zero lanes' run

struct WFrag {
    uint4 hdr, q[2], qh;   // qh: Q5_K only
};

template <bool Q5>
struct Blk {
    static constexpr int BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES;
    static constexpr int QS = Q5 ? 48 : 16;
};

static __host__ __device__ constexpr int lds_bytes_for(int nb, int tiles, int toks) {
    // codes [nb * 8][toks][32], zeros, d8 and d8 * S [nb * 8][2][toks] floats, reduce [4 tiles][4][64] floats
    return nb * 8 * toks * 32 + zero_bytes(toks) + nb * 8 * 2 * toks * 4 + KSPLIT * tiles * 4 * 64 * 4;
}

// Element `i` of a three-entry kernel argument without indexing it by a register (which would
// put the whole argument in scratch memory).
template <typename T>
static __device__ __forceinline__ T pick3(const T (&a)[3], int i) { return i == 0 ? a[0] : i == 1 ? a[1] : a[2]; }

// Row tile `vt` of the launch: tiles of the matrices one after another (DUAL: 2 t is the gate
// tile of rows 16 t.., 2 t + 1 the up tile of the same rows).
struct TileRef {
    int mat, row0;
};
template <bool DUAL>
static __device__ __forceinline__ TileRef tile_ref(const LkRows16& p, int vt) {
    if (DUAL) return {vt & 1, (vt >> 1) * TILE};
    int mat = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int tiles = (p.n[i] + TILE - 1) / TILE;
        if (mat == i && i + 1 < p.count && vt >= tiles) { vt -= tiles; mat = i + 1; }
    }
    return {mat, vt * TILE};
}

// TW: row tiles a workgroup takes at a time (four waves each). STEPS: super-blocks a wave owns of
// every tile when that is the same for all waves (rows of 4 STEPS super-blocks), 0 for any row length.
// T16: up to sixteen activation rows. The sixteen slots are then all rows, and every set of weight codes
// runs twice: once against sub-block s (the activation live in lane groups 0, 1) and once against s + 2
// (live in groups 2, 3). Lane l, register v is (weight row l % 16, activation row 4 (l / 16) + v) for
// both, so every lane unpacks all eight scales of its row and its sums are complete across sub-blocks.
template <bool DUAL, bool Q5, int STEPS, int TW, bool T16>
__global__ __launch_bounds__(256 * TW, TW == 4 ? 1 : 2) void q4k_rows16_kernel(LkRows16 p, int n_vt) {
    constexpr int WG = 256 * TW;
    constexpr int TOKS = T16 ? 16 : 8;
    constexpr int ZERO_BYTES = zero_bytes(TOKS);
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* codes = lds;                                               // [nb * 8][8][32]
    uint8_t* zeros = codes + (size_t)p.nb * 8 * TOKS * 32;              // ZERO_BYTES
    float* table = (float*)(zeros + ZERO_BYTES);                        // [nb * 8][2][TOKS]: d8, d8 * S
    float* reduce = table + p.nb * 8 * 2 * TOKS;                        // [4 TW][4][64]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tsel = wave >> 2, kq = wave & 3;   // which tile of the workgroup's TW, which share of its super-blocks
    const int l16 = lane & 15, grp = lane >> 4;
    const int half = grp & 1;   // which sixteen values of a sub-block (operands), which four rows (results)
    const int par = grp >> 1;   // which of an instruction's two sub-blocks
    const size_t row_bytes = (size_t)p.nb * Blk<Q5>::BYTES;
    const int entries = p.nb * 8 * TOKS;
    const int n_pairs = (n_vt + TW - 1) / TW;   // tile groups of the launch
    const int my_blocks = STEPS ? STEPS : (p.nb - kq + KSPLIT - 1) / KSPLIT;

    // the lane's first super-block of tile `vt`
    auto block0 = [&](int vt) {
        const TileRef t = tile_ref<DUAL>(p, vt);
        const int row = min(t.row0 + l16, (DUAL ? p.n[0] : pick3(p.n, t.mat)) - 1);
        return (const uint8_t*)(to_gbytes(pick3(p.w, t.mat)) + row * row_bytes + (size_t)kq * Blk<Q5>::BYTES);
    };
    auto loadw = [&](WFrag& f, const uint8_t* bp) {
        f.hdr = *(const uint4*)bp;
        if (Q5) f.qh = *(const uint4*)(bp + 16 + 16 * half);
        f.q[0] = *(const uint4*)(bp + Blk<Q5>::QS + 16 * grp);
        f.q[1] = *(const uint4*)(bp + Blk<Q5>::QS + 64 + 16 * grp);
    };
    constexpr size_t STEP_BYTES = (size_t)KSPLIT * Blk<Q5>::BYTES;   // between a wave's consecutive super-blocks

    // The activation: entry (sub-block, row) is one Q8_1 block. Its loads go out before the first
    // weight loads and are consumed after them (loads return in issue order: asked for after the
    // weights, the activation, which sits in L2, would wait for HBM).
    constexpr int PER = 2;
    uint32_t head[PER];
    uint4 lo[PER], hi[PER];
    auto issue = [&](int base) {
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = min(base + u * WG, entries - 1);
            const int sub = idx / TOKS, tok = min(idx % TOKS, p.m - 1);
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
                const int sub = idx / TOKS, tok = idx % TOKS;
                const bool real = tok < p.m;
                const float d8 = real ? f16_bits_to_f32(head[u] & 0xFFFFu) : 0.f;
                table[sub * 2 * TOKS + tok] = d8;
                table[sub * 2 * TOKS + TOKS + tok] = d8 * (float)dot16(ones, hi[u], dot16(ones, lo[u], 0));
                const uint32_t keep = real ? 0xFFFFFFFFu : 0u;   // rows the launch does not have: zeros
                *(uint4*)(codes + (size_t)idx * 32) = make_uint4(lo[u].x & keep, lo[u].y & keep, lo[u].z & keep, lo[u].w & keep);
                *(uint4*)(codes + (size_t)idx * 32 + 16) = make_uint4(hi[u].x & keep, hi[u].y & keep, hi[u].z & keep, hi[u].w & keep);
            }
        }
    };

    // The lane's piece of the activation operand. Up to eight rows: slot l16 is (sub-block l16 / 8 of the
    // two, row l16 % 8); the lane's K group belongs to sub-block par; where the two differ the piece is
    // zeros: those lanes read the run of zeros, at a stride of nothing. Up to sixteen rows: slot l16 is row
    // l16, and there are two pieces, one per run of the instruction: live for the lanes of sub-block 0
    // (groups 0, 1) in the first, for those of sub-block 1 in the second.
    const bool live = T16 ? par == 0 : (l16 >> 3) == par;
    const bool live2 = T16 && par == 1;
    const uint8_t* a_lane = live ? codes + (T16 ? l16 : 2 * par * TOKS + (l16 & 7)) * 32 + 16 * half : zeros;
    const uint8_t* a_lane2 = live2 ? codes + (2 * TOKS + l16) * 32 + 16 * half : zeros;
    const int a_step = live ? 8 * TOKS * 32 : 0;   // bytes per super-block
    const int a_step2 = live2 ? 8 * TOKS * 32 : 0;
    // the lane's results: up to eight rows: sub-blocks 2 par + {0, 1, 4, 5}, rows 4 half .. 4 half + 3;
    // up to sixteen: every sub-block, rows 4 grp .. 4 grp + 3
    const float* t_lane = T16 ? table + 4 * grp : table + 2 * par * 2 * TOKS + 4 * half;
    const int sh16 = T16 ? 0 : 16 * par, sh2 = 2 * par;

    float acc[4] = {0.f, 0.f, 0.f, 0.f};

    auto compute = [&](const WFrag& w, int kb) {
        // the row's (scale, min) pairs of sub-blocks 2 par, 2 par + 1, 4 + 2 par, 5 + 2 par, six bits
        // each (get_scale_min_k4 of the format)
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
        // one instruction's four results into the sums: sub-block `sub` of the super-block
        auto fold = [&](const v4i& c, float dsc, float dmm, int sub) {
            const float off = -MAGIC * dsc;
            const float4 t = *(const float4*)(t_blk + sub * 2 * TOKS);
            const float4 s = *(const float4*)(t_blk + sub * 2 * TOKS + TOKS);
            acc[0] = fmaf(fmaf(__int_as_float(c[0]), dsc, off), t.x, fmaf(dmm, s.x, acc[0]));
            acc[1] = fmaf(fmaf(__int_as_float(c[1]), dsc, off), t.y, fmaf(dmm, s.y, acc[1]));
            acc[2] = fmaf(fmaf(__int_as_float(c[2]), dsc, off), t.z, fmaf(dmm, s.z, acc[2]));
            acc[3] = fmaf(fmaf(__int_as_float(c[3]), dsc, off), t.w, fmaf(dmm, s.w, acc[3]));
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
                if constexpr (T16) {
                    // sub-blocks 4 c2 + nib (lane groups 0, 1) and 4 c2 + 2 + nib (groups 2, 3)
                    const v4i a0 = *(const v4i*)(a_blk + (4 * c2 + nib) * TOKS * 32);
                    const v4i a1 = *(const v4i*)(a_blk2 + (4 * c2 + nib) * TOKS * 32);
                    const v4i c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b, magic, 0, 0, 0);
                    const v4i c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b, magic, 0, 0, 0);
                    fold(c0, d * (float)((scw >> (8 * nib)) & 0xFFu), -(dmin * (float)((mnw >> (8 * nib)) & 0xFFu)), 4 * c2 + nib);
                    fold(c1, d * (float)((scw >> (8 * nib + 16)) & 0xFFu), -(dmin * (float)((mnw >> (8 * nib + 16)) & 0xFFu)),
                         4 * c2 + 2 + nib);
                } else {
                    // this lane's sub-block: 4 c2 + 2 par + nib (its scale words are shifted to it)
                    const v4i a = *(const v4i*)(a_blk + (4 * c2 + nib) * TOKS * 32);
                    const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, magic, 0, 0, 0);
                    fold(c, d * (float)((scw >> (8 * nib)) & 0xFFu), -(dmin * (float)((mnw >> (8 * nib)) & 0xFFu)), 4 * c2 + nib);
                }
            }
        }
    };

    // Adds the partial tiles of the workgroup's row tiles (tiles vt0 .. vt0 + TW - 1) and writes them.
    auto finish_pair = [&](int vt0) {
        float* mine = reduce + wave * (4 * 64);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            mine[v * 64 + lane] = acc[v];
            acc[v] = 0.f;
        }
        __syncthreads();
        // Up to eight rows: thread (tile ts, register v, lane l < 32) adds the four shares of the tile's
        // super-blocks and the two sub-blocks of an instruction (lanes l and l + 32). Up to sixteen: thread
        // (ts, v, l < 64) adds the four shares.
        constexpr int LANES = T16 ? 64 : 32, PER_TILE = 4 * LANES;
        const int t = threadIdx.x;
        if (t < (DUAL ? PER_TILE * TW / 2 : PER_TILE * TW)) {
            const int ts = (t / PER_TILE) * (DUAL ? 2 : 1), v = (t / LANES) & 3, l = t % LANES;
            auto total_of = [&](int which) {
                const float* col = reduce + which * (KSPLIT * 256) + v * 64 + l;
                if (T16) return (col[0] + col[256]) + (col[512] + col[768]);
                return ((col[0] + col[32]) + (col[256] + col[288])) + ((col[512] + col[544]) + (col[768] + col[800]));
            };
            float sum = total_of(ts);
            const int vt = vt0 + ts;
            if (DUAL) {
                LkGateAct act;
                act.kind = p.gelu ? LK_GATE_GELU : LK_GATE_SILU;
                sum = lk_gated(act, sum, total_of(ts + 1), 0);
            }
            if (vt < n_vt) {
                const TileRef tr = tile_ref<DUAL>(p, vt);
                const int out = DUAL ? 0 : tr.mat;
                const int tok = (T16 ? 4 * (l >> 4) : 4 * ((l >> 4) & 1)) + v, row = tr.row0 + (l & 15);
                if (tok < p.m && row < pick3(p.n, out)) pick3(p.dst, out)[(size_t)tok * pick3(p.ldd, out) + row] = sum;
            }
        }
        __syncthreads();   // the partial tiles may be overwritten
    };

    auto stage = [&]() {
        place(threadIdx.x);
        for (int r = WG * PER; r < entries; r += WG * PER) {
            issue(r + threadIdx.x);
            place(r + threadIdx.x);
        }
        for (int i = threadIdx.x * 16; i < ZERO_BYTES; i += WG * 16) *(uint4*)(zeros + i) = make_uint4(0, 0, 0, 0);
        __syncthreads();
    };

    const int stride = (int)gridDim.x;
    int pair = (int)blockIdx.x;
    if constexpr (STEPS > 0) {
        WFrag f[STEPS];
        issue(threadIdx.x);
        bool mine = TW * pair + tsel < n_vt;
        if (mine) {
            const uint8_t* bp = block0(TW * pair + tsel);
#pragma unroll
            for (int d = 0; d < STEPS; ++d) loadw(f[d], bp + d * STEP_BYTES);
        }
        stage();
        for (; pair < n_pairs; pair += stride) {
            if (mine) {
#pragma unroll
                for (int d = 0; d < STEPS; ++d) compute(f[d], kq + d * KSPLIT);
            }
            // the next tile's loads go out into the registers just read, and fly under the reduction
            const int next = TW * (pair + stride) + tsel;
            const bool next_mine = next < n_vt;
            if (next_mine) {
                const uint8_t* bp = block0(next);
#pragma unroll
                for (int d = 0; d < STEPS; ++d) loadw(f[d], bp + d * STEP_BYTES);
            }
            finish_pair(TW * pair);
            mine = next_mine;
        }
    } else {
        constexpr int DEPTH = 4;   // steps of weight loads a wave keeps in flight
        WFrag f[DEPTH];
        issue(threadIdx.x);
        bool mine = TW * pair + tsel < n_vt && my_blocks > 0;
        const uint8_t* bp = nullptr;
        if (mine) {
            bp = block0(TW * pair + tsel);
#pragma unroll
            for (int d = 0; d < DEPTH; ++d)
                if (d < my_blocks) loadw(f[d], bp + d * STEP_BYTES);
        }
        stage();
        for (; pair < n_pairs; pair += stride) {
            if (mine) {
                for (int j0 = 0; j0 < my_blocks; j0 += DEPTH) {
#pragma unroll
                    for (int d = 0; d < DEPTH; ++d) {
                        const int j = j0 + d;
                        if (j < my_blocks) {
                            compute(f[d], kq + j * KSPLIT);
                            if (j + DEPTH < my_blocks) loadw(f[d], bp + (size_t)(j + DEPTH) * STEP_BYTES);
                        }
                    }
                }
            }
            const int next = TW * (pair + stride) + tsel;
            mine = next < n_vt && my_blocks > 0;
            if (mine) {   // the next tile's first loads fly under the reduction
                bp = block0(next);
#pragma unroll
                for (int d = 0; d < DEPTH; ++d)
                    if (d < my_blocks) loadw(f[d], bp + d * STEP_BYTES);
            }
            finish_pair(TW * pair);
        }
    }
}

// Workgroups per CU the kernel can keep resident with `lds_bytes` of LDS each; 0: does not fit.
template <bool DUAL, bool Q5, int STEPS, int TW, bool T16>
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
               hipFuncSetAttribute((const void*)q4k_rows16_kernel<DUAL, Q5, STEPS, TW, T16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        r = 0;
    } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q4k_rows16_kernel<DUAL, Q5, STEPS, TW, T16>, 256 * TW,
                                                            (size_t)lds_bytes) != hipSuccess || r < 1) {
        (void)hipGetLastError();
        r = 1;
    }
    by_lds.emplace(lds_bytes, r);
    return r;
}

template <bool DUAL, bool Q5, int STEPS, int TW, bool T16>
int launch_shape(const LkRows16& a, int n_vt, hipStream_t stream) {
    const int lds_bytes = lds_bytes_for(a.nb, TW, T16 ? 16 : 8);
    const int per_cu = resident_cap<DUAL, Q5, STEPS, TW, T16>(lds_bytes);
    if (per_cu == 0) return -1;
    const int units = (n_vt + TW - 1) / TW;   // tile groups
    // Every workgroup stages the activation, so a workgroup should walk a few tile groups; all of
    // them resident at once, and as equal a share each as the count allows.
    int cap = lk_device().cus * per_cu;
    const int forced = lk_tune_env("LK_TUNE_ROWS16_WGS");
    if (forced > 0) cap = forced;
    const int passes = (units + cap - 1) / cap;
    const int wgs = (units + passes - 1) / passes;
    hipLaunchKernelGGL((q4k_rows16_kernel<DUAL, Q5, STEPS, TW, T16>), dim3(wgs), dim3(256 * TW), lds_bytes, stream, a, n_vt);
    return lk_launch_status();
}

template <bool DUAL, bool Q5, int STEPS, bool T16>
int launch_steps(const LkRows16& a, hipStream_t stream) {
    int n_vt = 0;
    if (DUAL) {
        n_vt = 2 * ((a.n[0] + TILE - 1) / TILE);
    } else {
        for (int i = 0; i < a.count; ++i) n_vt += (a.n[i] + TILE - 1) / TILE;
    }
    if (n_vt == 0) return LK_OK;
    // Four tiles per workgroup (sixteen waves, one workgroup per CU) once that still gives every CU
    // a workgroup: half the copies of the activation staged.
    int tw = n_vt >= 4 * lk_device().cus ? 4 : 2;
    const int forced = lk_tune_env("LK_TUNE_ROWS16_TW");
    if (forced == 2 || forced == 4) tw = forced;
    if (tw == 4) {
        const int rc = launch_shape<DUAL, Q5, STEPS, 4, T16>(a, n_vt, stream);
        if (rc >= 0) return rc;
    }
    return launch_shape<DUAL, Q5, STEPS, 2, T16>(a, n_vt, stream);
}

template <bool DUAL, bool Q5, bool T16>
int launch_rows(const LkRows16& a, hipStream_t stream) {
    const int forced = lk_tune_env("LK_TUNE_ROWS16_GENERIC");
    if (a.nb == 16 && !forced) return launch_steps<DUAL, Q5, 4, T16>(a, stream);
    if (a.nb == 8 && !forced) return launch_steps<DUAL, Q5, 2, T16>(a, stream);
    return launch_steps<DUAL, Q5, 0, T16>(a, stream);
}

template <bool DUAL, bool Q5>
int launch(const LkRows16& a, hipStream_t stream) {
    return a.m <= 8 ? launch_rows<DUAL, Q5, false>(a, stream) : launch_rows<DUAL, Q5, true>(a, stream);
}

}  // namespace

bool lk_rows16_serves(int size_m, int nb) {
    return size_m >= 1 && size_m <= MAX_TOKS && nb >= 1 && lds_bytes_for(nb, 2, size_m <= 8 ? 8 : 16) <= lk_device().lds_bytes;
}

int lk_rows16_launch(const LkRows16& a, bool dual, bool q5, hipStream_t stream) {
    if (a.m < 1 || a.m > MAX_TOKS || a.nb < 1 || a.count < 1 || a.count > 3 || (dual && a.count != 2)) return LK_ERR_ARG;
    if (dual && a.n[0] != a.n[1]) return LK_ERR_ARG;
    int rc;
    if (dual) rc = q5 ? launch<true, true>(a, stream) : launch<true, false>(a, stream);
    else rc = q5 ? launch<false, true>(a, stream) : launch<false, false>(a, stream);
    return rc < 0 ? LK_ERR_ARG : rc;
}

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
#include "rows16_core.h"

#include <mutex>
#include <unordered_map>

namespace {

constexpr int KSPLIT = 4;   // waves that share a row tile
constexpr int MAX_TOKS = 16;   // activation rows a launch serves: kernels for up to 8 and up to 16
using rows16::Blk;
using rows16::TILE;
using rows16::WFrag;

static __host__ __device__ constexpr int lds_bytes_for(int nb, int tiles, int toks, bool q81 = false) {
    // the staged activation, reduce [4 tiles][4][64] floats, with Q8_1 output the 32 results of every row
    return rows16::staged_bytes(nb, toks) + KSPLIT * tiles * 4 * 64 * 4 + (q81 ? toks * 32 * 4 : 0);
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
// Q81 (gate + up, four tiles per workgroup: the 32 consecutive output rows of a Q8_1 block): the result
// leaves as the Q8_1 rows the next linear reads, with the quantizer's steps.
template <bool DUAL, bool Q5, int STEPS, int TW, bool T16, bool Q81 = false>
__global__ __launch_bounds__(256 * TW, TW == 4 ? 1 : 2) void q4k_rows16_kernel(LkRows16 p, int n_vt) {
    static_assert(!Q81 || (DUAL && TW == 4), "Q8_1 output: the dual launch with four tiles per workgroup");
    constexpr int WG = 256 * TW;
    extern __shared__ __align__(16) uint8_t lds[];
    rows16::Core<Q5, T16> core;
    float* reduce = (float*)core.init(lds, p.nb);                       // [4 TW][4][64]
    float* meet = reduce + KSPLIT * TW * 4 * 64;                        // Q81: [TOKS][32]
    const rows16::RowsIn rows{p.y, p.stride_y, nullptr, 0};

    const int lane = core.lane, l16 = core.l16;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tsel = wave >> 2, kq = wave & 3;   // which tile of the workgroup's TW, which share of its super-blocks
    const size_t row_bytes = (size_t)p.nb * Blk<Q5>::BYTES;
    const int entries = p.nb * 8 * core.TOKS;
    const int n_pairs = (n_vt + TW - 1) / TW;   // tile groups of the launch
    const int my_blocks = STEPS ? STEPS : (p.nb - kq + KSPLIT - 1) / KSPLIT;

    // the lane's first super-block of tile `vt`
    auto block0 = [&](int vt) {
        const TileRef t = tile_ref<DUAL>(p, vt);
        const int row = min(t.row0 + l16, (DUAL ? p.n[0] : pick3(p.n, t.mat)) - 1);
        return (const uint8_t*)(to_gbytes(pick3(p.w, t.mat)) + row * row_bytes + (size_t)kq * Blk<Q5>::BYTES);
    };
    auto loadw = [&](WFrag& f, const uint8_t* bp) { core.loadw(f, bp); };
    constexpr size_t STEP_BYTES = (size_t)KSPLIT * Blk<Q5>::BYTES;   // between a wave's consecutive super-blocks
    // The activation's first loads go out before the first weight loads and are consumed after them
    // (loads return in issue order: asked for after the weights, the activation, which sits in L2, would
    // wait for HBM).
    auto issue = [&](int base) { core.issue(rows, p.m, entries, entries, base, WG); };

    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const WFrag& w, int kb) { core.compute(w, kb, acc); };

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
            if (Q81) {
                // (n is a multiple of 32 here: every tile of the launch is whole)
                const int tok = (T16 ? 4 * (l >> 4) : 4 * ((l >> 4) & 1)) + v;
                meet[tok * 32 + 8 * ts + (l & 15)] = sum;
            } else if (vt < n_vt) {
                const TileRef tr = tile_ref<DUAL>(p, vt);
                const int out = DUAL ? 0 : tr.mat;
                const int tok = (T16 ? 4 * (l >> 4) : 4 * ((l >> 4) & 1)) + v, row = tr.row0 + (l & 15);
                if (tok < p.m && row < pick3(p.n, out)) pick3(p.dst, out)[(size_t)tok * pick3(p.ldd, out) + row] = sum;
            }
        }
        __syncthreads();   // the partial tiles may be overwritten
        if (Q81) {
            // eight lanes per activation row write its block; the next group's results reach `meet` only
            // after the barrier these lanes pass next
            if (t < 8 * p.m && vt0 < n_vt) {
                const int tok = t >> 3, l8 = t & 7;
                const float4 v4 = *(const float4*)(meet + tok * 32 + 4 * l8);
                lk_store_q8_1_block(v4, l8, (uint32_t*)(p.q81_dst + ((size_t)tok * p.q81_stride + vt0 / 4) * Q81_BYTES));
            }
        }
    };

    auto stage = [&]() {
        core.finish_staging(rows, p.m, p.nb, WG);
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
            // the next tile's loads go out into each set of registers as it has been read: they fly under
            // the arithmetic of the sets still to come, and under the reduction
            const int next = TW * (pair + stride) + tsel;
            const bool next_mine = next < n_vt;
            const uint8_t* bp = next_mine ? block0(next) : nullptr;
#pragma unroll
            for (int d = 0; d < STEPS; ++d) {
                if (mine) compute(f[d], kq + d * KSPLIT);
                if (next_mine) {
                    __builtin_amdgcn_sched_barrier(0);
                    loadw(f[d], bp + d * STEP_BYTES);
                    __builtin_amdgcn_sched_barrier(0);
                }
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
template <bool DUAL, bool Q5, int STEPS, int TW, bool T16, bool Q81 = false>
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
               hipFuncSetAttribute((const void*)q4k_rows16_kernel<DUAL, Q5, STEPS, TW, T16, Q81>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        r = 0;
    } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q4k_rows16_kernel<DUAL, Q5, STEPS, TW, T16, Q81>, 256 * TW,
                                                            (size_t)lds_bytes) != hipSuccess || r < 1) {
        (void)hipGetLastError();
        r = 1;
    }
    by_lds.emplace(lds_bytes, r);
    return r;
}

template <bool DUAL, bool Q5, int STEPS, int TW, bool T16, bool Q81 = false>
int launch_shape(const LkRows16& a, int n_vt, hipStream_t stream) {
    const int lds_bytes = lds_bytes_for(a.nb, TW, T16 ? 16 : 8, Q81);
    const int per_cu = resident_cap<DUAL, Q5, STEPS, TW, T16, Q81>(lds_bytes);
    if (per_cu == 0) return -1;
    const int units = (n_vt + TW - 1) / TW;   // tile groups
    // Every workgroup stages the activation, so a workgroup should walk a few tile groups; all of
    // them resident at once, and as equal a share each as the count allows.
    int cap = lk_device().cus * per_cu;
    const int forced = lk_tune_env("LK_TUNE_ROWS16_WGS");
    if (forced > 0) cap = forced;
    const int passes = (units + cap - 1) / cap;
    const int wgs = (units + passes - 1) / passes;
    hipLaunchKernelGGL((q4k_rows16_kernel<DUAL, Q5, STEPS, TW, T16, Q81>), dim3(wgs), dim3(256 * TW), lds_bytes, stream, a, n_vt);
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
    if (a.q81_dst) {   // Q8_1 output: the straight-line dual launch at four tiles per workgroup, or nothing
        if constexpr (DUAL && STEPS != 0) return launch_shape<DUAL, Q5, STEPS, 4, T16, true>(a, n_vt, stream);
        return -1;
    }
    // Four tiles per workgroup (sixteen waves, one workgroup per CU) once that still gives every CU
    // a workgroup: half the copies of the activation staged.
    int tw = n_vt >= 4 * lk_device().cus ? 4 : 2;
    const int forced = lk_tune_env("LK_TUNE_ROWS16_TW");
    if (forced == 2 || forced == 4) tw = forced;
    if constexpr (STEPS != 0) {   // (the any-row-length path at sixteen waves would not fit the register file)
        if (tw == 4) {
            const int rc = launch_shape<DUAL, Q5, STEPS, 4, T16>(a, n_vt, stream);
            if (rc >= 0) return rc;
        }
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
    if (a.q81_dst && (!dual || a.n[0] % 32 != 0 || (a.nb != 8 && a.nb != 16) || a.q81_stride < a.n[0] / 32)) return LK_ERR_ARG;
    int rc;
    if (dual) rc = q5 ? launch<true, true>(a, stream) : launch<true, false>(a, stream);
    else rc = q5 ? launch<false, true>(a, stream) : launch<false, false>(a, stream);
    return rc < 0 ? LK_ERR_ARG : rc;
}

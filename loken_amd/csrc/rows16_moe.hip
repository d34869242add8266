// Expert-batched Q4_K rows in 16-row tiles on v_mfma_i32_16x16x64_i8: the kernel of rows16_mfma.hip per
// expert over a sorted routing, for routings that give an expert a handful of rows (what
// lk_moe_q4k_rows_grouped launches for rows of at most eight super-blocks and at most sixteen expected
// rows per expert). The reference reaches these loads through its tiled expert kernel
// (launch_mmq_moe_gguf_q4_k, src/tensor/quantized/mmq.rs:274-286) or one mat-vec per routed pair; it has
// no launcher of this shape.
//
// Expert matrices are short and wide in count (Qwen3-30B-A3B: 128 experts of 768 x 2048 and 2048 x 768), so
// unlike the dense launch a WAVE owns a row tile outright: all of its row's super-blocks in turn, no
// split of k between waves, no partial tiles through LDS, nothing between waves but the staged
// activation. Grid y is the expert; its sorted rows go through in passes of 8, 16 or 48, each pass
// staging the rows' Q8_1 codes in LDS (gathered through the routing) in chunks of 16 and walking the
// workgroup's share of the expert's tiles: a super-block's codes and scales are unpacked once and run
// against every chunk (an expert with more rows than a pass holds takes another pass, its weights then
// from the caches). With a second matrix
// the wave takes the gate tile, keeps its sums in registers, takes the up tile of the same rows and
// stores act(gate) * up. Loads run D super-blocks ahead across tiles, with no branch around them.

#include "lk_common.h"
#include "rows16.h"
#include "rows16_core.h"

#include <mutex>
#include <type_traits>
#include <utility>
#include <unordered_map>

namespace {

using rows16::TILE;
using rows16::WFrag;
constexpr int BYTES = Q4K_BYTES;

// NB: super-blocks per row (a template constant: the step within a tile picks its load registers).
// D: super-blocks of loads in flight, a divisor of NB.
template <int NB>
struct Depth {
    static constexpr int D = NB % 4 == 0 ? 4 : NB % 3 == 0 ? 3 : NB % 2 == 0 ? 2 : 1;
};

template <class F, int... I>
static __device__ __forceinline__ void each_step(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}

// CHUNKS: groups of 16 rows a pass holds (1 with T16 off: up to 8 rows). WAVES: per workgroup (8 when the
// staged rows leave room for one workgroup per CU only).
template <bool DUAL, bool T16, int NB, int CHUNKS, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void q4k_rows16_moe_kernel(LkRows16 p, LkRows16Experts m) {
    constexpr int WG = 64 * WAVES;
    constexpr int D = Depth<NB>::D, TOKS = T16 ? 16 : 8, MATS = DUAL ? 2 : 1, PASS = TOKS * CHUNKS;
    extern __shared__ __align__(16) uint8_t lds[];
    const int e = blockIdx.y;
    const int begin = m.bounds[e], end = m.bounds[e + 1];
    if (end <= begin) return;
    rows16::Core<false, T16> core;
    core.init(lds, NB, CHUNKS);
    const int lane = core.lane, l16 = core.l16;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = p.n[0], n_tiles = (n + TILE - 1) / TILE;
    const int units = (int)gridDim.x * WAVES, unit = (int)blockIdx.x * WAVES + wave;
    const int my_tiles = unit < n_tiles ? (n_tiles - unit + units - 1) / units : 0;
    const size_t row_bytes = (size_t)NB * BYTES;
    const uint8_t* w_first = p.w[0] + (int64_t)e * m.expert_bytes;
    const uint8_t* w_second = DUAL ? p.w[1] + (int64_t)e * m.expert_bytes : nullptr;
    constexpr int per_chunk = NB * 8 * TOKS;

    auto block0 = [&](int which) {   // the lane's first super-block of the wave's `which`-th (tile, matrix)
        const int tile = unit + (which / MATS) * units;
        const int row = min(tile * TILE + l16, n - 1);
        return (DUAL && (which & 1) ? w_second : w_first) + row * row_bytes;
    };
    const int total = my_tiles * MATS;   // (tile, matrix) pairs of this wave in a pass

    for (int first = begin; first < end; first += PASS) {
        const int m_count = min(PASS, end - first);
        const int live = (m_count + TOKS - 1) / TOKS;   // chunks this pass has rows for
        const rows16::RowsIn rows{p.y, p.stride_y, m.src, first};
        core.issue(rows, m_count, live * per_chunk, per_chunk, threadIdx.x, WG);
        WFrag ring[D];
        int l_which = 0;
        const uint8_t* l_base = total > 0 ? block0(0) : nullptr;
        if (total > 0) {
#pragma unroll
            for (int i = 0; i < D; ++i) core.loadw(ring[i], l_base + i * BYTES);
        }
        core.finish_staging(rows, m_count, NB, WG, live);
        __syncthreads();

        // the pass's tiles against C chunks of rows
        auto run = [&](auto c_c) {
            constexpr int C = decltype(c_c)::value;
            float acc[C][4], gate_keep[C][4];
#pragma unroll
            for (int ch = 0; ch < C; ++ch)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[ch][v] = 0.f;
            for (int which = 0; which < total; ++which) {
                auto step = [&](auto i_c) {
                    constexpr int I = decltype(i_c)::value;
                    core.template compute_chunks<C>(ring[I % D], I, acc);
                    // one super-block at a time: left free, the compiler interleaves the arithmetic of all of
                    // a tile's super-blocks and runs out of registers
#pragma unroll
                    for (int ch = 0; ch < C; ++ch)
#pragma unroll
                        for (int v = 0; v < 4; ++v) asm volatile("" : "+v"(acc[ch][v]));
                    __builtin_amdgcn_sched_barrier(0);
                    // the super-block D ahead goes out into the registers just read: this tile's, or the next
                    // (tile, matrix)'s (past the last: the last one again, a load nobody waits for)
                    if constexpr (I + D == NB) {
                        l_which = min(which + 1, total - 1);
                        l_base = block0(l_which);
                    }
                    core.loadw(ring[I % D], l_base + ((I + D) % NB) * BYTES);
                };
                each_step(step, std::make_integer_sequence<int, NB>{});

                const int tile = unit + (which / MATS) * units, row = tile * TILE + l16;
#pragma unroll
                for (int ch = 0; ch < C; ++ch) {
                    // the tile's sums: up to eight rows the two sub-blocks of an instruction sit in lanes l, l + 32
                    float sum[4];
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        sum[v] = T16 ? acc[ch][v] : swap_add32(acc[ch][v]);
                        acc[ch][v] = 0.f;
                    }
                    if (DUAL && (which & 1) == 0) {
#pragma unroll
                        for (int v = 0; v < 4; ++v) gate_keep[ch][v] = sum[v];
                        continue;
                    }
                    if (row < n && (T16 || lane < 32)) {
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const int tok = ch * TOKS + (T16 ? 4 * core.grp : 4 * core.half) + v;
                            if (tok < m_count) {
                                float out = sum[v];
                                if (DUAL) {
                                    LkGateAct act;
                                    act.kind = p.gelu ? LK_GATE_GELU : LK_GATE_SILU;
                                    out = lk_gated(act, gate_keep[ch][v], out, 0);
                                }
                                const int r = m.dst_map ? m.dst_map[first + tok] : first + tok;
                                p.dst[0][(size_t)r * p.ldd[0] + row] = out;
                            }
                        }
                    }
                }
            }
        };
        if (CHUNKS >= 3 && live == 3) run(std::integral_constant<int, CHUNKS >= 3 ? 3 : 1>{});
        else if (CHUNKS >= 2 && live == 2) run(std::integral_constant<int, CHUNKS >= 2 ? 2 : 1>{});
        else run(std::integral_constant<int, 1>{});
        __syncthreads();   // every wave is done with the staged rows: the next pass may replace them
    }
}

template <bool DUAL, bool T16, int NB, int CHUNKS, int WAVES>
int launch_shape(const LkRows16& a, const LkRows16Experts& m, int n_experts, hipStream_t stream) {
    static std::mutex mu;
    static int per_cu = -1;
    const int lds_bytes = rows16::staged_bytes(NB, T16 ? 16 : 8, CHUNKS);
    if (lds_bytes > lk_device().lds_bytes) return -1;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (per_cu < 0) {
            int r = 0;
            if (lds_bytes > 48 * 1024 &&
                hipFuncSetAttribute((const void*)q4k_rows16_moe_kernel<DUAL, T16, NB, CHUNKS, WAVES>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
                (void)hipGetLastError();
                r = 0;
            } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q4k_rows16_moe_kernel<DUAL, T16, NB, CHUNKS, WAVES>,
                                                                    64 * WAVES, (size_t)lds_bytes) != hipSuccess || r < 1) {
                (void)hipGetLastError();
                r = 1;
            }
            per_cu = r;
        }
        if (per_cu == 0) return -1;
    }
    // workgroups per expert: enough for a couple of rounds of the chip over all experts, at least one, and
    // no more than a wave per tile
    const int n_tiles = (a.n[0] + TILE - 1) / TILE, most = (n_tiles + WAVES - 1) / WAVES;
    int per_expert = (2 * lk_device().cus * per_cu + n_experts - 1) / n_experts;
    const int forced = lk_tune_env("LK_TUNE_ROWS16_MOE_WGS");
    if (forced > 0) per_expert = forced;
    if (per_expert < 1) per_expert = 1;
    if (per_expert > most) per_expert = most;
    hipLaunchKernelGGL((q4k_rows16_moe_kernel<DUAL, T16, NB, CHUNKS, WAVES>), dim3(per_expert, n_experts), dim3(64 * WAVES), lds_bytes,
                       stream, a, m);
    return lk_launch_status();
}

// The pass a routing of `rows_hint` expected rows per expert takes: up to 8 rows, one chunk of 16, or three
// (measured at 128 experts of 768 x 2048 and 2048 x 768: three chunks win from about 24 expected rows on;
// two never did).
template <bool DUAL, int NB>
int launch_nb(const LkRows16& a, const LkRows16Experts& m, int n_experts, int rows_hint, hipStream_t stream) {
    const int forced = lk_tune_env("LK_TUNE_ROWS16_MOE_CHUNKS");
    if (rows_hint <= 8 && forced <= 0) return launch_shape<DUAL, false, NB, 1, 4>(a, m, n_experts, stream);
    if (forced > 0 ? forced >= 3 : rows_hint > 24) {
        const int rc = launch_shape<DUAL, true, NB, 3, 8>(a, m, n_experts, stream);
        if (rc >= 0) return rc;
    }
    return launch_shape<DUAL, true, NB, 1, 4>(a, m, n_experts, stream);
}

template <bool DUAL>
int launch(const LkRows16& a, const LkRows16Experts& m, int n_experts, int rows_hint, hipStream_t stream) {
    switch (a.nb) {
        case 2: return launch_nb<DUAL, 2>(a, m, n_experts, rows_hint, stream);
        case 3: return launch_nb<DUAL, 3>(a, m, n_experts, rows_hint, stream);
        case 4: return launch_nb<DUAL, 4>(a, m, n_experts, rows_hint, stream);
        case 8: return launch_nb<DUAL, 8>(a, m, n_experts, rows_hint, stream);
        default: return -1;
    }
}

}  // namespace

int lk_rows16_launch_experts(const LkRows16& a, const LkRows16Experts& m, int n_experts, bool dual, int rows_hint,
                             hipStream_t stream) {
    if (a.nb < 1 || n_experts < 1 || n_experts > 65535) return -1;
    if (lk_tune_env("LK_TUNE_ROWS16_OFF") != 0) return -1;
    return dual ? launch<true>(a, m, n_experts, rows_hint, stream) : launch<false>(a, m, n_experts, rows_hint, stream);
}

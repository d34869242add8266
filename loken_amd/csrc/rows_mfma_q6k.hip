// Q6_K weights x a handful of Q8_1 activation rows on the int8 matrix unit: the Q6_K member of the
// mid-batch family in rows_mfma.hip (same shape of work: a wave owns 32 weight rows and up to 32
// activation rows, lanes stand for weight rows, accumulator registers for activation rows, the four
// waves of a workgroup split a row's super-blocks and add their tiles through LDS).
//
// The reference has no matrix-unit kernel for this format at these row counts; its Q6_K rows go
// through vec_dot_q6_K_q8_1 (cuda/moe/gguf.cuh:782-816, 1089-1108) one activation row at a time. The
// sums formed here are the same: per 16-value group, d * scale[g] * d8 * sum (code - 32) * a.
//
// What differs from Q4_K:
//   - A group is 16 values with its own int8 scale, and v_mfma_i32_32x32x32_i8 sums 32. A lane half
//     (lanes 0-31 / 32-63) supplies 16 of the 32, so each 32-value quarter runs twice, once with the
//     other half's weight codes zeroed: two tiles of 16-value dots, one per group.
//   - The codes go in signed (code - 32 fits int8), so no offset term remains: per byte,
//     ((nibble | two high bits << 4) + 0x60) ^ 0x80 = code - 32 modulo 256, without carries between
//     bytes (code + 0x60 <= 0x9F).
//   - Lane (row, half lh) reads 16 bytes of each of the four ql half-rows at 16 lh, 16 bytes of both
//     qh half-rows at 16 lh, the 16 scales and d: every byte of ql and qh once per wave.

#include "lk_common.h"
#include "rows16.h"

#include <cstdlib>
#include <mutex>
#include <type_traits>
#include <unordered_map>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((aligned(4))) u32x4_a4;

// Waves per workgroup: four, or eight for a matrix of so few 32-row tiles that every workgroup has a
// CU to itself (the waves then split a row's super-blocks eight ways instead of four).
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
};

struct WFrag {
    uint4 ql[4];   // [2 half + c]: bytes 64 half + 32 c + 16 lh of ql
    uint4 qh[2];   // [half]: bytes 32 half + 16 lh of qh
    uint4 sc;      // the 16 group scales
    uint32_t d;    // f16 bits
};

static __device__ __forceinline__ void load_weights(WFrag& f, const uint8_t* bp, int lh) {
#pragma unroll
    for (int c = 0; c < 4; ++c) f.ql[c] = *(const uint4_a2*)(bp + 32 * c + 16 * lh);
#pragma unroll
    for (int half = 0; half < 2; ++half) f.qh[half] = *(const uint4_a2*)(bp + 128 + 32 * half + 16 * lh);
    f.sc = *(const uint4_a2*)(bp + 192);
    f.d = *(const uint16_t*)(bp + 208);
}

// The lane's 16 signed codes of quarter (half, qt): values 128 half + 32 qt + 16 lh + 0..15.
template <int QT>
static __device__ __forceinline__ void quarter_codes(const uint4& ql, const uint4& qh, uint32_t z[4]) {
    const uint32_t u[4] = {ql.x, ql.y, ql.z, ql.w}, h[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t nib = (QT & 2) ? (u[e] >> 4) & 0x0F0F0F0Fu : u[e] & 0x0F0F0F0Fu;
        // the quarter's two high bits sit at 2 QT of the qh byte; they belong at bits 4 and 5
        const uint32_t up = QT == 0 ? h[e] << 4 : QT == 1 ? h[e] << 2 : QT == 2 ? h[e] : h[e] >> 2;
        const uint32_t code = nib | (up & 0x30303030u);
        z[e] = (code + 0x60606060u) ^ 0x80808080u;
    }
}

// The fix-up of one quarter: both groups' tiles into the live accumulator registers.
template <int G>
static __device__ __forceinline__ void fold_quarter(const v16i& c0, const v16i& c1, float dsc0, float dsc1,
                                                    const float* d8_row, int lh, float acc[4 * G]) {
    // The int32 accumulators started at the bit pattern of 1.5 * 2^23: an integer of magnitude below
    // 2^22 added to that pattern is the float 1.5 * 2^23 + integer, so the dots leave the matrix unit
    // as floats. The offset comes off in the first fused multiply-add, exactly: d * scale is an f16
    // times an int8 (18 significant bits), MAGIC * d * scale has 20, so neither product rounds and the
    // fma rounds dot * d * scale once.
    constexpr float MAGIC = 12582912.0f;
    const float off0 = -MAGIC * dsc0, off1 = -MAGIC * dsc1;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const float4 t = *(const float4*)(d8_row + 8 * g + 4 * lh);
        const float d8[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int v = 4 * g + e;
            const float both = fmaf(__int_as_float(c0[v]), dsc0, off0) + fmaf(__int_as_float(c1[v]), dsc1, off1);
            acc[v] = fmaf(both, d8[e], acc[v]);
            // the sum is wanted here, not where it is next read: left free, the compiler sinks every
            // quarter's fix-up to the end of the block and keeps all sixteen result tiles alive
            asm volatile("" : "+v"(acc[v]));
        }
    }
}

// One super-block of the wave's 32 rows against the activation codes `a_of(quarter)` supplies.
template <int G, class AOf>
static __device__ __forceinline__ void block_step(const WFrag& w, bool live, int sub0, const float* d8_table, int lh,
                                                  uint32_t keep0, uint32_t keep1, AOf&& a_of, float acc[4 * G]) {
    constexpr int TW = 8 * G;
    constexpr int MAGIC_BITS = 0x4B400000;
    const float d = live ? f16_bits_to_f32(w.d) : 0.f;
    const uint32_t scd[4] = {w.sc.x, w.sc.y, w.sc.z, w.sc.w};
    auto quarter = [&](auto half_c, auto qt_c) {
        constexpr int HALF = decltype(half_c)::value, QT = decltype(qt_c)::value;
        uint32_t z[4];
        quarter_codes<QT>(w.ql[2 * HALF + (QT & 1)], w.qh[HALF], z);
        const v4i b0 = {(int)(z[0] & keep0), (int)(z[1] & keep0), (int)(z[2] & keep0), (int)(z[3] & keep0)};
        const v4i b1 = {(int)(z[0] & keep1), (int)(z[1] & keep1), (int)(z[2] & keep1), (int)(z[3] & keep1)};
        const v4i a = a_of(4 * HALF + QT);
        v16i c0, c1;
#pragma unroll
        for (int v = 0; v < 16; ++v) c0[v] = c1[v] = MAGIC_BITS;
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b0, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b1, c1, 0, 0, 0);
        // scales 8 HALF + 2 QT (the first 16 values of the quarter) and + 1 (the second 16)
        const uint32_t word = scd[2 * HALF + (QT >> 1)];
        const float dsc0 = d * (float)(int)__builtin_amdgcn_sbfe(word, 16 * (QT & 1), 8);
        const float dsc1 = d * (float)(int)__builtin_amdgcn_sbfe(word, 16 * (QT & 1) + 8, 8);
        fold_quarter<G>(c0, c1, dsc0, dsc1, d8_table + (sub0 + 4 * HALF + QT) * TW, lh, acc);
        // one quarter's two tiles at a time: left free, the scheduler starts every matrix
        // instruction of the block first and holds 16 x 16 result registers
        __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    quarter(I0{}, I0{}); quarter(I0{}, I1{}); quarter(I0{}, I2{}); quarter(I0{}, I3{});
    quarter(I1{}, I0{}); quarter(I1{}, I1{}); quarter(I1{}, I2{}); quarter(I1{}, I3{});
}

template <int G, bool STAGED, int WAVES>
static __host__ __device__ constexpr int lds_bytes_for(int nb) {
    // [codes [nb * 8][8 G][32] when staged,] d8 [nb * 8][8 G] floats, reduce [WAVES][4 G][64] floats
    return (STAGED ? nb * 8 * 8 * G * 32 : 0) + nb * 8 * 8 * G * 4 + WAVES * 4 * G * 64 * 4;
}

// STAGED: at most 8 G activation rows whose codes fit in LDS beside the scales; the workgroup stages
// them once and a wave keeps DEPTH steps of weight loads in flight. Otherwise the lane reads its
// activation row's codes from memory with every step's weights (two steps in flight), 32 rows per
// pass, grid y over the passes.
template <int G, bool STAGED, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WAVES == 4 ? 2 : 1) void q6k_rows_kernel(Args p) {
    constexpr int TW = 8 * G, NV = 4 * G, WG = 64 * WAVES;
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* codes = lds;                                                              // STAGED: [nb * 8][TW][32]
    float* d8_table = (float*)(lds + (STAGED ? (size_t)p.nb * 8 * TW * 32 : 0));       // [nb * 8][TW]
    float* reduce = d8_table + p.nb * 8 * TW;                                          // [WAVES][NV][64]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const uint32_t keep0 = lh ? 0u : 0xFFFFFFFFu, keep1 = ~keep0;
    const int m0 = STAGED ? 0 : blockIdx.y * TOK;
    const int m_count = min(STAGED ? TW : TOK, p.m - m0);
    const int n_tiles = (p.n + 31) >> 5;
    const size_t row_bytes = (size_t)p.nb * Q6K_BYTES;
    const uint8_t* y0 = p.y + (size_t)m0 * p.stride_y * Q81_BYTES;
    const int entries = p.nb * 8 * TW;

    const int my_blocks = (p.nb - wave + WAVES - 1) / WAVES;   // super-blocks wave, wave + 4, ...: may be zero
    const int my_tiles = (int)blockIdx.x < n_tiles ? (n_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    const int total = my_tiles * my_blocks;
    auto weights_at = [&](int j) {
        const int tile = blockIdx.x + (j / my_blocks) * gridDim.x, kb = wave + (j % my_blocks) * WAVES;
        const int row = min(tile * 32 + l32, p.n - 1);
        return (const uint8_t*)(to_gbytes(p.w) + row * row_bytes + (size_t)kb * Q6K_BYTES);
    };

    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.f;

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
            if (wave >= 4) break;   // the first four waves write the NV registers' rows, G each
            const int v = wave * G + r;
            float sum = (reduce[v * 64 + lane] + reduce[(NV + v) * 64 + lane]) +
                        (reduce[(2 * NV + v) * 64 + lane] + reduce[(3 * NV + v) * 64 + lane]);
            if (WAVES == 8)
                sum += (reduce[(4 * NV + v) * 64 + lane] + reduce[(5 * NV + v) * 64 + lane]) +
                       (reduce[(6 * NV + v) * 64 + lane] + reduce[(7 * NV + v) * 64 + lane]);
            const int tok = (v >> 2) * 8 + lh * 4 + (v & 3), row = ((int)blockIdx.x + ordinal * (int)gridDim.x) * 32 + l32;
            if (tok < m_count && row < p.n) p.dst[(size_t)(m0 + tok) * p.ldd + row] = sum;
        }
        __syncthreads();   // the partial tiles may be overwritten
    };

    if constexpr (STAGED) {
        // Every (quarter, row) entry is one Q8_1 block: its codes go to LDS as they are, its scale into
        // the table. The first round's loads are issued before the first weight loads and consumed
        // after them (loads return in issue order: asked for after the weights, the activation, which
        // sits in L2, would wait for HBM).
        constexpr int PER = 4;
        uint32_t head[PER];
        u32x4 lo[PER], hi[PER];   // (native vectors: the struct type of the same shape stays in scratch memory here)
        auto issue = [&](int base) {
#pragma unroll
            for (int u = 0; u < PER; ++u) {
                const int idx = min(base + u * WG, entries - 1);
                const int sub = idx / TW, tok = min(idx % TW, m_count - 1);
                const uint8_t* b = y0 + ((size_t)tok * p.stride_y + sub) * Q81_BYTES;
                head[u] = *(const uint32_t*)b;
                lo[u] = *(const u32x4_a4*)(b + 4);
                hi[u] = *(const u32x4_a4*)(b + 20);
            }
        };
        auto place = [&](int base) {
#pragma unroll
            for (int u = 0; u < PER; ++u) {
                const int idx = base + u * WG;
                if (idx < entries) {
                    d8_table[idx] = idx % TW < m_count ? f16_bits_to_f32(head[u] & 0xFFFFu) : 0.f;
                    *(u32x4*)(codes + (size_t)idx * 32) = lo[u];
                    *(u32x4*)(codes + (size_t)idx * 32 + 16) = hi[u];
                }
            }
        };
        constexpr int DEPTH = 3;   // steps of weight loads a wave keeps in flight (registers)
        WFrag f[DEPTH];
        issue(threadIdx.x);
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
            if (d < total) load_weights(f[d], weights_at(d), lh);
        place(threadIdx.x);
        for (int r = WG * PER; r < entries; r += WG * PER) {
            issue(r + threadIdx.x);
            place(r + threadIdx.x);
        }
        __syncthreads();
        if (my_blocks == 0) {   // rows shorter than four super-blocks: this wave only keeps the barriers
            for (int t = 0; t < my_tiles; ++t) finish_tile(t);
            return;
        }
        // the lane's A operand: activation row l32 (rows the launch does not have repeat the live
        // ones; their results sit in registers nobody reads), codes 16 lh .. 16 lh + 15 of the quarter
        const uint8_t* a_lane = codes + (l32 % TW) * 32 + 16 * lh;
        for (int j0 = 0; j0 < total; j0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                const int j = j0 + d;
                if (j < total) {
                    const int kb = wave + (j % my_blocks) * WAVES;
                    block_step<G>(f[d], true, kb * 8, d8_table, lh, keep0, keep1,
                                  [&](int q) { return *(const v4i*)(a_lane + (size_t)(kb * 8 + q) * TW * 32); }, acc);
                    if (j + DEPTH < total) load_weights(f[d], weights_at(j + DEPTH), lh);
                    if ((j + 1) % my_blocks == 0) finish_tile(j / my_blocks);
                }
            }
        }
    } else {
        // Activation scales of this pass, zero for the rows the pass does not have. Eight loads are
        // issued before the first is used: one at a time, each would cost a memory latency.
        for (int base = threadIdx.x; base < entries; base += WG * 8) {
            uint32_t bits[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = min(base + u * WG, entries - 1);
                const int sub = idx / TW, tok = min(idx % TW, m_count - 1);
                bits[u] = *(const uint16_t*)(y0 + ((size_t)tok * p.stride_y + sub) * Q81_BYTES);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = base + u * WG;
                if (idx < entries) d8_table[idx] = idx % TW < m_count ? f16_bits_to_f32(bits[u]) : 0.f;
            }
        }
        // The lane's activation row (a row past the end re-reads the last one; its scales are zero).
        const uint8_t* y_lane = y0 + (size_t)min(l32, m_count - 1) * p.stride_y * Q81_BYTES + 4 + 16 * lh;
        struct Frag {
            WFrag w;
            v4i a[8];
        };
        auto load = [&](Frag& f, int j) {
            load_weights(f.w, weights_at(j), lh);
            const int kb = wave + (j % my_blocks) * WAVES;
            const uint8_t* ap = y_lane + (size_t)kb * 8 * Q81_BYTES;
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const uint4 t = *(const uint4_a4*)(ap + s * Q81_BYTES);
                f.a[s] = v4i{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
        };
        Frag fa, fb;
        if (total > 0) load(fa, 0);
        __syncthreads();   // the scale table is complete
        if (my_blocks == 0) {
            for (int t = 0; t < my_tiles; ++t) finish_tile(t);
            return;
        }
        auto step = [&](const Frag& f, int j) {
            const int kb = wave + (j % my_blocks) * WAVES;
            block_step<G>(f.w, true, kb * 8, d8_table, lh, keep0, keep1, [&](int q) { return f.a[q]; }, acc);
            if ((j + 1) % my_blocks == 0) finish_tile(j / my_blocks);
        };
        for (int j = 0; j < total; j += 2) {
            if (j + 1 < total) load(fb, j + 1);
            step(fa, j);
            if (j + 1 >= total) break;
            if (j + 2 < total) load(fa, j + 2);
            step(fb, j + 1);
        }
    }
}

template <int G, bool STAGED, int WAVES>
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
               hipFuncSetAttribute((const void*)q6k_rows_kernel<G, STAGED, WAVES>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        r = 0;
    } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q6k_rows_kernel<G, STAGED, WAVES>, 64 * WAVES,
                                                            (size_t)lds_bytes) != hipSuccess || r < 1) {
        (void)hipGetLastError();
        r = 1;
    }
    by_lds.emplace(lds_bytes, r);
    return r;
}

// -1: the kernel's LDS image does not fit (the caller tries the next form).
template <int G, bool STAGED, int WAVES>
int launch_waves(const Args& a, hipStream_t stream) {
    const int lds_bytes = lds_bytes_for<G, STAGED, WAVES>(a.nb);
    const int per_cu = resident_cap<G, STAGED, WAVES>(lds_bytes);
    if (per_cu == 0) return -1;
    const int n_tiles = (a.n + 31) / 32, groups = STAGED ? 1 : (a.m + TOK - 1) / TOK;
    if (groups > 65535) return LK_ERR_ARG;
    int cap = lk_device().cus * per_cu / groups;
    if (cap < 1) cap = 1;
    hipLaunchKernelGGL((q6k_rows_kernel<G, STAGED, WAVES>), dim3(n_tiles < cap ? n_tiles : cap, groups), dim3(64 * WAVES), lds_bytes, stream, a);
    return lk_launch_status();
}

template <int G, bool STAGED>
int launch(const Args& a, hipStream_t stream) {
    // eight waves when the tiles (times the passes of 32 rows) do not fill the CUs and a wave would
    // otherwise walk four super-blocks or more in turn (measured at 32 / 64 rows, four against eight waves:
    // 2048 x 6144 41.8 / 42.6 -> 36.5 / 37.6 us, 4096 x 4096 34.6 / 35.8 -> 31.9 / 33.4; rows of eight
    // super-blocks lose, 25.8 -> 27.4)
    const int n_tiles = (a.n + 31) / 32, groups = STAGED ? 1 : (a.m + TOK - 1) / TOK;
    const int forced = lk_tune_env("LK_TUNE_ROWS_WAVES");
    const bool eight = forced ? forced == 8 : (n_tiles * groups <= lk_device().cus && a.nb >= 16);
    if (eight) {
        const int rc = launch_waves<G, STAGED, 8>(a, stream);
        if (rc >= 0) return rc;
    }
    return launch_waves<G, STAGED, 4>(a, stream);
}

}  // namespace

// Q6_K weight [size_n rows, size_k] x plain Q8_1 rows [size_m, stride_y blocks apart] -> output
// [size_m, ldd floats apart] f32. LK_ERR_ARG (nothing launched) when the rows are too long for the
// scale table in LDS.
int lk_q6k_rows_mfma(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k, int stride_y,
                     int ldd, hipStream_t stream) {
    if (size_m == 0 || size_n == 0) return LK_OK;
    if (!w || !q8_1 || !output || size_m < 0 || size_n < 0 || size_k <= 0 || size_k % 256 != 0) return LK_ERR_ARG;
    if (stride_y < size_k / 32 || ldd < size_n) return LK_ERR_ARG;
    if ((((uintptr_t)w) & 1) != 0 || (((uintptr_t)q8_1) & 3) != 0) return LK_ERR_ARG;
    Args a{(const uint8_t*)w, (const uint8_t*)q8_1, output, size_k / 256, size_n, size_m, stride_y, ldd};
    int rc = -1;
    if (size_m <= 64) {
        // 16-row tiles (rows16_q6k.hip): a quarter of the matrix-unit time per weight, and every CU a tile
        // (above 16 rows: sets of eight rows, for a small matrix that L2 holds; the launcher declines the rest)
        rc = lk_rows16_q6k(w, q8_1, output, size_m, size_n, size_k, stride_y, ldd, stream);
        if (rc >= 0) return rc;
    }
    if (size_m <= 8) {
        rc = launch<1, true>(a, stream);
        if (rc < 0) rc = launch<1, false>(a, stream);
    } else if (size_m <= 16) {
        rc = launch<2, true>(a, stream);
        if (rc < 0) rc = launch<2, false>(a, stream);
    } else {
        rc = launch<4, false>(a, stream);
    }
    return rc < 0 ? LK_ERR_ARG : rc;
}

extern "C" int lk_dense_q6k_rows(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                                 void* stream) {
    return lk_q6k_rows_mfma(w, q8_1, output, size_m, size_n, size_k, size_k / 32, size_n, (hipStream_t)stream);
}

// Kernels and launch geometry of the mat-vec family, shared by the per-engine translation units
// (one per weight format engine, so that they compile side by side) and by mmvq.hip, which holds
// the entry points.
#pragma once

#include "mmvq_core.h"

#include <cstdlib>
#include <mutex>
#include <unordered_map>

namespace mmvq {


// Up to four same-format, same-k matrices over one activation in one launch (q/k/v, gate/up).
// Workgroups [wg_begin[i], wg_begin[i+1]) serve matrix i.
constexpr int MAX_MULTI = 4;
struct MultiArgs {
    const uint8_t* vx[MAX_MULTI];
    void* dst[MAX_MULTI];
    const float* bias[MAX_MULTI];
    int n[MAX_MULTI];
    int wg_begin[MAX_MULTI + 1];
    int count;
};

template <class E, int B, int R, typename T>
__global__ __launch_bounds__(WG) void mmvq_kernel(MultiArgs m, const uint8_t* __restrict__ vy, int nb,
                                                  int stride_col_y, int stride_col_dst, int act_stride_f32) {
    extern __shared__ __align__(16) uint8_t lds[];
    // Which matrix this workgroup serves. Every field is read at a fixed index and picked with a
    // mask, so the kernel arguments the first loads need arrive in one round of scalar loads
    // (indexing the arrays by a computed `w`, or reading them under a branch, costs further
    // dependent rounds before the first weight load can go out).
    static_assert(MAX_MULTI == 4, "the pin below lists four matrices");
    uintptr_t vxs[MAX_MULTI];
    int ns[MAX_MULTI], begins[MAX_MULTI + 1], count = m.count;
#pragma unroll
    for (int i = 0; i < MAX_MULTI; ++i) {
        vxs[i] = (uintptr_t)m.vx[i];
        ns[i] = m.n[i];
        begins[i] = m.wg_begin[i];
    }
    begins[MAX_MULTI] = m.wg_begin[MAX_MULTI];
    // Pinned together: left alone, the compiler reads m.vx only after it has waited for the
    // other fields, which puts a second scalar round trip in front of the first weight load.
    asm volatile("" : "+s"(vxs[0]), "+s"(vxs[1]), "+s"(vxs[2]), "+s"(vxs[3]), "+s"(ns[0]), "+s"(ns[1]), "+s"(ns[2]),
                 "+s"(ns[3]), "+s"(begins[1]), "+s"(begins[2]), "+s"(begins[3]), "+s"(begins[4]), "+s"(count));
    int w = 0;
#pragma unroll
    for (int i = 1; i < MAX_MULTI; ++i)
        if (i < count && (int)blockIdx.x >= begins[i]) w = i;
    uintptr_t vx_bits = 0, dst_bits = 0, bias_bits = 0;
    uint32_t n_bits = 0, first_bits = 0, end_bits = 0;
#pragma unroll
    for (int i = 0; i < MAX_MULTI; ++i) {
        const uint32_t pick = 0u - (uint32_t)(w == i);
        const uintptr_t pick64 = (uintptr_t)(int64_t)(int32_t)pick;
        vx_bits |= vxs[i] & pick64;
        dst_bits |= (uintptr_t)m.dst[i] & pick64;
        bias_bits |= (uintptr_t)m.bias[i] & pick64;
        n_bits |= (uint32_t)ns[i] & pick;
        first_bits |= (uint32_t)(i ? begins[i] : 0) & pick;
        end_bits |= (uint32_t)begins[i + 1] & pick;
    }
    const gbytes_t vx = to_gbytes((uint64_t)vx_bits);
    T* dst = (T*)(uint8_t*)to_gbytes((uint64_t)dst_bits);
    const float* bias = (const float*)to_gbytes((uint64_t)bias_bits);
    const int n = (int)n_bits, wg_first = (int)first_bits, wg_end = (int)end_bits;
    RowJob<1> job{{vx}, vy, nb, n, stride_col_y, (wg_end - wg_first) * WAVES, ((int)blockIdx.x - wg_first) * WAVES,
                  act_stride_f32};
    E::template run<B, R, 1>(job, lds, [&](int row, int c, const float* tot) {
        float v = tot[0];
        if (bias) v += bias[row];
        dst[(size_t)c * stride_col_dst + row] = from_f32<T>(v);
    });
}

// gate and up rows over one activation, out = act(gate) * up (fast_mmvq::try_fused of the
// reference, src/tensor/quantized/fast_mmvq.rs:97-282; kernels mmvq_gguf_pair_*_silu and
// *_fused_{silu,gelu}, src/inference/cuda/mmvq_gguf.cu:588-758).
static __device__ __forceinline__ float act_silu(float g) { return g / (1.0f + expf(-g)); }
static __device__ __forceinline__ float act_gelu_tanh(float g) {
    return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * g * (1.0f + 0.044715f * g * g)));
}

template <class E, int B, int R, typename T, int ACT>
__global__ __launch_bounds__(WG) void mmvq_pair_kernel(const uint8_t* __restrict__ gate, const uint8_t* __restrict__ up,
                                                       const uint8_t* __restrict__ vy, T* __restrict__ dst, int nb,
                                                       int n, int stride_col_y, int stride_col_dst) {
    extern __shared__ __align__(16) uint8_t lds[];
    RowJob<2> job{{to_gbytes(gate), to_gbytes(up)}, vy, nb, n, stride_col_y, (int)gridDim.x * WAVES, (int)blockIdx.x * WAVES};
    E::template run<B, R, 2>(job, lds, [&](int row, int c, const float* tot) {
        const float a = ACT == 0 ? act_silu(tot[0]) : act_gelu_tanh(tot[0]);
        dst[(size_t)c * stride_col_dst + row] = from_f32<T>(a * tot[1]);
    });
}

// The same pair launch handing its result on as Q8_1 blocks: out = Q8_1(act(gate . x) * (up . x)),
// which is what the down projection reads, so a decode layer needs no quantizer launch between
// the two. A workgroup owns whole blocks of 32 consecutive output rows (wave w rows 8w .. 8w + 7 of
// the block, one after the other); the 32 results meet in LDS and eight lanes quantize them with
// the stand-alone quantizer's steps (d = amax / 127, codes = round_half_away(v * (1 / d)),
// s = f16(sum * d)), so the bytes are those lk_quantize_q8_1 writes for the same f32 values.
template <class E, int B, int R, int ACT>
__global__ __launch_bounds__(WG) void mmvq_pair_q8_1_kernel(const uint8_t* __restrict__ gate, const uint8_t* __restrict__ up,
                                                            const uint8_t* __restrict__ vy, uint32_t* __restrict__ dst,
                                                            int nb, int n, int stride_col_y, int stride_dst_blocks,
                                                            int act_stride_f32, int lds_act_bytes) {
#pragma clang fp contract(off)
    extern __shared__ __align__(16) uint8_t lds[];
    float* meet = (float*)(lds + lds_act_bytes);   // [2][B][32]: two blocks in flight
    // tiles of R rows: a block of 32 rows is 32 / R tiles, a wave's run 8 / R of them
    constexpr int RUN = 8 / R;
    RowJob<2> job{{to_gbytes(gate), to_gbytes(up)}, vy, nb, n, stride_col_y, (32 / R) * (int)gridDim.x - (RUN - 1),
                  (32 / R) * (int)blockIdx.x, act_stride_f32, RUN, RUN};
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int half = 0;   // which of the two meeting buffers this workgroup's current block uses
    E::template run<B, R, 2>(
        job, lds,
        [&](int row, int c, const float* tot) {
            const float a = ACT == 0 ? act_silu(tot[0]) : act_gelu_tanh(tot[0]);
            meet[(half * B + c) * 32 + (row & 31)] = a * tot[1];
        },
        [&](int tile) {
            if (((tile + 1) & (RUN - 1)) != 0) return;   // the wave's run of eight rows is not over
            const int row = tile * R;
            __syncthreads();              // every wave of the workgroup has delivered its eight
            const int mine = half;
            half ^= 1;   // the next block meets in the other buffer: a wave may run one block ahead
            if (wave == 0 && lane < 8 * B) {
                const int c = lane >> 3, l8 = lane & 7, block = row >> 5;
                const float4 v = *(const float4*)(meet + (mine * B + c) * 32 + 4 * l8);
                const float amax = max8(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
                const float d = amax / 127.0f;
                const float inv = d != 0.0f ? 1.0f / d : 0.0f;
                const int q0 = (int)roundf(v.x * inv), q1 = (int)roundf(v.y * inv);
                const int q2 = (int)roundf(v.z * inv), q3 = (int)roundf(v.w * inv);
                int quad;
                const int sum = sum8(q0 + q1 + q2 + q3, quad);
                uint32_t* out = dst + ((size_t)c * stride_dst_blocks + block) * 9;
                out[1 + l8] = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
                              ((uint32_t)(q3 & 0xFF) << 24);
                if (l8 == 0) {
                    const uint32_t dh = __half_as_ushort(__float2half_rn(d));
                    float scaled_sum = (float)sum * d;
                    asm volatile("" : "+v"(scaled_sum));   // two roundings, as the quantizer's
                    out[0] = dh | ((uint32_t)__half_as_ushort(__float2half_rn(scaled_sum)) << 16);
                }
            }
        });
}

// `groups` weights of one shape, each over its OWN activation row: weight g (address table[g])
// reads the Q8_1 blocks from g * k/32 and writes dst from g * n (mmvq_f32_grouped,
// src/tensor/cuda/quant.rs:3418-3466).
template <class E, int R>
__global__ __launch_bounds__(WG) void mmvq_grouped_kernel(const uint64_t* __restrict__ table,
                                                          const uint8_t* __restrict__ vy, float* __restrict__ dst,
                                                          int nb, int n, int k32) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int g = blockIdx.y;
    RowJob<1> job{{to_gbytes(table[g])}, vy + (size_t)g * k32 * Q81_BYTES, nb, n, k32,
                  (int)gridDim.x * WAVES, (int)blockIdx.x * WAVES};
    float* out = dst + (size_t)g * n;
    E::template run<1, R, 1>(job, lds, [&](int row, int, const float* tot) { out[row] = tot[0]; });
}


// --------------------------------------------------------------------------------------------
// Host dispatch
// --------------------------------------------------------------------------------------------

// Launch geometry. `R` rows per wave and the number of resident workgroups per CU set how many
// bytes are in flight; both have measured optima below "as many as fit" (HBM throughput drops
// when too many requests are outstanding). LK_TUNE_WGS_PER_CU overrides the built-in cap for
// measurement runs.

// Per kernel instance and LDS size: raise the dynamic-LDS limit once and ask the runtime how many
// workgroups a CU holds. Cached, so steady-state launches (and launches recorded into a graph)
// make no runtime query. Returns workgroups resident per CU, 0 on failure.
template <typename K>
static int resident_per_cu(K kernel, int lds_bytes, int engine_cap = 8) {
    static std::mutex mu;
    static std::unordered_map<int, int> by_lds;
    std::lock_guard<std::mutex> lock(mu);
    auto it = by_lds.find(lds_bytes);
    if (it != by_lds.end()) return it->second;
    if (lds_bytes > lk_device().lds_bytes) return 0;
    if (lds_bytes > 48 * 1024 &&
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int r = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)kernel, WG, (size_t)lds_bytes) != hipSuccess || r < 1) {
        (void)hipGetLastError();
        r = 1;
    }
    static const int forced = lk_tune_env("LK_TUNE_WGS_PER_CU");
    const int cap = forced > 0 ? forced : engine_cap;
    r = r > cap ? cap : r;
    by_lds.emplace(lds_bytes, r);
    return r;
}

static inline int wgs_for_rows(int n, int rows_per_wave) {
    const int tiles = (n + rows_per_wave - 1) / rows_per_wave;
    return (tiles + WAVES - 1) / WAVES;
}

struct MmvqCall {
    MultiArgs m;
    const uint8_t* vy;
    int nb, stride_col_y, stride_col_dst;
    int act_stride_f32;  // non-zero: vy is f32 rows, quantized in the kernel
    hipStream_t stream;
};

template <class E, int B, int R, typename T>
static int launch_plain_r(MmvqCall& a) {
    auto kernel = mmvq_kernel<E, B, R, T>;
    const int lds_bytes = lds_bytes_for<typename E::Fmt>(a.nb, B);
    const int per_cu = resident_per_cu(kernel, lds_bytes, B == 1 && R == 1 ? E::WGS_PER_CU_ONE_ROW : 8);
    if (per_cu == 0) return LK_ERR_ARG;
    // Persistent grid: no more workgroups than are resident at once, shared out over the
    // matrices in proportion to their rows.
    const int capacity = lk_device().cus * per_cu;
    int need[MAX_MULTI], total = 0;
    for (int i = 0; i < a.m.count; ++i) {
        need[i] = wgs_for_rows(a.m.n[i], R * E::rows_per_pass(a.nb));
        total += need[i];
    }
    a.m.wg_begin[0] = 0;
    for (int i = 0; i < a.m.count; ++i) {
        int share = need[i];
        if (total > capacity) {
            share = (int)((int64_t)need[i] * capacity / total);
            if (share < 1) share = 1;
        }
        a.m.wg_begin[i + 1] = a.m.wg_begin[i] + share;
    }
    for (int i = a.m.count; i < MAX_MULTI; ++i) a.m.wg_begin[i + 1] = a.m.wg_begin[i];
    hipLaunchKernelGGL(kernel, dim3(a.m.wg_begin[a.m.count]), dim3(WG), lds_bytes, a.stream, a.m, a.vy, a.nb,
                       a.stride_col_y, a.stride_col_dst, a.act_stride_f32);
    return lk_launch_status();
}

// Rows per wave: two rows share every activation read, except where an engine measured faster with
// one row per tile at one activation row (E::ONE_ROW_TILES: Q6_K long rows, with three workgroups per
// CU: 4096 x 14336 12.8 against 13.7 us, 2048 x 6144 5.0 against 5.8; Q4_K / Q5_K / Q8_0 lose with it).
// LK_TUNE_R = 1 / 2 selects the form for measurement runs (batch <= 4).
template <class E, int B, typename T>
static int launch_plain(MmvqCall& a) {
    static const int forced = lk_tune_env("LK_TUNE_R");
    // (not from f32 rows: there every workgroup quantizes the row first, and more, lighter workgroups pay that more often)
    const bool one = forced ? forced == 1 : (B == 1 && E::ONE_ROW_TILES && a.act_stride_f32 == 0);
    if (B <= 4 && one) return launch_plain_r<E, B, 1, T>(a);
    return launch_plain_r<E, B, 2, T>(a);
}

#define LK_BATCH_SWITCH(FN, E, T, ARG)                                                                 \
    switch (batch) {                                                                                  \
        case 1: return FN<E, 1, T>(ARG);                                                              \
        case 2: return FN<E, 2, T>(ARG);                                                              \
        case 3: return FN<E, 3, T>(ARG);                                                              \
        case 4: return FN<E, 4, T>(ARG);                                                              \
        case 5: return FN<E, 5, T>(ARG);                                                              \
        case 6: return FN<E, 6, T>(ARG);                                                              \
        case 7: return FN<E, 7, T>(ARG);                                                              \
        case 8: return FN<E, 8, T>(ARG);                                                              \
        default: return LK_ERR_ARG;                                                                   \
    }


template <class E, int B, typename T>
static int launch_pair(const uint8_t* gate, const uint8_t* up, const uint8_t* vy, void* dst, int nb, int n,
                       int stride_col_y, int stride_col_dst, int act, hipStream_t s) {
    constexpr int R = 1;
    const int lds_bytes = lds_bytes_for<typename E::Fmt>(nb, B);
    auto launch = [&](auto kernel) {
        const int per_cu = resident_per_cu(kernel, lds_bytes);
        if (per_cu == 0) return (int)LK_ERR_ARG;
        const int need = wgs_for_rows(n, R * E::rows_per_pass(nb)), cap = lk_device().cus * per_cu;
        hipLaunchKernelGGL(kernel, dim3(need < cap ? need : cap), dim3(WG), lds_bytes, s, gate, up, vy, (T*)dst, nb, n,
                           stride_col_y, stride_col_dst);
        return lk_launch_status();
    };
    return act == 0 ? launch(mmvq_pair_kernel<E, B, R, T, 0>) : launch(mmvq_pair_kernel<E, B, R, T, 1>);
}

template <class E, int B>
static int launch_pair_q8_1(const uint8_t* gate, const uint8_t* up, const uint8_t* vy, void* dst, int nb, int n,
                            int stride_col_y, int stride_dst_blocks, int act_stride_f32, int act, hipStream_t s) {
    const int lds_act = lds_bytes_for<typename E::Fmt>(nb, B), lds_bytes = lds_act + 2 * B * 32 * (int)sizeof(float);
    auto launch = [&](auto kernel) {
        const int per_cu = resident_per_cu(kernel, lds_bytes);
        if (per_cu == 0) return (int)LK_ERR_ARG;
        const int blocks = n / 32, cap = lk_device().cus * per_cu;
        hipLaunchKernelGGL(kernel, dim3(blocks < cap ? blocks : cap), dim3(WG), lds_bytes, s, gate, up, vy, (uint32_t*)dst,
                           nb, n, stride_col_y, stride_dst_blocks, act_stride_f32, lds_act);
        return lk_launch_status();
    };
    constexpr int R = 1;   // (two rows per tile measured slower here: 16.5 against 15.7 us on 2 x 14336 x 4096)
    return act == 0 ? launch(mmvq_pair_q8_1_kernel<E, B, R, 0>) : launch(mmvq_pair_q8_1_kernel<E, B, R, 1>);
}

template <class E>
static int launch_grouped(const uint64_t* table, int groups, const uint8_t* vy, float* dst, int nb, int n, int k32,
                          hipStream_t s) {
    constexpr int R = 2;
    auto kernel = mmvq_grouped_kernel<E, R>;
    const int lds_bytes = lds_bytes_for<typename E::Fmt>(nb, 1);
    const int per_cu = resident_per_cu(kernel, lds_bytes);
    if (per_cu == 0) return LK_ERR_ARG;
    const int need = wgs_for_rows(n, R * E::rows_per_pass(nb));
    int cap = lk_device().cus * per_cu / groups;
    if (cap < 1) cap = 1;
    hipLaunchKernelGGL(kernel, dim3(need < cap ? need : cap, groups), dim3(WG), lds_bytes, s, table, vy, dst, nb, n, k32);
    return lk_launch_status();
}


// What an engine's translation unit defines, for every batch and output type it serves.
template <class E>
static int eng_plain(int batch, int dst_type, MmvqCall& a) {
    switch (dst_type) {
        case LK_TYPE_F32: LK_BATCH_SWITCH(launch_plain, E, float, a)
        case LK_TYPE_F16: LK_BATCH_SWITCH(launch_plain, E, __half, a)
        case LK_TYPE_BF16: LK_BATCH_SWITCH(launch_plain, E, __hip_bfloat16, a)
        default: return LK_ERR_TYPE;
    }
}

struct PairCall {
    const uint8_t *gate, *up, *vy;
    void* dst;
    int nb, n, stride_col_y, stride_col_dst, act;
    int act_stride_f32;   // pair_q8_1 only
    hipStream_t stream;
};

template <class E>
static int eng_pair(int batch, int dst_type, const PairCall& c) {
#define LK_PAIR(T)                                                                                                       \
    switch (batch) {                                                                                                     \
        case 1: return launch_pair<E, 1, T>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act, c.stream);  \
        case 2: return launch_pair<E, 2, T>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act, c.stream);  \
        case 3: return launch_pair<E, 3, T>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act, c.stream);  \
        default: return launch_pair<E, 4, T>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act, c.stream); \
    }
    switch (dst_type) {
        case LK_TYPE_F32: LK_PAIR(float)
        case LK_TYPE_BF16: LK_PAIR(__hip_bfloat16)
        default: return LK_ERR_TYPE;
    }
#undef LK_PAIR
}

template <class E>
static int eng_pair_q8_1(int batch, const PairCall& c) {
    switch (batch) {
        case 1: return launch_pair_q8_1<E, 1>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act_stride_f32, c.act, c.stream);
        case 2: return launch_pair_q8_1<E, 2>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act_stride_f32, c.act, c.stream);
        case 3: return launch_pair_q8_1<E, 3>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act_stride_f32, c.act, c.stream);
        default: return launch_pair_q8_1<E, 4>(c.gate, c.up, c.vy, c.dst, c.nb, c.n, c.stride_col_y, c.stride_col_dst, c.act_stride_f32, c.act, c.stream);
    }
}

}  // namespace mmvq

// One set of functions per engine, defined in mmvq_eng_<name>.hip.
#define LK_DECLARE_ENGINE(NAME)                                                                                   \
    int lk_eng_plain_##NAME(int batch, int dst_type, mmvq::MmvqCall& a);                                           \
    int lk_eng_pair_##NAME(int batch, int dst_type, const mmvq::PairCall& c);                                      \
    int lk_eng_pair_q8_1_##NAME(int batch, const mmvq::PairCall& c);                                               \
    int lk_eng_grouped_##NAME(const uint64_t* table, int groups, const uint8_t* vy, float* dst, int nb, int n, int k32, \
                              hipStream_t s);
#define LK_DEFINE_ENGINE(NAME, E)                                                                                  \
    int lk_eng_plain_##NAME(int batch, int dst_type, mmvq::MmvqCall& a) { return mmvq::eng_plain<E>(batch, dst_type, a); } \
    int lk_eng_pair_##NAME(int batch, int dst_type, const mmvq::PairCall& c) { return mmvq::eng_pair<E>(batch, dst_type, c); } \
    int lk_eng_pair_q8_1_##NAME(int batch, const mmvq::PairCall& c) { return mmvq::eng_pair_q8_1<E>(batch, c); }   \
    int lk_eng_grouped_##NAME(const uint64_t* table, int groups, const uint8_t* vy, float* dst, int nb, int n, int k32, \
                              hipStream_t s) {                                                                     \
        return mmvq::launch_grouped<E>(table, groups, vy, dst, nb, n, k32, s);                                     \
    }
LK_DECLARE_ENGINE(q4k)
LK_DECLARE_ENGINE(q4k_short)
LK_DECLARE_ENGINE(q5k)
LK_DECLARE_ENGINE(q5k_short)
LK_DECLARE_ENGINE(q6k)
LK_DECLARE_ENGINE(q6k_short)
LK_DECLARE_ENGINE(q80)

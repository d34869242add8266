// Decode mat-vec launchers: GGUF weight rows (Q4_K / Q6_K / Q8_0) against 1..8 Q8_1 activation
// rows, plus the fused neighbours that share its engine (several matrices over one activation,
// gate/up pairs with the activation function applied in the store, grouped launches).
//
// Bandwidth work, so the design is about bytes in flight, not arithmetic:
//   * a lane loads 16 weight bytes per instruction (global_load_dwordx4); a wave takes whole
//     super-blocks side by side (Q4_K 4 lanes per 256-value block and 16 blocks = 4096 values
//     per pass; Q6_K 8 lanes per block; Q8_0 2 lanes per 32-value block);
//   * a wave owns R consecutive weight rows end to end (no cross-wave reduction) and persists
//     over row tiles, with the next tile's loads in flight while the current one is consumed;
//   * the Q8_1 activation is staged ONCE per workgroup into LDS, re-laid so that the 16 bytes a
//     lane needs sit at lane*16 of a plane (conflict-free ds_read_b128), with its f16 scales
//     widened to f32 and, for Q4_K, d8 * sum(codes) precomputed for the min term;
//   * 6-bit scales / mins are unpacked in registers from the 16-byte block header;
//   * integer products are v_dot4_i32_i8; per-lane f32 partials meet in one wave64 DPP
//     reduction per row.
// The engines live in mmvq_core.h.

#include "mmvq_core.h"

#include <cstdlib>
#include <mutex>
#include <unordered_map>

using namespace mmvq;

namespace {

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
// Sub-block-dot probe: one wave per (row, pass), activation read straight from global memory.
// --------------------------------------------------------------------------------------------
static __device__ __forceinline__ void load_act16(const uint8_t* vy, int q81_block, int lh, uint4& a) {
    const uint32_t* src = (const uint32_t*)(vy + (size_t)q81_block * Q81_BYTES) + 1 + 4 * lh;
    a = make_uint4(src[0], src[1], src[2], src[3]);
}

__global__ __launch_bounds__(64) void subdots_q4k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7, p = ch >> 1, lh = ch & 1;
    int d_lo = 0, d_hi = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q4K_BYTES;
        const uint4 q = *(const uint4*)(bp + 16 + 16 * ch);
        uint4 a_lo, a_hi;
        load_act16(vy, blk * 8 + 2 * p, lh, a_lo);
        load_act16(vy, blk * 8 + 2 * p + 1, lh, a_hi);
        q4k_dots(q, a_lo, a_hi, d_lo, d_hi);
    }
    d_lo += __shfl_xor(d_lo, 1);
    d_hi += __shfl_xor(d_hi, 1);
    if (blk < nb && lh == 0) {
        int32_t* out = dots + (size_t)row * nb * 8 + blk * 8 + 2 * p;
        out[0] = d_lo;
        out[1] = d_hi;
    }
}

__global__ __launch_bounds__(64) void subdots_q5k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7, p = ch >> 1, lh = ch & 1;
    int d_lo = 0, d_hi = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q5K_BYTES;
        const uint4 q = *(const uint4*)(bp + 48 + 16 * ch);
        const uint4 qh = *(const uint4*)(bp + 16 + 16 * lh);
        uint4 a_lo, a_hi;
        load_act16(vy, blk * 8 + 2 * p, lh, a_lo);
        load_act16(vy, blk * 8 + 2 * p + 1, lh, a_hi);
        q5k_dots(q, shr4(qh, 2 * p), a_lo, a_hi, d_lo, d_hi);
    }
    d_lo += __shfl_xor(d_lo, 1);
    d_hi += __shfl_xor(d_hi, 1);
    if (blk < nb && lh == 0) {
        int32_t* out = dots + (size_t)row * nb * 8 + blk * 8 + 2 * p;
        out[0] = d_lo;
        out[1] = d_hi;
    }
}

__global__ __launch_bounds__(64) void subdots_q6k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7;
    const int h = ch >> 2, g0 = (ch >> 1) & 1, lh = ch & 1;
    if (blk >= nb) return;
    const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q6K_BYTES;
    const uint4 ql = *(const uint4_a2*)(bp + 16 * ch);
    const uint4 qh = *(const uint4_a2*)(bp + 128 + 16 * (2 * h + lh));
    uint4 a_a, a_b;
    load_act16(vy, blk * 8 + 4 * h + g0, lh, a_a);
    load_act16(vy, blk * 8 + 4 * h + g0 + 2, lh, a_b);
    int d_a, d_b;
    q6k_dots(ql, qh, g0, a_a, a_b, d_a, d_b);
    int32_t* out = dots + (size_t)row * nb * 16 + blk * 16;
    out[8 * h + 2 * g0 + lh] = d_a;
    out[8 * h + 2 * (g0 + 2) + lh] = d_b;
}

__global__ __launch_bounds__(64) void subdots_q80_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 32 + (lane >> 1), lh = lane & 1;
    int d = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q80_BYTES;
        const uint4 q = *(const uint4_a2*)(bp + 2 + 16 * lh);
        uint4 a;
        load_act16(vy, blk, lh, a);
        d = dot16(q, a, 0);
    }
    d += __shfl_xor(d, 1);
    if (blk < nb && lh == 0) dots[(size_t)row * nb + blk] = d;
}

__global__ void act_sums_kernel(const uint8_t* __restrict__ vy, int32_t* __restrict__ sums, int k32) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= k32) return;
    uint4 lo, hi;
    load_act16(vy, j, 0, lo);
    load_act16(vy, j, 1, hi);
    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
    sums[j] = dot16(ones, hi, dot16(ones, lo, 0));
}

// --------------------------------------------------------------------------------------------
// Host dispatch
// --------------------------------------------------------------------------------------------

// Launch geometry. `R` rows per wave and the number of resident workgroups per CU set how many
// bytes are in flight; both have measured optima below "as many as fit" (HBM throughput drops
// when too many requests are outstanding). LK_TUNE_WGS_PER_CU overrides the built-in cap for
// measurement runs.
static int tune_env(const char* name) {
    const char* v = getenv(name);
    return v ? atoi(v) : 0;
}

// Per kernel instance and LDS size: raise the dynamic-LDS limit once and ask the runtime how many
// workgroups a CU holds. Cached, so steady-state launches (and launches recorded into a graph)
// make no runtime query. Returns workgroups resident per CU, 0 on failure.
template <typename K>
static int resident_per_cu(K kernel, int lds_bytes) {
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
    static const int forced = tune_env("LK_TUNE_WGS_PER_CU");
    const int cap = forced > 0 ? forced : 8;
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
    const int per_cu = resident_per_cu(kernel, lds_bytes);
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

// Rows per wave: two rows share every activation read. LK_TUNE_R=1 selects one row per tile for
// measurement runs (batch <= 4).
template <class E, int B, typename T>
static int launch_plain(MmvqCall& a) {
    static const int forced = tune_env("LK_TUNE_R");
    if (B <= 4 && forced == 1) return launch_plain_r<E, B, 1, T>(a);
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

template <typename T>
static int dispatch_plain(int wtype, int batch, MmvqCall& a) {
    switch (wtype) {
        case LK_TYPE_Q4_K:
            if (a.nb <= 8) { LK_BATCH_SWITCH(launch_plain, EngQ4KShort, T, a) }
            LK_BATCH_SWITCH(launch_plain, EngQ4K, T, a)
        case LK_TYPE_Q5_K:
            if (a.nb <= 8) { LK_BATCH_SWITCH(launch_plain, EngQ5KShort, T, a) }
            LK_BATCH_SWITCH(launch_plain, EngQ5K, T, a)
        case LK_TYPE_Q6_K: LK_BATCH_SWITCH(launch_plain, EngQ6K, T, a)
        case LK_TYPE_Q8_0: LK_BATCH_SWITCH(launch_plain, EngQ80, T, a)
        default: return LK_ERR_TYPE;
    }
}

static int check_common(int wtype, const void* vy, int ncols_x, int batch, int stride_col_y) {
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (!vy || ncols_x <= 0 || ncols_x % bl != 0) return LK_ERR_ARG;
    if (batch < 1 || batch > 8 || stride_col_y < ncols_x / 32) return LK_ERR_ARG;
    if (((uintptr_t)vy & 3) != 0) return LK_ERR_ARG;
    return LK_OK;
}
static int check_weight(int wtype, const void* vx) {
    if (!vx) return LK_ERR_ARG;
    if ((wtype == LK_TYPE_Q4_K || wtype == LK_TYPE_Q5_K) && ((uintptr_t)vx & 15) != 0) return LK_ERR_ARG;
    if (((uintptr_t)vx & 1) != 0) return LK_ERR_ARG;
    return LK_OK;
}

static int run_multi(int wtype, int count, const void* const* vx, const void* vy, void* const* dst, int dst_type,
                     int ncols_x, const int* nrows_x, int batch, int stride_col_y, int stride_col_dst,
                     const float* const* bias, void* stream, int act_stride_f32 = 0) {
    if (int rc = check_common(wtype, vy, ncols_x, batch, act_stride_f32 ? ncols_x / 32 : stride_col_y)) return rc;
    if (act_stride_f32 && (act_stride_f32 < ncols_x || act_stride_f32 % 4 != 0 || ((uintptr_t)vy & 15) != 0)) return LK_ERR_ARG;
    if (count < 1 || count > MAX_MULTI) return LK_ERR_ARG;
    MmvqCall a{};
    a.vy = (const uint8_t*)vy;
    a.nb = ncols_x / block_len_of(wtype);
    a.stride_col_y = stride_col_y;
    a.stride_col_dst = stride_col_dst;
    a.act_stride_f32 = act_stride_f32;
    a.stream = (hipStream_t)stream;
    int live = 0;
    for (int i = 0; i < count; ++i) {
        if (nrows_x[i] < 0) return LK_ERR_ARG;
        if (nrows_x[i] == 0) continue;
        if (int rc = check_weight(wtype, vx[i])) return rc;
        if (!dst[i] || stride_col_dst < nrows_x[i]) return LK_ERR_ARG;
        a.m.vx[live] = (const uint8_t*)vx[i];
        a.m.dst[live] = dst[i];
        a.m.bias[live] = bias ? bias[i] : nullptr;
        a.m.n[live] = nrows_x[i];
        ++live;
    }
    if (live == 0) return LK_OK;
    a.m.count = live;
    if (dst_type != LK_TYPE_F32 && dst_type != LK_TYPE_F16 && dst_type != LK_TYPE_BF16) return LK_ERR_TYPE;
    // A launch stages all its activation rows in LDS; a batch that does not fit (long rows) goes
    // out as several launches over equal shares of the rows.
    const int fit = lk_device().lds_bytes / lds_bytes_of(wtype, a.nb, 1);
    if (fit < 1) return LK_ERR_ARG;
    const int launches = (batch + fit - 1) / fit, share = (batch + launches - 1) / launches;
    const size_t dst_elem = dst_type == LK_TYPE_F32 ? 4 : 2;
    for (int b0 = 0; b0 < batch; b0 += share) {
        const int b = batch - b0 < share ? batch - b0 : share;
        MmvqCall c = a;
        c.vy = a.vy + (act_stride_f32 ? (size_t)b0 * act_stride_f32 * sizeof(float) : (size_t)b0 * stride_col_y * Q81_BYTES);
        for (int i = 0; i < live; ++i) c.m.dst[i] = (uint8_t*)a.m.dst[i] + (size_t)b0 * stride_col_dst * dst_elem;
        int rc;
        switch (dst_type) {
            case LK_TYPE_F32: rc = dispatch_plain<float>(wtype, b, c); break;
            case LK_TYPE_F16: rc = dispatch_plain<__half>(wtype, b, c); break;
            default: rc = dispatch_plain<__hip_bfloat16>(wtype, b, c); break;
        }
        if (rc != LK_OK) return rc;
    }
    return LK_OK;
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

}  // namespace

extern "C" int lk_mmvq(int wtype, const void* vx, const void* vy_q8_1, void* dst, int dst_type,
                       int ncols_x, int nrows_x, int batch, int stride_col_y, int stride_col_dst,
                       const float* bias, int decode_order, void* stream) {
    (void)decode_order;  // a row's sum never depends on batch here
    if (lk_is_legacy_type(wtype))   // Q4_0, Q4_1, Q5_0, Q5_1: the plain kernel of mmvq_legacy.hip
        return lk_mmvq_legacy(wtype, vx, vy_q8_1, dst, dst_type, ncols_x, nrows_x, batch, stride_col_y, stride_col_dst,
                              bias, (hipStream_t)stream);
    if (block_len_of(wtype) == 0) return LK_ERR_TYPE;
    if (nrows_x == 0) return LK_OK;
    return run_multi(wtype, 1, &vx, vy_q8_1, &dst, dst_type, ncols_x, &nrows_x, batch, stride_col_y, stride_col_dst,
                     bias ? &bias : nullptr, stream);
}

extern "C" int lk_mmvq_multi(int wtype, int count, const void* const* vx, const void* vy_q8_1, void* const* dst,
                             int dst_type, int ncols_x, const int* nrows_x, int batch, int stride_col_y,
                             int stride_col_dst, const float* const* bias, void* stream) {
    if (!vx || !dst || !nrows_x) return LK_ERR_ARG;
    return run_multi(wtype, count, vx, vy_q8_1, dst, dst_type, ncols_x, nrows_x, batch, stride_col_y, stride_col_dst,
                     bias, stream);
}

extern "C" int lk_mmvq_fused(int wtype, int count, const void* const* vx, const float* x, int stride_x,
                             void* const* dst, int dst_type, int ncols_x, const int* nrows_x, int batch,
                             int stride_col_dst, const float* const* bias, void* stream) {
    if (!vx || !dst || !nrows_x || stride_x <= 0) return LK_ERR_ARG;
    return run_multi(wtype, count, vx, x, dst, dst_type, ncols_x, nrows_x, batch, 0, stride_col_dst, bias, stream,
                     stride_x);
}

extern "C" int lk_mmvq_pair_act(int wtype, const void* gate, const void* up, const void* vy_q8_1, void* dst,
                                int dst_type, int ncols_x, int nrows_x, int batch, int stride_col_y,
                                int stride_col_dst, int act, void* stream) {
    if (int rc = check_common(wtype, vy_q8_1, ncols_x, batch, stride_col_y)) return rc;
    if (nrows_x == 0) return LK_OK;
    if (int rc = check_weight(wtype, gate)) return rc;
    if (int rc = check_weight(wtype, up)) return rc;
    if (!dst || nrows_x < 0 || stride_col_dst < nrows_x || (act != 0 && act != 1)) return LK_ERR_ARG;
    if (batch > 4) return LK_ERR_ARG;
    const int nb = ncols_x / block_len_of(wtype);
    if (dst_type != LK_TYPE_F32 && dst_type != LK_TYPE_BF16) return LK_ERR_TYPE;
    const int fit = lk_device().lds_bytes / lds_bytes_of(wtype, nb, 1);
    if (fit < 1) return LK_ERR_ARG;
    if (batch > fit) {   // rows too long to stage the whole batch: one launch per share of it
        for (int b0 = 0; b0 < batch; b0 += fit) {
            const int b = batch - b0 < fit ? batch - b0 : fit;
            const int rc = lk_mmvq_pair_act(wtype, gate, up, (const uint8_t*)vy_q8_1 + (size_t)b0 * stride_col_y * Q81_BYTES,
                                            (uint8_t*)dst + (size_t)b0 * stride_col_dst * (dst_type == LK_TYPE_F32 ? 4 : 2),
                                            dst_type, ncols_x, nrows_x, b, stride_col_y, stride_col_dst, act, stream);
            if (rc != LK_OK) return rc;
        }
        return LK_OK;
    }
    hipStream_t s = (hipStream_t)stream;
    const uint8_t *g = (const uint8_t*)gate, *u = (const uint8_t*)up, *y = (const uint8_t*)vy_q8_1;
#define LK_PAIR(E, T)                                                                                          \
    switch (batch) {                                                                                           \
        case 1: return launch_pair<E, 1, T>(g, u, y, dst, nb, nrows_x, stride_col_y, stride_col_dst, act, s);  \
        case 2: return launch_pair<E, 2, T>(g, u, y, dst, nb, nrows_x, stride_col_y, stride_col_dst, act, s);  \
        case 3: return launch_pair<E, 3, T>(g, u, y, dst, nb, nrows_x, stride_col_y, stride_col_dst, act, s);  \
        default: return launch_pair<E, 4, T>(g, u, y, dst, nb, nrows_x, stride_col_y, stride_col_dst, act, s); \
    }
#define LK_PAIR_TYPE(E)                                          \
    switch (dst_type) {                                          \
        case LK_TYPE_F32: LK_PAIR(E, float)                      \
        case LK_TYPE_BF16: LK_PAIR(E, __hip_bfloat16)            \
        default: return LK_ERR_TYPE;                             \
    }
    switch (wtype) {
        case LK_TYPE_Q4_K:
            if (nb <= 8) { LK_PAIR_TYPE(EngQ4KShort) }
            LK_PAIR_TYPE(EngQ4K)
        case LK_TYPE_Q5_K: LK_PAIR_TYPE(EngQ5K)
        case LK_TYPE_Q6_K: LK_PAIR_TYPE(EngQ6K)
        case LK_TYPE_Q8_0: LK_PAIR_TYPE(EngQ80)
        default: return LK_ERR_TYPE;
    }
}

extern "C" int lk_mmvq_pair_act_q8_1(int wtype, const void* gate, const void* up, const void* act, int act_is_f32,
                                     int stride_act, void* dst_q8_1, int stride_dst_blocks, int ncols_x, int nrows_x,
                                     int batch, int act_fn, void* stream) {
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (nrows_x == 0) return LK_OK;
    if (!act || !dst_q8_1 || ncols_x <= 0 || ncols_x % bl != 0 || nrows_x < 0 || nrows_x % 32 != 0) return LK_ERR_ARG;
    if (batch < 1 || batch > 4 || stride_dst_blocks < nrows_x / 32 || (act_fn != 0 && act_fn != 1)) return LK_ERR_ARG;
    if (((uintptr_t)dst_q8_1 & 3) != 0) return LK_ERR_ARG;
    if (act_is_f32 ? (stride_act < ncols_x || stride_act % 4 != 0 || ((uintptr_t)act & 15) != 0)
                   : (stride_act < ncols_x / 32 || ((uintptr_t)act & 3) != 0))
        return LK_ERR_ARG;
    if (int rc = check_weight(wtype, gate)) return rc;
    if (int rc = check_weight(wtype, up)) return rc;
    const int nb = ncols_x / bl;
    if (lds_bytes_of(wtype, nb, batch) + 2 * batch * 32 * (int)sizeof(float) > lk_device().lds_bytes) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const uint8_t *g = (const uint8_t*)gate, *u = (const uint8_t*)up, *y = (const uint8_t*)act;
    const int sy = act_is_f32 ? 0 : stride_act, sf = act_is_f32 ? stride_act : 0;
#define LK_PAIR_Q(E)                                                                                        \
    switch (batch) {                                                                                        \
        case 1: return launch_pair_q8_1<E, 1>(g, u, y, dst_q8_1, nb, nrows_x, sy, stride_dst_blocks, sf, act_fn, s);  \
        case 2: return launch_pair_q8_1<E, 2>(g, u, y, dst_q8_1, nb, nrows_x, sy, stride_dst_blocks, sf, act_fn, s);  \
        case 3: return launch_pair_q8_1<E, 3>(g, u, y, dst_q8_1, nb, nrows_x, sy, stride_dst_blocks, sf, act_fn, s);  \
        default: return launch_pair_q8_1<E, 4>(g, u, y, dst_q8_1, nb, nrows_x, sy, stride_dst_blocks, sf, act_fn, s); \
    }
    switch (wtype) {
        case LK_TYPE_Q4_K: LK_PAIR_Q(EngQ4K)
        case LK_TYPE_Q5_K: LK_PAIR_Q(EngQ5K)
        case LK_TYPE_Q6_K: LK_PAIR_Q(EngQ6K)
        case LK_TYPE_Q8_0: LK_PAIR_Q(EngQ80)
        default: return LK_ERR_TYPE;
    }
}

extern "C" int lk_mmvq_grouped(int wtype, const uint64_t* table, int groups, const void* vy_q8_1, float* dst,
                               int ncols_x, int nrows_x, void* stream) {
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (groups == 0 || nrows_x == 0) return LK_OK;
    if (!table || !vy_q8_1 || !dst || groups < 0 || groups > 65535 || nrows_x < 0 || ncols_x <= 0) return LK_ERR_ARG;
    if (ncols_x % LK_ROW_PADDING != 0 || ncols_x % bl != 0 || ((uintptr_t)vy_q8_1 & 3) != 0) return LK_ERR_ARG;
    const int nb = ncols_x / bl, k32 = ncols_x / 32;
    hipStream_t s = (hipStream_t)stream;
    const uint8_t* y = (const uint8_t*)vy_q8_1;
    switch (wtype) {
        case LK_TYPE_Q4_K:
            return nb <= 8 ? launch_grouped<EngQ4KShort>(table, groups, y, dst, nb, nrows_x, k32, s)
                           : launch_grouped<EngQ4K>(table, groups, y, dst, nb, nrows_x, k32, s);
        case LK_TYPE_Q5_K: return launch_grouped<EngQ5K>(table, groups, y, dst, nb, nrows_x, k32, s);
        case LK_TYPE_Q6_K: return launch_grouped<EngQ6K>(table, groups, y, dst, nb, nrows_x, k32, s);
        default: return launch_grouped<EngQ80>(table, groups, y, dst, nb, nrows_x, k32, s);
    }
}

extern "C" int lk_mmvq_subdots(int wtype, const void* vx, const void* vy_q8_1, int32_t* dots,
                               int32_t* sums, int ncols_x, int nrows_x, void* stream) {
    if (lk_is_legacy_type(wtype)) {
        if (int rc = lk_mmvq_subdots_legacy(wtype, vx, vy_q8_1, dots, ncols_x, nrows_x, (hipStream_t)stream)) return rc;
        if (sums) {
            const int k32 = ncols_x / 32;
            hipLaunchKernelGGL(act_sums_kernel, dim3((k32 + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                               (const uint8_t*)vy_q8_1, sums, k32);
        }
        return lk_launch_status();
    }
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (!vx || !vy_q8_1 || !dots || ncols_x <= 0 || nrows_x <= 0 || ncols_x % bl != 0) return LK_ERR_ARG;
    if (nrows_x > 65535) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int nb = ncols_x / bl;
    const uint8_t* w = (const uint8_t*)vx;
    const uint8_t* y = (const uint8_t*)vy_q8_1;
    if (wtype == LK_TYPE_Q4_K) {
        hipLaunchKernelGGL(subdots_q4k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else if (wtype == LK_TYPE_Q5_K) {
        hipLaunchKernelGGL(subdots_q5k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else if (wtype == LK_TYPE_Q6_K) {
        hipLaunchKernelGGL(subdots_q6k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else {
        hipLaunchKernelGGL(subdots_q80_kernel, dim3((nb + 31) / 32, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    }
    if (sums) {
        const int k32 = ncols_x / 32;
        hipLaunchKernelGGL(act_sums_kernel, dim3((k32 + 255) / 256), dim3(256), 0, s, y, sums, k32);
    }
    return lk_launch_status();
}

// Shared device helpers for the gfx950 quantized-matmul kernels. wave64 only.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stdlib.h>

#include "../../include/loken_gfx950.h"

#define LK_WAVE 64

// GGUF block geometry (src/tensor/quantized/dtype.rs:66-96 of the reference).
#define Q4K_BYTES 144
#define Q5K_BYTES 176
#define Q6K_BYTES 210
#define Q80_BYTES 34
#define Q81_BYTES 36

// 16-byte loads from blocks that are only 2-byte aligned (Q6_K 210 B, Q8_0 34 B): global memory
// on gfx950 serves unaligned dwordx4, the type only tells the compiler not to assume more.
typedef uint4 __attribute__((aligned(2))) uint4_a2;
typedef uint4 __attribute__((aligned(4))) uint4_a4;
typedef uint2 __attribute__((aligned(2))) uint2_a2;
typedef uint4 __attribute__((aligned(4))) uint4_a4;
typedef uint32_t __attribute__((aligned(2))) uint32_a2;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// A byte address typed as global memory. Weight addresses travel in this type: one rebuilt from
// integers, read from a table or passed through an opaque statement is otherwise a generic
// pointer and is read with flat loads, which also count against the LDS wait counter.
typedef const __attribute__((address_space(1))) uint8_t* gbytes_t;
static __device__ __forceinline__ gbytes_t to_gbytes(const void* p) { return (gbytes_t)p; }
static __device__ __forceinline__ gbytes_t to_gbytes(uint64_t bits) { return (gbytes_t)bits; }

static __device__ __forceinline__ int dot4(int a, int b, int c) {
    return __builtin_amdgcn_sdot4(a, b, c, false);
}

static __device__ __forceinline__ int dot16(const uint4& w, const uint4& a, int c) {
    c = dot4((int)w.x, (int)a.x, c);
    c = dot4((int)w.y, (int)a.y, c);
    c = dot4((int)w.z, (int)a.z, c);
    return dot4((int)w.w, (int)a.w, c);
}

static __device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short)h));
}

template <int ctrl>
static __device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xF, 0xF, true));
}

template <int ctrl>
static __device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, ctrl, 0xF, 0xF, true);
}

// Sum over the 64 lanes of a wave; every lane returns the total. Lane exchanges inside a row of
// 16 are DPP moves; the four row totals cross through scalar registers (an LDS-crossbar
// permute costs two orders of magnitude more latency than either).
static __device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    const int bits = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(bits, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(bits, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
    return (r0 + r1) + (r2 + r3);
}

// The sum over each aligned group of LANES (16, 32 or 64) lanes, every lane of the group returns
// it. Same order of additions as wave_sum: pairs, quads, the two quads of a half row, the two half
// rows, then rows 0+1 and 2+3, then the two halves of the wave. The rows cross through the two
// row-swap instructions (v_permlane16_swap, v_permlane32_swap), which stay in the vector unit.
static __device__ __forceinline__ float swap_add16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
static __device__ __forceinline__ float swap_add32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <int LANES>
static __device__ __forceinline__ float group_sum(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    if (LANES >= 32) v = swap_add16(v);
    if (LANES >= 64) v = swap_add32(v);
    return v;
}
// The maximum over each aligned group of 32 lanes (every lane of the group returns it).
static __device__ __forceinline__ float group_max32(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// Thirty-two f32 values, one per lane of an aligned group of 32, as one Q8_1 block at `out` (36 bytes, 4-byte
// aligned): the stand-alone quantizer's steps, as lk_store_q8_1_block. `l32`: the lane's place in the group.
// Every lane of the wave calls it (the lane exchanges want them all); `store` false: nothing is written.
static __device__ __forceinline__ void lk_store_q8_1_block_by_lane(float x, int l32, uint8_t* out, bool store) {
#pragma clang fp contract(off)
    const float amax = group_max32(fabsf(x));
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const int q = (int)roundf(x * inv);
    const float sum = group_sum<32>((float)q);   // an integer below 2^12: exact whatever the order
    if (store) out[4 + l32] = (uint8_t)(q & 0xFF);
    if (store && l32 == 0) {
        const uint32_t dh = __half_as_ushort(__float2half_rn(d));
        float scaled_sum = sum * d;
        asm volatile("" : "+v"(scaled_sum));   // two roundings, as the quantizer's
        *(uint32_t*)out = dh | ((uint32_t)__half_as_ushort(__float2half_rn(scaled_sum)) << 16);
    }
}

// Two values at once: the even lanes of a group return the group's sum of `x0`, the odd lanes that
// of `x1`, each with the additions of group_sum in the same order as far as lanes 0 and 1 of the
// group are concerned, the only lanes whose result is defined (the first step hands every lane its
// neighbour's value of the row it keeps, the later steps move by even distances only: shifts by 4
// and 8 inside a row of 16, so lane 0 adds (Q0 + Q1) + (Q2 + Q3) over the row's quads as
// group_sum's mirrors do).
template <int LANES>
static __device__ __forceinline__ float group_sum2(float x0, float x1, bool odd) {
    const float keep = odd ? x1 : x0, send = odd ? x0 : x1;
    float v = keep + dpp_f32<0xB1>(send);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x104>(v);   // row_shl:4: lane i takes lane i + 4 (the next quad; nothing past the row)
    v += dpp_f32<0x108>(v);   // row_shl:8
    if (LANES >= 32) v = swap_add16(v);
    if (LANES >= 64) v = swap_add32(v);
    return v;
}

// Maximum / sum over each aligned group of 8 lanes; every lane of the group returns it.
// `quad` receives the value after the first two steps (the lane's group of 4).
static __device__ __forceinline__ float max8(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    return fmaxf(v, dpp_f32<0x141>(v));   // quads are uniform by now, so the mirror is "the other quad"
}
static __device__ __forceinline__ int sum8(int v, int& quad) {
    v += dpp_i32<0xB1>(v);
    v += dpp_i32<0x4E>(v);
    quad = v;
    return v + dpp_i32<0x141>(v);
}

// Thirty-two f32 values as one Q8_1 block, by the eight lanes of an aligned group (lane l8 brings values
// 4 l8 .. 4 l8 + 3): the steps of the stand-alone quantizer (d = amax / 127, stored as f16; codes =
// round-half-away(x * (1 / d)) with d before its rounding; s = f16(f32(sum of codes * d))), so the bytes
// are those lk_quantize_q8_1 writes. `out`: the block's nine words.
static __device__ __forceinline__ void lk_store_q8_1_block(float4 v, int l8, uint32_t* out) {
#pragma clang fp contract(off)
    const float amax = max8(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const int q0 = (int)roundf(v.x * inv), q1 = (int)roundf(v.y * inv);
    const int q2 = (int)roundf(v.z * inv), q3 = (int)roundf(v.w * inv);
    int quad;
    const int sum = sum8(q0 + q1 + q2 + q3, quad);
    out[1 + l8] = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
                  ((uint32_t)(q3 & 0xFF) << 24);
    if (l8 == 0) {
        const uint32_t dh = __half_as_ushort(__float2half_rn(d));
        float scaled_sum = (float)sum * d;
        asm volatile("" : "+v"(scaled_sum));   // two roundings, as the quantizer's
        out[0] = dh | ((uint32_t)__half_as_ushort(__float2half_rn(scaled_sum)) << 16);
    }
}

static __device__ __forceinline__ int wave_sum_i32(int v) {
    for (int o = 1; o < 64; o <<= 1) v += __shfl_xor(v, o);
    return v;
}

// Dword-aligned read of 16 bytes that start on any even address. A 2-byte-aligned dwordx4 load
// runs at about three quarters of the rate of a dword-aligned one on this part, so the load is
// made from the enclosing dwords and shifted into place. The fifth dword is the one that holds
// the run's last two bytes (the run's own last dword when the address is already aligned), so
// nothing outside dwords the run touches is read.
struct Run16 {
    uint4 w;
    uint32_t e;
};
static __device__ __forceinline__ Run16 load_run16(const uint8_t* p) {
    const uintptr_t a = (uintptr_t)p;
    const uint8_t* b = (const uint8_t*)(a & ~(uintptr_t)3);
    Run16 r;
    r.w = *(const uint4_a4*)b;
    r.e = *(const uint32_t*)(b + 12 + 2 * (a & 2));
    return r;
}
static __device__ __forceinline__ uint4 run16_value(const Run16& r, uint32_t shift_bits) {
    uint4 v;
    v.x = __builtin_amdgcn_alignbit(r.w.y, r.w.x, shift_bits);
    v.y = __builtin_amdgcn_alignbit(r.w.z, r.w.y, shift_bits);
    v.z = __builtin_amdgcn_alignbit(r.w.w, r.w.z, shift_bits);
    v.w = __builtin_amdgcn_alignbit(r.e, r.w.w, shift_bits);
    return v;
}

// Output element conversion.
template <typename T> static __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f32<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __hip_bfloat16 from_f32<__hip_bfloat16>(float v) { return __float2bfloat16(v); }

template <typename T> static __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }
template <> __device__ __forceinline__ float to_f32<__hip_bfloat16>(__hip_bfloat16 v) { return __bfloat162float(v); }

// Host side: device facts fetched once.
struct LkDevice {
    int cus;
    int lds_bytes;
};
const LkDevice& lk_device();

// Q4_K x up to any number of Q8_1 rows on the matrix unit (rows_mfma.hip); LK_* status.
int lk_q4k_rows_mfma(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k, int stride_y,
                     int ldd, hipStream_t stream);

// Q4_K x one or two activation rows with the rows' codes held in registers (mmvq_reg.hip): weight rows of
// at most 16 super-blocks. Up to four matrices over the activation; `act_f32` non-zero: `act` holds f32
// rows, quantized by every workgroup itself. `batch` rows, act_stride Q8_1 blocks (floats) apart, their
// outputs dst_stride elements apart. LK_* status.
#define LK_REG_MAX_BATCH 2
struct LkRegMulti {
    const uint8_t* vx[4];
    void* dst[4];
    const float* bias[4];
    int n[4];
    int count;
};
bool lk_q4k_reg_serves(int nb);
int lk_q4k_reg_multi(const LkRegMulti& m, const void* act, int act_f32, int nb, int dst_type, int batch, int act_stride,
                     int dst_stride, hipStream_t stream);
// The gate/up pair over the activation rows: dst = act(gate . x) * (up . x) as f32 / bf16 (`dst_q8_1`
// false; rows dst_stride elements apart) or as Q8_1 blocks of 32 consecutive rows (true; n a multiple of
// 32; rows dst_stride blocks apart).
int lk_q4k_reg_pair(const uint8_t* gate, const uint8_t* up, const void* act, int act_f32, void* dst, int dst_type,
                    bool dst_q8_1, int nb, int n, int act_fn, int batch, int act_stride, int dst_stride, hipStream_t stream);

// The 32-value nibble formats (mmvq_legacy.hip); status LK_*.
bool lk_is_legacy_type(int wtype);
int lk_mmvq_legacy(int wtype, const void* vx, const void* vy_q8_1, void* dst, int dst_type, int ncols_x, int nrows_x,
                   int batch, int stride_col_y, int stride_col_dst, const float* bias, hipStream_t stream);
int lk_mmvq_subdots_legacy(int wtype, const void* vx, const void* vy_q8_1, int32_t* dots, int ncols_x, int nrows_x,
                           hipStream_t stream);
// What the gated MoE decode launch makes of a row's gate product g and up product u
// (cuda/moe/moe_gguf.cu:994-1003, 1178-1184, 1280-1289 of the reference):
//   SILU      g / (1 + exp(-g)) * u
//   OAI       g += gate_bias, u += up_bias (per expert, nullable); x = min(g, limit); u' = clamp(u, +-limit);
//             x * sigmoid(alpha x) * (1 + u')
//   LIMITED   g = min(g, limit), u = clamp(u, +-limit); g / (1 + exp(-g)) * u
//   GELU      0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * u
enum { LK_GATE_SILU = 0, LK_GATE_OAI = 1, LK_GATE_LIMITED = 2, LK_GATE_GELU = 3 };
struct LkGateAct {
    int kind = LK_GATE_SILU;
    float alpha = 0.f, limit = 0.f;
    const float* gate_bias = nullptr;
    const float* up_bias = nullptr;
};
static __device__ __forceinline__ float lk_gated(const LkGateAct& a, float g, float u, size_t bias_at) {
    switch (a.kind) {
        case LK_GATE_OAI: {
            if (a.gate_bias) g += a.gate_bias[bias_at];
            if (a.up_bias) u += a.up_bias[bias_at];
            const float x = fminf(g, a.limit);
            const float uc = fminf(fmaxf(u, -a.limit), a.limit);
            return (x * (1.0f / (1.0f + expf(-a.alpha * x)))) * (1.0f + uc);
        }
        case LK_GATE_LIMITED: {
            g = fminf(g, a.limit);
            u = fminf(fmaxf(u, -a.limit), a.limit);
            return g / (1.0f + expf(-g)) * u;
        }
        case LK_GATE_GELU:
            return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * (g * g * g)))) * u;
        default:
            return g / (1.0f + expf(-g)) * u;
    }
}

// A layer's experts over two tensors (cuda/moe/moe_gguf.cu:239-257 of the reference): the slots from
// `alt_from` on are slot (expert - alt_from) of the second tensor; `alt_at`, when given, is a pair of
// addresses on the card read when the kernel runs (gate / down at [0], up at [1]).
struct LkMoeAlt {
    const uint8_t* alt0 = nullptr;
    const uint8_t* alt1 = nullptr;
    int alt_from = 0;
    const void* const* alt_at = nullptr;
};
static __device__ __forceinline__ const uint8_t* lk_expert_slab(const uint8_t* base, int which, const LkMoeAlt& alt, int e,
                                                                int64_t slab_bytes) {
    const uint8_t* second = alt.alt_at ? (const uint8_t*)alt.alt_at[which] : (which ? alt.alt1 : alt.alt0);
    if (second != nullptr && e >= alt.alt_from) return second + (int64_t)(e - alt.alt_from) * slab_bytes;
    return base + (int64_t)e * slab_bytes;
}

// The Q4_K gate / up pair per routed pair of an MoE layer with the activation row's codes in
// registers (mmvq_reg.hip): f32 activation rows `acts` [tokens][256 nb], output rows in slot order.
// -1: not served (rows longer than 16 super-blocks, more than 65535 pairs, misaligned), else LK_*.
int lk_q4k_reg_moe_pair(const uint8_t* gate, const uint8_t* up, const float* acts, const int32_t* sorted_token_ids,
                        const int32_t* expert_ids, float* out, int experts, int topk, int pairs, int n, int nb,
                        int64_t slab_bytes, const LkGateAct& act, hipStream_t stream);

// MoE decode for the expert formats the K-quant engines do not serve (mmvq_legacy.hip): block length
// of a wire id (0: not one of them), and the per-pair launch over Q8_1 activation rows. An expert's
// slab is `slab_rows` weight rows (cols, or twice that where gate and up share a tensor); with `live`
// only the first *live pairs run (the count is read on the card).
int lk_moe_wire_block_len_legacy(int quant_type);
int lk_moe_rows_legacy(int mode, int quant_type, const uint8_t* w0, const uint8_t* w1, const uint8_t* acts_q8_1,
                       const int32_t* sorted_token_ids, const int32_t* expert_ids, const float* topk_weights,
                       const float* down_bias, float* out, int experts, int topk, int pairs, int cols, int size_k,
                       int k32_stride, const LkGateAct& act, int slab_rows, const unsigned int* live,
                       const LkMoeAlt& alt, hipStream_t s);

// Measurement runs and A/B tests: an integer from the environment (0 when unset). Every LK_TUNE_* /
// LK_MMQ_* variable only overrides a launch-shape or path choice; none changes what a result means.
// A call site reads the environment once and keeps the value: the launch path pays one relaxed load
// and a compare. lk_tune_refresh() (device.hip) makes every site read again, for a process that
// changes its environment while it runs.
struct LkTuneSite {
    const char* name;
    unsigned epoch;   // the refresh count this value was read at (0: never)
    int value;
};
unsigned lk_tune_epoch();
int lk_tune_read(LkTuneSite& site);
#define lk_tune_env(NAME)                                                        \
    ([]() -> int {                                                               \
        static LkTuneSite site{NAME, 0u, 0};                                     \
        return site.epoch == lk_tune_epoch() ? site.value : lk_tune_read(site);  \
    }())
static inline bool lk_env_flag_site(int v) { return v != 0; }
#define lk_env_flag(NAME) lk_env_flag_site(lk_tune_env(NAME))

static inline int lk_launch_status() {
    return hipGetLastError() == hipSuccess ? LK_OK : LK_ERR_LAUNCH;
}

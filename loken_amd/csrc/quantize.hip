// Activation rows -> Q8_1 blocks of 32 (the decode-path quantizer).
//
// Statement followed: loken's BlockQ8_1::quantize (src/tensor/quant_cpu/format/q8_1.rs:46-61):
// d = amax / 127 (f32, true division), stored as f16; inv = d != 0 ? 1/d : 0; codes =
// round-half-away(x * inv); s = f16(sum(codes) * d) with d BEFORE its f16 rounding. The sum is
// an integer sum, so it does not depend on reduction order (the reference's GPU quantizer sums
// the float inputs instead, cuda/moe/gguf.cuh:1125-1153; no kernel here reads s).
//
// Layout: one lane owns four consecutive values (one 16-byte load, one 4-byte store), eight
// lanes own a block, a 256-lane workgroup covers 1024 values of one row.

#include "lk_common.h"

// Every float step below is one IEEE operation in the reference, so none may be fused here:
// with contraction on, f16(sum * d) becomes a single-rounding mixed-precision multiply and the
// `s` field drifts by an ulp from the host quantizer's double rounding.
#pragma clang fp contract(off)

namespace {

template <typename T> struct Load4;
template <> struct Load4<float> {
    static __device__ __forceinline__ float4 at(const float* p) { return *(const float4*)p; }
};
template <> struct Load4<__half> {
    static __device__ __forceinline__ float4 at(const __half* p) {
        const uint2 raw = *(const uint2*)p;
        const __half2 a = *(const __half2*)&raw.x, b = *(const __half2*)&raw.y;
        return make_float4(__low2float(a), __high2float(a), __low2float(b), __high2float(b));
    }
};
template <> struct Load4<__hip_bfloat16> {
    static __device__ __forceinline__ float4 at(const __hip_bfloat16* p) {
        const uint2 raw = *(const uint2*)p;
        return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xFFFF0000u),
                           __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xFFFF0000u));
    }
};

static __device__ __forceinline__ int round_code(float v) {
    // roundf is half away from zero, as f32::round.
    return (int)roundf(v);
}

template <typename T>
__global__ __launch_bounds__(256) void quantize_q8_1_kernel(const T* __restrict__ x,
                                                            uint32_t* __restrict__ vy, int kx,
                                                            int kx_padded, int vec_ok) {
    const int row = blockIdx.y;
    const int i0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i0 >= kx_padded) return;  // whole groups of 8 lanes leave together: kx_padded % 32 == 0

    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    const T* xr = x + (size_t)row * kx;
    if (vec_ok && i0 + 3 < kx) {
        v = Load4<T>::at(xr + i0);
    } else {
        if (i0 + 0 < kx) v.x = to_f32<T>(xr[i0 + 0]);
        if (i0 + 1 < kx) v.y = to_f32<T>(xr[i0 + 1]);
        if (i0 + 2 < kx) v.z = to_f32<T>(xr[i0 + 2]);
        if (i0 + 3 < kx) v.w = to_f32<T>(xr[i0 + 3]);
    }

    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = max8(amax);

    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const int q0 = round_code(v.x * inv), q1 = round_code(v.y * inv);
    const int q2 = round_code(v.z * inv), q3 = round_code(v.w * inv);

    int quad_sum;
    const int sum = sum8(q0 + q1 + q2 + q3, quad_sum);

    const size_t block = (size_t)row * (kx_padded / 32) + i0 / 32;
    uint32_t* out = vy + block * 9;  // 36 bytes = 9 words
    const int lane8 = (i0 / 4) & 7;
    out[1 + lane8] = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) |
                     ((uint32_t)(q2 & 0xFF) << 16) | ((uint32_t)(q3 & 0xFF) << 24);
    if (lane8 == 0) {
        const uint32_t dh = __half_as_ushort(__float2half_rn(d));
        // The product must round to f32 before it rounds to f16 (two roundings, as on the host);
        // the empty asm keeps instruction selection from folding both into one v_fma_mixlo_f16.
        float scaled_sum = (float)sum * d;
        asm volatile("" : "+v"(scaled_sum));
        const uint32_t sh = __half_as_ushort(__float2half_rn(scaled_sum));
        out[0] = dh | (sh << 16);
    }
}

}  // namespace

extern "C" int lk_quantize_q8_1(const void* x, int x_type, void* vy, int kx, int kx_padded,
                                int rows, void* stream) {
    if (rows == 0) return LK_OK;
    if (!x || !vy || kx <= 0 || rows < 0 || kx_padded < kx || kx_padded % 32 != 0) return LK_ERR_ARG;
    if (((uintptr_t)vy & 3) != 0) return LK_ERR_ARG;
    const dim3 grid((kx_padded + 1023) / 1024, rows, 1);
    if (grid.y > 65535u) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    // Four-value vector loads need every row to start on a 4-element boundary.
    const auto vec_ok = [&](size_t elem) { return (int)(((uintptr_t)x % (4 * elem)) == 0 && kx % 4 == 0); };
    switch (x_type) {
        case LK_TYPE_F32:
            if ((uintptr_t)x % 4 != 0) return LK_ERR_ARG;
            hipLaunchKernelGGL(quantize_q8_1_kernel<float>, grid, dim3(256), 0, s, (const float*)x,
                               (uint32_t*)vy, kx, kx_padded, vec_ok(4));
            break;
        case LK_TYPE_F16:
            if ((uintptr_t)x % 2 != 0) return LK_ERR_ARG;
            hipLaunchKernelGGL(quantize_q8_1_kernel<__half>, grid, dim3(256), 0, s,
                               (const __half*)x, (uint32_t*)vy, kx, kx_padded, vec_ok(2));
            break;
        case LK_TYPE_BF16:
            if ((uintptr_t)x % 2 != 0) return LK_ERR_ARG;
            hipLaunchKernelGGL(quantize_q8_1_kernel<__hip_bfloat16>, grid, dim3(256), 0, s,
                               (const __hip_bfloat16*)x, (uint32_t*)vy, kx, kx_padded, vec_ok(2));
            break;
        default:
            return LK_ERR_TYPE;
    }
    return lk_launch_status();
}

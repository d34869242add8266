// The exact mode: Q4_K / Q6_K weight rows against Q8_K activation rows with the reference's own
// cross-device contract (BlockFormat / ExactDot, src/tensor/quant_cpu/format/blocks.rs:80-96;
// dot_exact, format/q4_k.rs:117-156, format/q6_k.rs:121-163): per super-block the integer sums are exact
// in any order, and the f32 fold is fixed,
//     Q4_K   total += d8 * (d * f32(sum_s sc_s * dot_s) - dmin * f32(sum_s m_s * bsum_s))
//     Q6_K   total += d8 * (d * f32(sum_j scale_j * dot_j))
// from -0.0, one rounding per written operation, blocks in order. A device that keeps to it returns the
// bits of the CPU's dot_exact. This kernel does: it exists for that comparison, not for speed. (The fast
// kernels' contract is the bit-exact integers plus the f32 tolerance.)
//
// A wave owns a weight row and an activation row; lane l takes super-blocks l, l + 64, ... whole (its
// integers need no exchange), forms the block's f32 term with contraction off, and the terms are added
// by one lane in block order.

#include "lk_common.h"

namespace {

constexpr int Q8K_BYTES = 292;   // f32 d, 256 x i8, 16 x i16 sums of 16 (format/q8_k.rs:20)

static __device__ __forceinline__ float f32_at(const uint8_t* p) { return __uint_as_float(*(const uint32_t*)p); }
static __device__ __forceinline__ int i16_at(const uint8_t* p) { return (int)(int16_t)(p[0] | (p[1] << 8)); }

// get_scale_min_k4 of the format (blocks.rs:146-165): the eight six-bit (scale, min) pairs of the 12 packed bytes.
static __device__ __forceinline__ void unpack_scales_mins(const uint8_t* packed, int (&sc)[8], int (&mn)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        sc[i] = packed[i] & 0x3F;
        mn[i] = packed[i + 4] & 0x3F;
    }
#pragma unroll
    for (int i = 4; i < 8; ++i) {
        const int low = packed[i + 4];
        sc[i] = (low & 0x0F) | ((packed[i - 4] >> 6) << 4);
        mn[i] = (low >> 4) | ((packed[i] >> 6) << 4);
    }
}

// One super-block's term. x: the weight block, y: the Q8_K block.
static __device__ __forceinline__ float term_q4k(const uint8_t* x, const uint8_t* y) {
#pragma clang fp contract(off)
    int sc[8], mn[8];
    unpack_scales_mins(x + 4, sc, mn);
    const int8_t* yq = (const int8_t*)(y + 4);
    int scaled = 0, offset = 0;
    for (int s = 0; s < 8; ++s) {
        const uint8_t* group = x + 16 + (s >> 1) * 32;
        const int shift = (s & 1) ? 4 : 0;
        int dot = 0;
        for (int l = 0; l < 32; ++l) dot += (int)((group[l] >> shift) & 0x0F) * (int)yq[32 * s + l];
        scaled += sc[s] * dot;
        offset += mn[s] * (i16_at(y + 260 + 4 * s) + i16_at(y + 260 + 4 * s + 2));
    }
    const float d = f16_bits_to_f32(x[0] | (x[1] << 8)), dmin = f16_bits_to_f32(x[2] | (x[3] << 8));
    const float a = d * (float)scaled;
    const float b = dmin * (float)offset;
    const float diff = a - b;
    return f32_at(y) * diff;
}

static __device__ __forceinline__ float term_q6k(const uint8_t* x, const uint8_t* y) {
#pragma clang fp contract(off)
    const int8_t* yq = (const int8_t*)(y + 4);
    const int8_t* scales = (const int8_t*)(x + 192);
    int scaled = 0;
    for (int h = 0; h < 2; ++h)
        for (int g = 0; g < 4; ++g)
            for (int half = 0; half < 2; ++half) {   // the group's two runs of sixteen, each with its own scale
                int dot = 0;
                for (int l = 16 * half; l < 16 * half + 16; ++l) {
                    const int low = (x[64 * h + 32 * (g & 1) + l] >> (g < 2 ? 0 : 4)) & 0x0F;
                    const int high = (x[128 + 32 * h + l] >> (2 * g)) & 0x03;
                    dot += ((low | (high << 4)) - 32) * (int)yq[128 * h + 32 * g + l];
                }
                scaled += (int)scales[8 * h + 2 * g + half] * dot;
            }
    const float d = f16_bits_to_f32(x[208] | (x[209] << 8));
    const float a = d * (float)scaled;
    return f32_at(y) * a;
}

template <bool Q6>
__global__ __launch_bounds__(256) void mmvq_exact_kernel(const uint8_t* __restrict__ vx, const uint8_t* __restrict__ vy,
                                                         float* __restrict__ dst, int nb, int nrows_x, int batch) {
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), col = blockIdx.y;
    if (row >= nrows_x) return;   // (whole waves)
    const uint8_t* x = vx + (size_t)row * nb * (Q6 ? Q6K_BYTES : Q4K_BYTES);
    const uint8_t* y = vy + (size_t)col * nb * Q8K_BYTES;
    float total = -0.0f;
    for (int b0 = 0; b0 < nb; b0 += 64) {
        const int b = b0 + lane;
        float term = 0.f;
        if (b < nb) term = Q6 ? term_q6k(x + (size_t)b * Q6K_BYTES, y + (size_t)b * Q8K_BYTES)
                              : term_q4k(x + (size_t)b * Q4K_BYTES, y + (size_t)b * Q8K_BYTES);
        // the fold, in block order (every lane runs it on the same values)
        const int live = min(64, nb - b0);
        for (int i = 0; i < live; ++i) total += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(term), i));
    }
    if (lane == 0) dst[(size_t)col * nrows_x + row] = total;
}

}  // namespace

extern "C" int lk_mmvq_exact(int wtype, const void* vx, const void* vy_q8_k, float* dst, int ncols_x, int nrows_x, int batch,
                             void* stream) {
    if (wtype != LK_TYPE_Q4_K && wtype != LK_TYPE_Q6_K) return LK_ERR_TYPE;
    if (nrows_x == 0 || batch == 0) return LK_OK;
    if (!vx || !vy_q8_k || !dst || ncols_x <= 0 || ncols_x % 256 != 0 || nrows_x < 0 || batch < 0 || batch > 65535 ||
        (((uintptr_t)vy_q8_k) & 3) != 0)
        return LK_ERR_ARG;
    const dim3 grid((nrows_x + 3) / 4, batch);
    if (wtype == LK_TYPE_Q6_K)
        hipLaunchKernelGGL(mmvq_exact_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)vx,
                           (const uint8_t*)vy_q8_k, dst, ncols_x / 256, nrows_x, batch);
    else
        hipLaunchKernelGGL(mmvq_exact_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)vx,
                           (const uint8_t*)vy_q8_k, dst, ncols_x / 256, nrows_x, batch);
    return lk_launch_status();
}

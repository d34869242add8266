// Decode-step producers that end in the activation a mat-vec reads: RMSNorm (plain, after a
// residual add, and the post-attention norm + add + feed-forward norm chain) and the gate/up
// split activation, each writing its f32 row as before AND the same row as Q8_1 blocks, so the
// mat-vec that follows needs no quantizer launch.
//
// Statements followed (src/inference/cuda/mmvq_gguf.cu): rmsnorm_wide_q8_1_f32 (:805-837),
// add_rmsnorm_dual_wide_q8_1_f32 (:839-877), post_norm_add_norm_wide_q8_1_f32 (:879-936),
// split_silu_mul_q8_1_f32 / split_gelu_mul_q8_1_f32 (:971-999), quantize_lane_to_q8_1 (:789-801).
// Kept from them: lane t of 256 accumulates the squares of values t, t + 256, ... in that order
// (fused multiply-add, as the reference's build contracts `sum += v * v`), the 256 partial sums
// fold as a stride-halving tree (t with t + 128, then + 64, ... + 1), each value is
// (x * rms) * weight, every product of the chain kernel is rounded before it is added, and the
// quantized value is the f32 value that was stored. Different on purpose: rms = 1 / sqrt(mean + eps)
// with both operations correctly rounded (the reference's rsqrtf is an approximation whose bits
// depend on the card), and the Q8_1 block follows lk_quantize_q8_1's rule (s = f16(sum of codes *
// d)), so the blocks are byte for byte what lk_quantize_q8_1 makes of the f32 row.
//
// One workgroup of 256 lanes per row; a row is `cols` values, a multiple of 512 (the quantized
// row has no padding). The row sits in LDS between the passes. Lane t owns values t + 256 j
// throughout, so a Q8_1 block is 32 consecutive lanes: half a wave.

#include "lk_common.h"

#pragma clang fp contract(off)

namespace {

constexpr int NORM_WG = 256;

// Sum over each aligned group of 32 lanes (half a wave); every lane returns its group's total.
template <typename T, class Op>
static __device__ __forceinline__ T fold32(T v, Op op) {
#pragma unroll
    for (int o = 1; o < 32; o <<= 1) v = op(v, __shfl_xor(v, o));
    return v;
}

// The value a lane holds, into its Q8_1 block: 32 consecutive lanes own one block.
static __device__ __forceinline__ void quantize_lane(uint8_t* __restrict__ row_blocks, int i, float v) {
    const float amax = fold32(fabsf(v), [](float a, float b) { return fmaxf(a, b); });
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const int q = (int)roundf(v * inv);
    const int sum = fold32(q, [](int a, int b) { return a + b; });
    uint8_t* block = row_blocks + (size_t)(i / 32) * Q81_BYTES;
    block[4 + (i & 31)] = (uint8_t)(int8_t)q;
    if ((i & 31) == 0) {
        const uint32_t dh = __half_as_ushort(__float2half_rn(d));
        // two roundings (f32 product, then f16), as on the host: the empty asm keeps instruction
        // selection from folding both into one mixed-precision multiply
        float scaled_sum = (float)sum * d;
        asm volatile("" : "+v"(scaled_sum));
        const uint32_t sh = __half_as_ushort(__float2half_rn(scaled_sum));
        *(uint32_t*)block = dh | (sh << 16);
    }
}

// 1 / sqrt(mean of squares + eps) of the row in `srow`, the same bits in every lane.
// `tree` holds 256 floats. Ends with every lane past its reads of `tree`.
static __device__ __forceinline__ float inv_rms(const float* srow, float* tree, int cols, float eps) {
    const int t = threadIdx.x;
    float part = 0.0f;
    for (int i = t; i < cols; i += NORM_WG) part = fmaf(srow[i], srow[i], part);
    tree[t] = part;
    __syncthreads();
    // strides 128 and 64 cross the waves; every wave folds them itself from the shared partials
    const int l = t & 63;
    float v = (tree[l] + tree[l + 128]) + (tree[l + 64] + tree[l + 192]);
    // strides 32 .. 1 stay inside a wave; a + b == b + a, so the exchange form gives each lane the
    // bits the one-sided tree leaves in lane 0
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = v + __shfl_xor(v, o);
    __syncthreads();
    return 1.0f / sqrtf(v / (float)cols + eps);
}

// MODE 0: out = rmsnorm(x, w).  MODE 1: sum = x + residual; out = rmsnorm(sum, w).
// MODE 2: x_out = rmsnorm(x, w_first) + residual; out = rmsnorm(x_out, w).
static __device__ __forceinline__ float row_value(const float* x, size_t i) { return x[i]; }
static __device__ __forceinline__ float row_value(const __hip_bfloat16* x, size_t i) { return __bfloat162float(x[i]); }

// `out` may be null (MODE 0 only): the row then leaves as Q8_1 alone.
template <int MODE, typename XT = float>
__global__ __launch_bounds__(NORM_WG) void norm_q8_1_kernel(const XT* __restrict__ x, const float* __restrict__ w_first,
                                                            const float* __restrict__ residual,
                                                            const float* __restrict__ w, float* __restrict__ mid_out,
                                                            float* __restrict__ out, uint8_t* __restrict__ vy,
                                                            float eps_first, float eps, int cols) {
    extern __shared__ __align__(16) float srow[];
    __shared__ float tree[NORM_WG];
    const int t = threadIdx.x;
    const size_t offset = (size_t)blockIdx.x * cols;
    for (int i = t; i < cols; i += NORM_WG) {
        float v = row_value(x, offset + i);
        if (MODE == 1) {
            v = v + residual[offset + i];
            mid_out[offset + i] = v;
        }
        srow[i] = v;
    }
    if (MODE == 2) {
        const float rms_first = inv_rms(srow, tree, cols, eps_first);
        for (int i = t; i < cols; i += NORM_WG) {
            const float y = (srow[i] * rms_first) * w_first[i];
            const float r = y + residual[offset + i];
            srow[i] = r;
            mid_out[offset + i] = r;
        }
    }
    const float rms = inv_rms(srow, tree, cols, eps);
    uint8_t* row_blocks = vy + (size_t)blockIdx.x * (cols / 32) * Q81_BYTES;
    for (int i = t; i < cols; i += NORM_WG) {
        const float v = (srow[i] * rms) * w[i];
        if (out) out[offset + i] = v;
        quantize_lane(row_blocks, i, v);
    }
}

// out[r, i] = act(gu[r, i]) * gu[r, n + i], rows 2 n apart, also as Q8_1. ACT 0 SiLU, 1 tanh-GELU.
template <int ACT>
__global__ __launch_bounds__(NORM_WG) void split_act_mul_q8_1_kernel(const float* __restrict__ gu, float* __restrict__ out,
                                                                     uint8_t* __restrict__ vy, int n) {
    const int i = blockIdx.x * NORM_WG + threadIdx.x;
    if (i >= n) return;   // n is a multiple of 32: groups of 32 lanes leave together
    const size_t row = blockIdx.y;
    const float g = gu[row * 2 * n + i], u = gu[row * 2 * n + n + i];
    float a;
    if (ACT == 0) {
        a = g / (1.0f + expf(-g));
    } else {
        const float k0 = 0.7978845608028654f, k1 = 0.044715f;
        a = 0.5f * g * (1.0f + tanhf(k0 * (g + k1 * g * g * g)));
    }
    const float v = a * u;
    out[row * n + i] = v;
    quantize_lane(vy + row * (n / 32) * Q81_BYTES, i, v);
}

static bool norm_args_ok(int cols, int rows, int lds_limit) {
    return cols > 0 && cols % 512 == 0 && rows > 0 && (int64_t)cols * 4 + NORM_WG * 4 <= lds_limit;
}

template <class K>
static int prepare_lds(K kernel, int bytes) {
    // a kernel gets 64 KB of LDS unless the runtime is told otherwise (the static tree counts too)
    if (bytes + NORM_WG * 4 > 64 * 1024 &&
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return LK_ERR_LAUNCH;
    }
    return LK_OK;
}

}  // namespace

extern "C" int lk_rmsnorm_q8_1(const float* x, const float* weight, float* out, void* vy, float eps, int cols, int rows,
                               void* stream) {
    if (rows == 0) return LK_OK;
    if (!x || !weight || !out || !vy || ((uintptr_t)vy & 3) || !norm_args_ok(cols, rows, lk_device().lds_bytes)) return LK_ERR_ARG;
    if (prepare_lds(norm_q8_1_kernel<0>, cols * 4) != LK_OK) return LK_ERR_LAUNCH;
    hipLaunchKernelGGL(norm_q8_1_kernel<0>, dim3(rows), dim3(NORM_WG), cols * 4, (hipStream_t)stream, x, nullptr, nullptr,
                       weight, nullptr, out, (uint8_t*)vy, 0.0f, eps, cols);
    return lk_launch_status();
}

extern "C" int lk_add_rmsnorm_q8_1(const float* x, const float* residual, const float* weight, float* sum_out,
                                   float* norm_out, void* vy, float eps, int cols, int rows, void* stream) {
    if (rows == 0) return LK_OK;
    if (!x || !residual || !weight || !sum_out || !norm_out || !vy || ((uintptr_t)vy & 3) ||
        !norm_args_ok(cols, rows, lk_device().lds_bytes))
        return LK_ERR_ARG;
    if (prepare_lds(norm_q8_1_kernel<1>, cols * 4) != LK_OK) return LK_ERR_LAUNCH;
    hipLaunchKernelGGL(norm_q8_1_kernel<1>, dim3(rows), dim3(NORM_WG), cols * 4, (hipStream_t)stream, x, nullptr, residual,
                       weight, sum_out, norm_out, (uint8_t*)vy, 0.0f, eps, cols);
    return lk_launch_status();
}

extern "C" int lk_post_norm_add_norm_q8_1(const float* a, const float* w_post, const float* residual, const float* w_ffn,
                                          float* x_out, float* norm_out, void* vy, float eps_post, float eps_ffn,
                                          int cols, int rows, void* stream) {
    if (rows == 0) return LK_OK;
    if (!a || !w_post || !residual || !w_ffn || !x_out || !norm_out || !vy || ((uintptr_t)vy & 3) ||
        !norm_args_ok(cols, rows, lk_device().lds_bytes))
        return LK_ERR_ARG;
    if (prepare_lds(norm_q8_1_kernel<2>, cols * 4) != LK_OK) return LK_ERR_LAUNCH;
    hipLaunchKernelGGL(norm_q8_1_kernel<2>, dim3(rows), dim3(NORM_WG), cols * 4, (hipStream_t)stream, a, w_post, residual,
                       w_ffn, x_out, norm_out, (uint8_t*)vy, eps_post, eps_ffn, cols);
    return lk_launch_status();
}

extern "C" int lk_split_act_mul_q8_1(const float* gu, float* out, void* vy, int n, int rows, int act, void* stream) {
    if (rows == 0) return LK_OK;
    if (!gu || !out || !vy || ((uintptr_t)vy & 3) || n <= 0 || n % 32 != 0 || rows < 0 || rows > 65535) return LK_ERR_ARG;
    if (act != 0 && act != 1) return LK_ERR_TYPE;
    const dim3 grid((n + NORM_WG - 1) / NORM_WG, rows);
    if (act == 0)
        hipLaunchKernelGGL(split_act_mul_q8_1_kernel<0>, grid, dim3(NORM_WG), 0, (hipStream_t)stream, gu, out, (uint8_t*)vy, n);
    else
        hipLaunchKernelGGL(split_act_mul_q8_1_kernel<1>, grid, dim3(NORM_WG), 0, (hipStream_t)stream, gu, out, (uint8_t*)vy, n);
    return lk_launch_status();
}

// The reference's own names for the single-row launch in front of a mat-vec (cuda/moe/rms_qmatmul.cu:
// 152-169 f32 row, :221-238 bf16 row; declared src/inference/moe_cuda/mod.rs:117-119, 468-471; called
// from src/inference/moe_cuda/norm.rs:154, 206): y = Q8_1(rmsnorm(x, w_norm)), no f32 copy. Served
// by the kernel above, so the blocks are those of lk_rmsnorm_q8_1 (the sum of squares in the wide
// kernels' order, 1 / sqrt correctly rounded, lk_quantize_q8_1's block rule); hidden a multiple of
// 32 whose f32 row fits LDS. Void, as the reference's: nothing is launched on a bad argument.
extern "C" void loken_rms_quantize_q8_1(const float* x, const float* w_norm, void* y_q8_1, int hidden, float rms_eps,
                                        void* stream) {
    if (!x || !w_norm || !y_q8_1 || ((uintptr_t)y_q8_1 & 3) || hidden <= 0 || hidden % 32 != 0 ||
        (int64_t)hidden * 4 + NORM_WG * 4 > lk_device().lds_bytes)
        return;
    if (prepare_lds(norm_q8_1_kernel<0, float>, hidden * 4) != LK_OK) return;
    hipLaunchKernelGGL((norm_q8_1_kernel<0, float>), dim3(1), dim3(NORM_WG), hidden * 4, (hipStream_t)stream, x, nullptr, nullptr,
                       w_norm, nullptr, nullptr, (uint8_t*)y_q8_1, 0.0f, rms_eps, hidden);
}

extern "C" void loken_rms_quantize_q8_1_bf16(const void* x, const float* w_norm, void* y_q8_1, int hidden, float rms_eps,
                                             void* stream) {
    if (!x || !w_norm || !y_q8_1 || ((uintptr_t)y_q8_1 & 3) || ((uintptr_t)x & 1) || hidden <= 0 || hidden % 32 != 0 ||
        (int64_t)hidden * 4 + NORM_WG * 4 > lk_device().lds_bytes)
        return;
    if (prepare_lds(norm_q8_1_kernel<0, __hip_bfloat16>, hidden * 4) != LK_OK) return;
    hipLaunchKernelGGL((norm_q8_1_kernel<0, __hip_bfloat16>), dim3(1), dim3(NORM_WG), hidden * 4, (hipStream_t)stream,
                       (const __hip_bfloat16*)x, nullptr, nullptr, w_norm, nullptr, nullptr, (uint8_t*)y_q8_1, 0.0f, rms_eps,
                       hidden);
}

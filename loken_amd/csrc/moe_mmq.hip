// The small steps around the expert-batched tiled matmul of a MoE prefill: where each expert's
// run of sorted rows starts (plan / route), the gated activation between the two matmuls, and
// the weighted fold of a token's routed rows. Same entry points and arguments as loken's
// cuda/moe/moe_mmq.cu:180-218 (declared at src/inference/moe_cuda/mmq_experts.rs:42-56).
//
// Differences by design:
//   * route places rows in a stable order (ascending pair index inside an expert) by ranking
//     instead of atomics, so a launch is reproducible run to run;
//   * SiLU uses the accurate expf, as the host path does (src/inference/moe_cuda_cpu/mod.rs:598).
#include "lk_common.h"

namespace {

constexpr int THREADS = 256;
static inline int blocks_for(int64_t n) { return (int)((n + THREADS - 1) / THREADS); }

// bounds[e] = first sorted row whose expert is >= e, e in [0, n_experts]; src_rows[i] = token of row i.
__global__ void plan_kernel(const int32_t* __restrict__ experts, const int32_t* __restrict__ slots, int n,
                            int topk, int n_experts, int32_t* __restrict__ bounds,
                            int32_t* __restrict__ slots_out, int32_t* __restrict__ src_rows) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        slots_out[i] = slots[i];
        src_rows[i] = slots[i] / topk;
    }
    if (i <= n_experts) {
        int lo = 0, hi = n;
        while (lo < hi) {
            const int mid = (lo + hi) / 2;
            if (experts[mid] < i) lo = mid + 1; else hi = mid;
        }
        bounds[i] = lo;
    }
}

// One workgroup per expert: counts[e] = pairs that chose e.
__global__ __launch_bounds__(THREADS) void count_kernel(const int32_t* __restrict__ choices, int n,
                                                        int32_t* __restrict__ counts) {
    __shared__ int part[THREADS / 64];
    const int e = blockIdx.x;
    int c = 0;
    for (int i = threadIdx.x; i < n; i += THREADS) c += choices[i] == e;
    c = wave_sum_i32(c);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) counts[e] = part[0] + part[1] + part[2] + part[3];
}

__global__ void scan_kernel(const int32_t* __restrict__ counts, int n_experts, int32_t* __restrict__ bounds) {
    int at = 0;
    for (int e = 0; e < n_experts; ++e) {
        bounds[e] = at;
        at += counts[e];
    }
    bounds[n_experts] = at;
}

// Pair i goes to row bounds[e] + (number of earlier pairs that chose e): a stable grouping.
// One workgroup per expert walks the pairs in order, ranking 256 at a time.
__global__ __launch_bounds__(THREADS) void place_kernel(const int32_t* __restrict__ choices, int n, int topk,
                                                        const int32_t* __restrict__ bounds,
                                                        int32_t* __restrict__ slots, int32_t* __restrict__ src_rows) {
    __shared__ int wave_tot[THREADS / 64];
    const int e = blockIdx.x;
    int base = bounds[e];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i0 = 0; i0 < n; i0 += THREADS) {
        const int i = i0 + threadIdx.x;
        const bool mine = i < n && choices[i] == e;
        const unsigned long long ballot = __ballot(mine);
        const int before = __popcll(ballot & ((1ull << lane) - 1ull));
        if (lane == 0) wave_tot[wave] = __popcll(ballot);
        __syncthreads();
        int prior = 0, total = 0;
        for (int w = 0; w < THREADS / 64; ++w) {
            if (w < wave) prior += wave_tot[w];
            total += wave_tot[w];
        }
        if (mine) {
            const int row = base + prior + before;
            slots[row] = i;
            src_rows[row] = i / topk;
        }
        base += total;
        __syncthreads();
    }
}

__global__ void silu_mul_kernel(const float* __restrict__ gu, float* __restrict__ out, int64_t rows, int width) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * width) return;
    const int64_t r = i / width, c = i % width;
    const float g = gu[r * 2 * width + c];
    const float u = gu[r * 2 * width + width + c];
    out[i] = g / (1.0f + expf(-g)) * u;
}

static __device__ __forceinline__ int expert_of_row(const int32_t* __restrict__ bounds, int n_experts, int row) {
    int lo = 0, hi = n_experts;
    while (hi - lo > 1) {
        const int mid = (lo + hi) / 2;
        if (bounds[mid] <= row) lo = mid; else hi = mid;
    }
    return lo;
}

// x = min(g + gb, limit), u' = clamp(u + ub, -limit, limit), out = x * sigmoid(alpha x) * (1 + u')
__global__ void swiglu_oai_kernel(const float* __restrict__ gu, float* __restrict__ out, int64_t rows, int width,
                                  const int32_t* __restrict__ bounds, int n_experts,
                                  const float* __restrict__ gate_bias, const float* __restrict__ up_bias,
                                  float alpha, float limit) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * width) return;
    const int64_t r = i / width, c = i % width;
    float g = gu[r * 2 * width + c];
    float u = gu[r * 2 * width + width + c];
    if (gate_bias != nullptr || up_bias != nullptr) {
        const int64_t e = expert_of_row(bounds, n_experts, (int)r);
        if (gate_bias != nullptr) g += gate_bias[e * width + c];
        if (up_bias != nullptr) u += up_bias[e * width + c];
    }
    const float x = fminf(g, limit);
    const float uc = fminf(fmaxf(u, -limit), limit);
    const float sig = 1.0f / (1.0f + expf(-alpha * x));
    out[i] = (x * sig) * (1.0f + uc);
}

// out[t, c] += sum_k weights[p] * (pairs[p, c] + down_bias[choices[p], c]), p = t*topk + k, k ascending.
__global__ void fold_kernel(const float* __restrict__ pairs, const float* __restrict__ weights,
                            const int32_t* __restrict__ choices, const float* __restrict__ down_bias,
                            float* __restrict__ out, int64_t tokens, int topk, int cols) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= tokens * cols) return;
    const int64_t t = i / cols, c = i % cols;
    float acc = out[i];
    for (int k = 0; k < topk; ++k) {
        const int64_t p = t * topk + k;
        float v = pairs[p * cols + c];
        if (down_bias != nullptr) v += down_bias[(int64_t)choices[p] * cols + c];
        acc += weights[p] * v;
    }
    out[i] = acc;
}

}  // namespace

extern "C" void loken_moe_mmq_plan(const int32_t* experts, const int32_t* slots, int n, int topk, int n_experts,
                                   int32_t* bounds, int32_t* slots_out, int32_t* src_rows, void* stream) {
    const int span = n > n_experts + 1 ? n : n_experts + 1;
    hipLaunchKernelGGL(plan_kernel, dim3(blocks_for(span)), dim3(THREADS), 0, (hipStream_t)stream, experts, slots, n,
                       topk, n_experts, bounds, slots_out, src_rows);
    (void)hipGetLastError();
}

extern "C" void loken_moe_mmq_route(const int32_t* choices, int n, int topk, int n_experts, int32_t* counts,
                                    int32_t* bounds, int32_t* slots, int32_t* src_rows, void* stream) {
    if (n_experts <= 0) return;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(count_kernel, dim3(n_experts), dim3(THREADS), 0, s, choices, n, counts);
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1), 0, s, counts, n_experts, bounds);
    hipLaunchKernelGGL(place_kernel, dim3(n_experts), dim3(THREADS), 0, s, choices, n, topk, bounds, slots, src_rows);
    (void)hipGetLastError();
}

extern "C" void loken_moe_mmq_silu_mul(const float* gu, float* out, int64_t rows, int width, void* stream) {
    if (rows <= 0 || width <= 0) return;
    hipLaunchKernelGGL(silu_mul_kernel, dim3(blocks_for(rows * width)), dim3(THREADS), 0, (hipStream_t)stream, gu, out,
                       rows, width);
    (void)hipGetLastError();
}

extern "C" void loken_moe_mmq_swiglu_oai(const float* gu, float* out, int64_t rows, int width, const int32_t* bounds,
                                         int n_experts, const float* gate_bias, const float* up_bias, float alpha,
                                         float limit, void* stream) {
    if (rows <= 0 || width <= 0) return;
    hipLaunchKernelGGL(swiglu_oai_kernel, dim3(blocks_for(rows * width)), dim3(THREADS), 0, (hipStream_t)stream, gu,
                       out, rows, width, bounds, n_experts, gate_bias, up_bias, alpha, limit);
    (void)hipGetLastError();
}

extern "C" void loken_moe_mmq_fold(const float* pairs, const float* weights, const int32_t* choices,
                                   const float* down_bias, float* out, int64_t tokens, int topk, int cols,
                                   void* stream) {
    if (tokens <= 0 || cols <= 0) return;
    hipLaunchKernelGGL(fold_kernel, dim3(blocks_for(tokens * cols)), dim3(THREADS), 0, (hipStream_t)stream, pairs,
                       weights, choices, down_bias, out, tokens, topk, cols);
    (void)hipGetLastError();
}

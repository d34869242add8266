// The router step in front of the expert block: softmax over a row of expert logits, the k largest
// probabilities in descending order (ties to the lower expert id), optionally renormalized to sum
// to one. Same name and arguments as the reference's launcher (loken_topk_softmax,
// cuda/moe/gate_topk.cu:405-451; semantics of topk_softmax, src/inference/moe_cuda_cpu/mod.rs:
// 2098-2113: softmax -> argsort descending -> take k -> optional renorm).
//
// One wave per row, lane l holding experts l, l + 64, ...: the maximum, the sum and each of the k
// arg-max rounds are wave reductions; rows are tiny (128 logits), so the launch is latency only.

#include "lk_common.h"

namespace {

constexpr int MAX_PER_LANE = 8;   // up to 512 experts

static __device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    const int bits = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(bits, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(bits, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

__global__ __launch_bounds__(64) void topk_softmax_kernel(const float* __restrict__ logits, float* __restrict__ weights,
                                                          uint32_t* __restrict__ ids, int n_experts, int topk,
                                                          int with_norm) {
    const int row = blockIdx.x, lane = threadIdx.x;
    const float* x = logits + (size_t)row * n_experts;
    float p[MAX_PER_LANE];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        p[i] = e < n_experts ? x[e] : -INFINITY;
        mx = fmaxf(mx, p[i]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        p[i] = e < n_experts ? expf(p[i] - mx) : -1.f;   // -1: never chosen, probabilities are >= 0
        sum += e < n_experts ? p[i] : 0.f;
    }
    sum = wave_sum(sum);
    float picked_sum = 0.f, my_weight = 0.f;
    uint32_t my_id = 0;
    for (int j = 0; j < topk; ++j) {
        // the lane's best: largest probability, lowest expert id among equals
        float best = -1.f;
        int best_e = 0x7FFFFFFF;
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i)
            if (p[i] > best) { best = p[i]; best_e = lane + 64 * i; }
        // the wave's best, same order
        float w_best = best;
        int w_e = best_e;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float ob = __shfl_xor(w_best, o);
            const int oe = __shfl_xor(w_e, o);
            if (ob > w_best || (ob == w_best && oe < w_e)) { w_best = ob; w_e = oe; }
        }
        const float prob = w_best / sum;
        picked_sum += prob;
        if (lane == j) { my_weight = prob; my_id = (uint32_t)w_e; }
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i)
            if (lane + 64 * i == w_e) p[i] = -1.f;
    }
    if (lane < topk) {
        weights[(size_t)row * topk + lane] = with_norm ? my_weight / picked_sum : my_weight;
        ids[(size_t)row * topk + lane] = my_id;
    }
}

}  // namespace

extern "C" void loken_topk_softmax(const float* logits, float* weights, uint32_t* ids, int n_rows, int n_experts,
                                   int n_expert_used, int with_norm, void* stream) {
    if (!logits || !weights || !ids || n_rows <= 0) return;
    if (n_experts <= 0 || n_experts > 64 * MAX_PER_LANE || n_expert_used <= 0 || n_expert_used > 64 ||
        n_expert_used > n_experts)
        return;   // the caller falls back, as with the reference's launcher
    hipLaunchKernelGGL(topk_softmax_kernel, dim3(n_rows), dim3(64), 0, (hipStream_t)stream, logits, weights, ids,
                       n_experts, n_expert_used, with_norm);
    (void)hipGetLastError();
}

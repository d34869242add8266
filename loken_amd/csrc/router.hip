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

// Softmax over `x[0 .. n_experts)` and the k largest, by the 64 lanes of one wave.
static __device__ __forceinline__ void select_topk_softmax(const float* x, float* __restrict__ weights,
                                                           uint32_t* __restrict__ ids, int n_experts, int topk,
                                                           int with_norm, int lane) {
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
        weights[lane] = with_norm ? my_weight / picked_sum : my_weight;
        ids[lane] = my_id;
    }
}

__global__ __launch_bounds__(64) void topk_softmax_kernel(const float* __restrict__ logits, float* __restrict__ weights,
                                                          uint32_t* __restrict__ ids, int n_experts, int topk,
                                                          int with_norm) {
    const size_t row = blockIdx.x;
    select_topk_softmax(logits + row * n_experts, weights + row * topk, ids + row * topk, n_experts, topk, with_norm,
                        threadIdx.x);
}

// ---------------------------------------------------------------------------------------------
// The gate mat-vec, softmax and top-k of a token in one launch (loken_gate_topk_softmax,
// cuda/moe/gate_topk.cu:253-295, 366-403). The reference gives a token one warp and each lane
// whole weight rows, read four floats at a time at a stride of a row; here a token has a
// workgroup of 16 waves, a wave takes experts w, w + 16, ... and its lanes walk the row together
// (consecutive lanes read consecutive 16-byte pieces), so a one-token launch pulls the 1 MB of a
// 128 x 2048 gate at the rate one CU can stream rather than one lane's. Each logit is then
// a 64-lane sum instead of a serial one: same value up to f32 summation order. The selection is
// the wave-wide one above, run by wave 0 over the logits left in LDS.
// ---------------------------------------------------------------------------------------------
constexpr int GATE_WAVES = 16;

__global__ __launch_bounds__(64 * GATE_WAVES) void gate_topk_softmax_kernel(const float* __restrict__ x_in,
                                                                            const float* __restrict__ gate_w,
                                                                            float* __restrict__ weights,
                                                                            uint32_t* __restrict__ ids, int hidden,
                                                                            int n_experts, int topk, int with_norm) {
    extern __shared__ __align__(16) float gate_lds[];   // [hidden] the token, then [n_experts] logits
    float* xs = gate_lds;
    float* logits = gate_lds + ((hidden + 3) & ~3);
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const float* x = x_in + (size_t)row * hidden;
    const bool vec = (hidden & 3) == 0 && (((uintptr_t)x_in | (uintptr_t)gate_w) & 15) == 0;
    if (vec) {
        for (int i = tid; i < hidden / 4; i += 64 * GATE_WAVES) ((float4*)xs)[i] = ((const float4*)x)[i];
    } else {
        for (int i = tid; i < hidden; i += 64 * GATE_WAVES) xs[i] = x[i];
    }
    __syncthreads();
    for (int e = wave; e < n_experts; e += GATE_WAVES) {
        const float* w = gate_w + (size_t)e * hidden;
        float acc = 0.f;
        if (vec) {
            for (int i = lane; i < hidden / 4; i += 64) {
                const float4 a = ((const float4*)w)[i], b = ((const float4*)xs)[i];
                acc += a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
            }
        } else {
            for (int i = lane; i < hidden; i += 64) acc += w[i] * xs[i];
        }
        acc = wave_sum(acc);
        if (lane == 0) logits[e] = acc;
    }
    __syncthreads();
    if (wave == 0) select_topk_softmax(logits, weights + (size_t)row * topk, ids + (size_t)row * topk, n_experts, topk, with_norm, lane);
}

// A sigmoid router (loken_topk_sigmoid_post, cuda/moe/gate_topk.cu:140-200, 329-364, 479-512):
// every expert's probability stands alone, 1 / (1 + exp(-logit)); the k experts are chosen on the
// probability plus a per-expert bias (ties to the lower id) while the weight handed back is the
// unbiased probability, divided by max(sum of the k, 2^-14) when with_norm, then times `scale`.
__global__ __launch_bounds__(64) void topk_sigmoid_post_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ bias, float* __restrict__ weights,
                                                               uint32_t* __restrict__ ids, int n_experts, int topk,
                                                               int with_norm, float scale) {
    const int row = blockIdx.x, lane = threadIdx.x;
    const float* x = logits + (size_t)row * n_experts;
    float prob[MAX_PER_LANE], sel[MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        prob[i] = e < n_experts ? 1.0f / (1.0f + expf(-x[e])) : 0.f;
        sel[i] = e < n_experts ? prob[i] + (bias ? bias[e] : 0.f) : -INFINITY;
    }
    float picked_sum = 0.f, my_weight = 0.f;
    uint32_t my_id = 0;
    for (int j = 0; j < topk; ++j) {
        float best = -INFINITY, best_p = 0.f;
        int best_e = 0x7FFFFFFF;
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i)
            if (sel[i] > best) { best = sel[i]; best_p = prob[i]; best_e = lane + 64 * i; }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float ob = __shfl_xor(best, o), op = __shfl_xor(best_p, o);
            const int oe = __shfl_xor(best_e, o);
            if (ob > best || (ob == best && oe < best_e)) { best = ob; best_p = op; best_e = oe; }
        }
        picked_sum += best_p;
        if (lane == j) { my_weight = best_p; my_id = (uint32_t)best_e; }
#pragma unroll
        for (int i = 0; i < MAX_PER_LANE; ++i)
            if (lane + 64 * i == best_e) sel[i] = -INFINITY;
    }
    if (lane < topk) {
        if (with_norm) my_weight *= 1.0f / fmaxf(picked_sum, 6.103515625e-5f);
        weights[(size_t)row * topk + lane] = my_weight * scale;
        ids[(size_t)row * topk + lane] = my_id;
    }
}

// Stable ascending rank sort of u32 keys (loken_argsort_small_u32 and loken_stable_sort_u32,
// cuda/moe/gate_topk.cu:453-477, 515-548): key i lands after every smaller key and every equal
// key before it; `sorted` receives the keys, `order` the index each came from. One lane per key;
// the keys pass through LDS a chunk at a time, every lane reading each once.
constexpr int SORT_WG = 256, SORT_CHUNK = 2048;

__global__ __launch_bounds__(SORT_WG) void stable_rank_sort_u32_kernel(const uint32_t* __restrict__ keys,
                                                                       uint32_t* __restrict__ sorted,
                                                                       uint32_t* __restrict__ order, int n) {
    __shared__ uint32_t chunk[SORT_CHUNK];
    const int i = blockIdx.x * SORT_WG + threadIdx.x;
    const uint32_t k = i < n ? keys[i] : 0u;
    int rank = 0;
    for (int base = 0; base < n; base += SORT_CHUNK) {
        const int len = min(SORT_CHUNK, n - base);
        __syncthreads();
        for (int j = threadIdx.x; j < len; j += SORT_WG) chunk[j] = keys[base + j];
        __syncthreads();
        for (int j = 0; j < len; ++j) {
            const uint32_t kj = chunk[j];
            rank += (kj < k) || (kj == k && base + j < i);
        }
    }
    if (i < n) {
        sorted[rank] = k;
        order[rank] = (uint32_t)i;
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

static bool router_sizes_ok(int n_rows, int n_experts, int n_expert_used) {
    return n_rows > 0 && n_experts > 0 && n_experts <= 64 * MAX_PER_LANE && n_expert_used > 0 && n_expert_used <= 64 &&
           n_expert_used <= n_experts;
}

extern "C" void loken_gate_topk_softmax(const float* x_in, const float* gate_w, float* weights_out, uint32_t* ids_out,
                                        int hidden, int n_rows, int n_experts, int n_expert_used, int with_norm,
                                        void* stream) {
    if (!x_in || !gate_w || !weights_out || !ids_out || hidden <= 0 || hidden > 8192) return;   // the caller falls back
    if (!router_sizes_ok(n_rows, n_experts, n_expert_used)) return;
    const int lds = (((hidden + 3) & ~3) + n_experts) * 4;
    hipLaunchKernelGGL(gate_topk_softmax_kernel, dim3(n_rows), dim3(64 * GATE_WAVES), lds, (hipStream_t)stream, x_in,
                       gate_w, weights_out, ids_out, hidden, n_experts, n_expert_used, with_norm);
    (void)hipGetLastError();
}

extern "C" void loken_topk_sigmoid_post(const float* logits_in, const float* bias, float* weights_out, uint32_t* ids_out,
                                        int n_rows, int n_experts, int n_expert_used, int with_norm, float scale,
                                        void* stream) {
    if (!logits_in || !weights_out || !ids_out || !router_sizes_ok(n_rows, n_experts, n_expert_used)) return;
    hipLaunchKernelGGL(topk_sigmoid_post_kernel, dim3(n_rows), dim3(64), 0, (hipStream_t)stream, logits_in, bias,
                       weights_out, ids_out, n_experts, n_expert_used, with_norm, scale);
    (void)hipGetLastError();
}

extern "C" void loken_stable_sort_u32(const uint32_t* keys, uint32_t* sorted, uint32_t* order, int n, void* stream) {
    if (!keys || !sorted || !order || n <= 0) return;
    hipLaunchKernelGGL(stable_rank_sort_u32_kernel, dim3((n + SORT_WG - 1) / SORT_WG), dim3(SORT_WG), 0,
                       (hipStream_t)stream, keys, sorted, order, n);
    (void)hipGetLastError();
}

// The decode-size form of the same sort: the reference serves up to 32 keys with one warp and
// lets the caller fall back above; one workgroup here takes up to 256.
extern "C" void loken_argsort_small_u32(const uint32_t* in, uint32_t* sorted_out, uint32_t* index_out, int m,
                                        void* stream) {
    if (m <= 0 || m > SORT_WG) return;   // the caller falls back
    loken_stable_sort_u32(in, sorted_out, index_out, m, stream);
}

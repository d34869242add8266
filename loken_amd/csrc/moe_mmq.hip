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
constexpr int ROW_WAVES = THREADS / 64;   // the row-wise kernels give every wave a row

// A sorted routing -> where each expert's run starts. Entry i looks at the experts on both sides
// of position i (the one before position 0 counts as -1, the one at position n as n_experts) and
// writes i into bounds[e] for every e in (before, at]: exactly the experts whose first row, or
// whose empty run, sits at i. Every bounds entry is written once and nothing is searched.
__global__ __launch_bounds__(THREADS) void plan_kernel(const int32_t* __restrict__ experts,
                                                       const int32_t* __restrict__ slots, int n, int topk,
                                                       int n_experts, int32_t* __restrict__ bounds,
                                                       int32_t* __restrict__ slots_out, int32_t* __restrict__ src_rows) {
    const int i = blockIdx.x * THREADS + threadIdx.x;
    if (i > n) return;
    const int before = i > 0 ? min(max(experts[i - 1], -1), n_experts) : -1;
    const int at = i < n ? min(max(experts[i], -1), n_experts) : n_experts;
    for (int e = before + 1; e <= at; ++e) bounds[e] = i;
    if (i < n) {
        const int slot = slots[i];
        slots_out[i] = slot;
        src_rows[i] = slot / topk;
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

// The gated activations between the two expert matmuls. A wave takes one row of gu = [gate | up]
// and walks it in 16-byte pieces (both halves of a row are 16-byte aligned when width is a
// multiple of 4 and the buffers are; otherwise the wave falls back to single floats), so no
// element pays a division and a row's expert is found once, by the whole wave at a time.
struct GuRow {
    const float* gate;
    const float* up;
    float* out;
    bool vec;
};
static __device__ __forceinline__ GuRow gu_row(const float* gu, float* out, int64_t row, int width) {
    const float* g = gu + row * 2 * (int64_t)width;
    float* o = out + row * (int64_t)width;
    return GuRow{g, g + width, o, width % 4 == 0 && (((uintptr_t)g | (uintptr_t)o) & 15) == 0};
}
template <class F>
static __device__ __forceinline__ void for_row(const GuRow& r, int width, int lane, F&& f) {
    if (r.vec) {
        for (int c = 4 * lane; c < width; c += 256) {
            const float4 g = *(const float4*)(r.gate + c), u = *(const float4*)(r.up + c);
            *(float4*)(r.out + c) = make_float4(f(g.x, u.x, c), f(g.y, u.y, c + 1), f(g.z, u.z, c + 2), f(g.w, u.w, c + 3));
        }
    } else {
        for (int c = lane; c < width; c += 64) r.out[c] = f(r.gate[c], r.up[c], c);
    }
}

__global__ __launch_bounds__(THREADS) void silu_mul_kernel(const float* __restrict__ gu, float* __restrict__ out,
                                                           int64_t rows, int width) {
    const int64_t row = (int64_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    if (row >= rows) return;
    for_row(gu_row(gu, out, row, width), width, threadIdx.x & 63,
            [](float g, float u, int) { return g / (1.0f + expf(-g)) * u; });
}

// x = min(g + gb, limit), u' = clamp(u + ub, -limit, limit), out = x * sigmoid(alpha x) * (1 + u').
// The row's expert is the last one whose run starts at or before the row: the wave counts the
// starts that do, 64 at a time.
__global__ __launch_bounds__(THREADS) void swiglu_oai_kernel(const float* __restrict__ gu, float* __restrict__ out,
                                                             int64_t rows, int width, const int32_t* __restrict__ bounds,
                                                             int n_experts, const float* __restrict__ gate_bias,
                                                             const float* __restrict__ up_bias, float alpha, float limit) {
    const int64_t row = (int64_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const float* gb = nullptr;
    const float* ub = nullptr;
    if (gate_bias != nullptr || up_bias != nullptr) {
        int started = 0;
        for (int e0 = 0; e0 < n_experts; e0 += 64)
            started += __popcll(__ballot(e0 + lane < n_experts && bounds[e0 + lane] <= row));
        const int64_t e = started > 0 ? started - 1 : 0;
        if (gate_bias != nullptr) gb = gate_bias + e * width;
        if (up_bias != nullptr) ub = up_bias + e * width;
    }
    for_row(gu_row(gu, out, row, width), width, lane, [=](float g, float u, int c) {
        if (gb) g += gb[c];
        if (ub) u += ub[c];
        const float x = fminf(g, limit);
        const float clamped = fminf(fmaxf(u, -limit), limit);
        return (x * (1.0f / (1.0f + expf(-alpha * x)))) * (1.0f + clamped);
    });
}

// out[t, c] += sum over k ascending of weights[p] * (pairs[p, c] + down_bias[choices[p], c]),
// p = t * topk + k. A workgroup column of the grid is one token; a thread owns four columns and
// keeps four routed rows' loads in flight, adding them in k order.
constexpr int FOLD_AHEAD = 4;
template <bool VEC>
__global__ __launch_bounds__(THREADS) void fold_kernel(const float* __restrict__ pairs, const float* __restrict__ weights,
                                                       const int32_t* __restrict__ choices,
                                                       const float* __restrict__ down_bias, float* __restrict__ out,
                                                       int topk, int cols) {
    constexpr int W = VEC ? 4 : 1;
    const int c = (blockIdx.x * THREADS + threadIdx.x) * W;
    if (c >= cols) return;
    const int64_t t = blockIdx.y, p0 = t * topk;
    float* o = out + t * cols + c;
    float acc[W];
    if (VEC) {
        const float4 v = *(const float4*)o;
        acc[0] = v.x; acc[W > 1 ? 1 : 0] = v.y; acc[W > 2 ? 2 : 0] = v.z; acc[W > 3 ? 3 : 0] = v.w;
    } else {
        acc[0] = *o;
    }
    auto row_at = [&](const float* base, int64_t r, float (&v)[W]) {
        const float* src = base + r * cols + c;
        if (VEC) {
            const float4 x = *(const float4*)src;
            v[0] = x.x; v[W > 1 ? 1 : 0] = x.y; v[W > 2 ? 2 : 0] = x.z; v[W > 3 ? 3 : 0] = x.w;
        } else {
            v[0] = *src;
        }
    };
    for (int k0 = 0; k0 < topk; k0 += FOLD_AHEAD) {
        float v[FOLD_AHEAD][W], b[FOLD_AHEAD][W], w[FOLD_AHEAD];
#pragma unroll
        for (int j = 0; j < FOLD_AHEAD; ++j) {
            const int64_t p = p0 + min(k0 + j, topk - 1);   // past the end: a repeat, dropped below
            row_at(pairs, p, v[j]);
            w[j] = weights[p];
            if (down_bias != nullptr) row_at(down_bias, choices[p], b[j]);
        }
#pragma unroll
        for (int j = 0; j < FOLD_AHEAD; ++j) {
            if (k0 + j >= topk) break;
#pragma unroll
            for (int e = 0; e < W; ++e) acc[e] += w[j] * (down_bias != nullptr ? v[j][e] + b[j][e] : v[j][e]);
        }
    }
    if (VEC) *(float4*)o = make_float4(acc[0], acc[W > 1 ? 1 : 0], acc[W > 2 ? 2 : 0], acc[W > 3 ? 3 : 0]);
    else *o = acc[0];
}

}  // namespace

static inline unsigned row_groups(int64_t rows) { return (unsigned)((rows + ROW_WAVES - 1) / ROW_WAVES); }

extern "C" void loken_moe_mmq_plan(const int32_t* experts, const int32_t* slots, int n, int topk, int n_experts,
                                   int32_t* bounds, int32_t* slots_out, int32_t* src_rows, void* stream) {
    if (n < 0 || n_experts < 0 || topk <= 0) return;
    // positions 0 .. n inclusive: the one past the end closes the last runs
    hipLaunchKernelGGL(plan_kernel, dim3((unsigned)(n / THREADS + 1)), dim3(THREADS), 0, (hipStream_t)stream, experts,
                       slots, n, topk, n_experts, bounds, slots_out, src_rows);
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
    hipLaunchKernelGGL(silu_mul_kernel, dim3(row_groups(rows)), dim3(THREADS), 0, (hipStream_t)stream, gu, out, rows, width);
    (void)hipGetLastError();
}

extern "C" void loken_moe_mmq_swiglu_oai(const float* gu, float* out, int64_t rows, int width, const int32_t* bounds,
                                         int n_experts, const float* gate_bias, const float* up_bias, float alpha,
                                         float limit, void* stream) {
    if (rows <= 0 || width <= 0) return;
    hipLaunchKernelGGL(swiglu_oai_kernel, dim3(row_groups(rows)), dim3(THREADS), 0, (hipStream_t)stream, gu, out, rows,
                       width, bounds, n_experts, gate_bias, up_bias, alpha, limit);
    (void)hipGetLastError();
}

extern "C" void loken_moe_mmq_fold(const float* pairs, const float* weights, const int32_t* choices,
                                   const float* down_bias, float* out, int64_t tokens, int topk, int cols,
                                   void* stream) {
    if (tokens <= 0 || cols <= 0 || topk <= 0 || tokens > 65535 * (int64_t)65535) return;
    hipStream_t s = (hipStream_t)stream;
    const bool vec = cols % 4 == 0 && (((uintptr_t)pairs | (uintptr_t)out | (uintptr_t)down_bias) & 15) == 0;
    // tokens ride the grid's second axis, 65535 at a time
    for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
        const unsigned ty = (unsigned)(tokens - t0 < 65535 ? tokens - t0 : 65535);
        const float* p = pairs + t0 * topk * cols;
        const float* w = weights + t0 * topk;
        const int32_t* ch = choices ? choices + t0 * topk : nullptr;
        float* o = out + t0 * cols;
        if (vec)
            hipLaunchKernelGGL(fold_kernel<true>, dim3((unsigned)((cols / 4 + THREADS - 1) / THREADS), ty), dim3(THREADS), 0, s, p, w,
                               ch, down_bias, o, topk, cols);
        else
            hipLaunchKernelGGL(fold_kernel<false>, dim3((unsigned)((cols + THREADS - 1) / THREADS), ty), dim3(THREADS), 0, s, p, w,
                               ch, down_bias, o, topk, cols);
    }
    (void)hipGetLastError();
}

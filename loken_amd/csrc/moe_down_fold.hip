// MoE decode, the down projection and the fold over a token's routed pairs in ONE launch, for Q4_K
// experts with short rows (k <= 1024) and a handful of tokens. What it replaces is the pair of
// launches of loken_moe_gemm_gguf_down_reduce (cuda/moe/moe_gguf.cu:755-860 of the reference and the
// sum after it, :591-625): a mat-vec per routed pair into a scratch of pair rows, then a kernel that
// sums each token's rows in slot order. At one to sixteen tokens both are a few microseconds of
// dependent memory round trips each, so a launch saved is a quarter of the down side's time.
//
// grid (row groups, tokens). A workgroup owns one token and some output rows. Its 256 lanes first
// quantize the token's topk activation rows (f32, row `slot` of `inputs`) into LDS with the
// quantizer's steps, and find the expert of each of the token's slots by scanning the routing
// (sorted_token_ids / expert_ids name pairs in the router's order, not the token's). Lane
// (r, j, q) of a wave then holds, for the whole launch, the Q8_1 codes of quarter q of every
// super-block of activation row j in registers, and per pass loads the matching quarter of weight
// row r of expert e_j: 4 lanes per (row, expert), 4 * TKP lanes per output row. The four lanes'
// shares meet over DPP, the topk pair totals are weighted and summed in slot order, exactly the
// order of the fold kernel, and one lane stores the output element. No scratch, no atomics, and
// the same bits as the two launches give.

#include "mmvq_core.h"

using namespace mmvq;

namespace {

// The activation rows in LDS: codes in value order, then (d, d * sum of codes) per Q8_1 block.
struct FmtLinear {
    static constexpr int BLOCK_BYTES = Q4K_BYTES, BLOCK_LEN = 256;
    static constexpr int VPI = 1024;
    static constexpr int PLANES = 1, SCF = 2;
    static __device__ __forceinline__ int slot(int j, int lh) { return j * 32 + lh * 16; }
};

struct FoldDims {
    int experts, topk, pairs, cols, passes;
    int64_t slab_bytes;
};

constexpr int SCAN_ROUNDS = 2;              // routing entries a lane looks at: pairs <= 2 * 256
constexpr int MAX_PAIRS = SCAN_ROUNDS * WG;

template <int NB>
struct FoldFrag {
    uint4 hdr[NB], q0[NB], q1[NB];
    float prev, bias;
};

template <int NB, int TKP>
__global__ __launch_bounds__(WG) void moe_down_fold_q4k_kernel(const uint8_t* __restrict__ w,
                                                               const float* __restrict__ acts,
                                                               const int32_t* __restrict__ sorted_token_ids,
                                                               const int32_t* __restrict__ expert_ids,
                                                               const float* __restrict__ topk_weights,
                                                               const float* __restrict__ down_bias,
                                                               const float* __restrict__ add_after,
                                                               float* __restrict__ out, FoldDims d) {
    constexpr int LPR = 4 * TKP;            // lanes per output row
    constexpr int RPW = 64 / LPR;           // output rows per wave and pass
    constexpr int RPG = RPW * WAVES;        // per workgroup and pass
    constexpr int K = NB * 256, K32 = NB * 8, QUADS = K / 4;
    constexpr int N_ITER = (K + FmtLinear::VPI - 1) / FmtLinear::VPI;
    // 16 bytes on top of a row keep activation rows j and j + 1 off each other's banks
    constexpr int PITCH = lds_bytes_per_row<FmtLinear>(N_ITER) + 16;
    constexpr int ACT_LOADS = (TKP * QUADS + WG - 1) / WG;
    __shared__ __align__(16) uint8_t lds[TKP * PITCH];
    __shared__ int e_of[TKP];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane / LPR, j = (lane % LPR) >> 2, q = lane & 3;
    const int token = blockIdx.y;
    const int slot0 = token * d.topk;

    // ---- loads that depend on nothing: the routing, then the token's activation rows
    int s_at[SCAN_ROUNDS], e_at[SCAN_ROUNDS];
#pragma unroll
    for (int u = 0; u < SCAN_ROUNDS; ++u) {
        const int i = min(tid + u * WG, d.pairs - 1);
        s_at[u] = sorted_token_ids[i];
        e_at[u] = expert_ids[i];
    }
    const float scale = topk_weights[slot0 + min(j, d.topk - 1)];
    float4 x[ACT_LOADS];
#pragma unroll
    for (int u = 0; u < ACT_LOADS; ++u) {
        const int t = tid + u * WG;
        const int jj = min(t / QUADS, d.topk - 1), tq = t % QUADS;
        x[u] = *(const float4*)(acts + (size_t)(slot0 + jj) * K + (size_t)tq * 4);
    }
    load_fence(acts);

    // ---- the expert of each of the token's slots
    if (tid < TKP) e_of[tid] = -1;
    __syncthreads();
#pragma unroll
    for (int u = 0; u < SCAN_ROUNDS; ++u) {
        const int rel = s_at[u] - slot0;
        if (tid + u * WG < d.pairs && rel >= 0 && rel < d.topk) e_of[rel] = e_at[u];
    }
    __syncthreads();
    const int e = e_of[j];
    const bool routed = e >= 0 && e < d.experts;   // a slot no pair names, or an expert out of range, adds nothing

    const gbytes_t slab = to_gbytes(w) + (int64_t)(routed ? e : 0) * d.slab_bytes;
    const int group0 = blockIdx.x * d.passes;
    const size_t out_at = (size_t)token * d.cols;
    const float* before = add_after ? add_after : out;   // what the sum starts from / ends with
    auto row_of = [&](int p) { return (group0 + p) * RPG + wave * RPW + r; };
    auto load = [&](FoldFrag<NB>& f, int p) {
        const int row = min(row_of(p), d.cols - 1);
        const uint8_t* bp = (const uint8_t*)(slab + (size_t)row * (NB * Q4K_BYTES));
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            f.hdr[b] = *(const uint4*)(bp + b * Q4K_BYTES);
            f.q0[b] = *(const uint4*)(bp + b * Q4K_BYTES + 16 + 32 * q);
            f.q1[b] = *(const uint4*)(bp + b * Q4K_BYTES + 32 + 32 * q);
        }
        f.prev = before[out_at + row];
        f.bias = down_bias ? down_bias[(size_t)(routed ? e : 0) * d.cols + row] : 0.f;
    };
    FoldFrag<NB> fa, fb;
    load(fa, 0);
    load_fence(w);

    // ---- the activation rows into LDS as Q8_1
#pragma unroll
    for (int u = 0; u < ACT_LOADS; ++u) {
        const int t = tid + u * WG;
        if (t / QUADS < d.topk) put_f32_quad<FmtLinear>(lds + (t / QUADS) * PITCH, N_ITER, K32, t % QUADS, x[u]);
    }
    __syncthreads();

    // ---- this lane's quarter of every super-block of activation row j, for the whole launch
    uint4 a00[NB], a01[NB], a10[NB], a11[NB];
    float4 s4[NB];
    {
        const uint8_t* rowl = lds + j * PITCH;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint8_t* codes = rowl + b * 256 + q * 64;
            a00[b] = *(const uint4*)(codes);
            a01[b] = *(const uint4*)(codes + 16);
            a10[b] = *(const uint4*)(codes + 32);
            a11[b] = *(const uint4*)(codes + 48);
            s4[b] = *(const float4*)(rowl + N_ITER * FmtLinear::VPI + (b * 8 + 2 * q) * 8);
        }
    }
    const Q4KScaleSel sel(q);

    auto compute = [&](const FoldFrag<NB>& f, int p) {
        // Per super-block the four lanes' shares meet first, then the blocks add up as
        // (Q0 + Q1) + (Q2 + Q3): the order of the short-row mat-vec engine's fold over a row of 16
        // lanes, so a pair's total carries the same bits as the per-pair launch gives it.
        float quad[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            uint32_t sc, mn;
            sel.unpack(f.hdr[b].y, f.hdr[b].z, f.hdr[b].w, sc, mn);
            const float dd = f16_bits_to_f32(f.hdr[b].x & 0xFFFFu), dmin = f16_bits_to_f32(f.hdr[b].x >> 16);
            int d_lo = 0, d_hi = 0;
            q4k_dots(f.q0[b], a00[b], a10[b], d_lo, d_hi);
            q4k_dots(f.q1[b], a01[b], a11[b], d_lo, d_hi);
            float sh = q4k_pair_share(dd, dmin, (float)(sc & 0xFFu), (float)(sc >> 8), (float)(mn & 0xFFu), (float)(mn >> 8),
                                      s4[b].x, s4[b].z, s4[b].y, s4[b].w, (float)d_lo, (float)d_hi);
            sh += dpp_f32<0xB1>(sh);
            sh += dpp_f32<0x4E>(sh);
            quad[b] = sh;
        }
        const float acc = (quad[0] + quad[1]) + (quad[2] + quad[3]);
        float v = acc * scale;
        if (down_bias) v += scale * f.bias;
        const int bits = __float_as_int(routed ? v : 0.f);
        const int prev_bits = __float_as_int(f.prev);
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            float sum = add_after ? 0.f : __int_as_float(__builtin_amdgcn_readlane(prev_bits, rr * LPR));
#pragma unroll
            for (int jj = 0; jj < TKP; ++jj) sum += __int_as_float(__builtin_amdgcn_readlane(bits, rr * LPR + 4 * jj));
            if (add_after) sum += __int_as_float(__builtin_amdgcn_readlane(prev_bits, rr * LPR));
            const int row = (group0 + p) * RPG + wave * RPW + rr;
            if (lane == rr * LPR && row < d.cols) out[out_at + row] = sum;
        }
    };

    // Passes ping-pong between two fragments; a load past the last pass re-reads it (never a branch
    // around a load: the wait before the next use could then no longer count the loads ahead of it).
    const int last = d.passes - 1;
    if (last == 0) {
        compute(fa, 0);
        return;
    }
    for (int p = 0;; p += 2) {
        load(fb, min(p + 1, last));
        compute(fa, p);
        if (p + 1 > last) break;
        load(fa, min(p + 2, last));
        compute(fb, p + 1);
        if (p + 2 > last) break;
    }
}

template <int NB, int TKP>
int launch(const uint8_t* w, const float* acts, const int32_t* sti, const int32_t* eid, const float* tkw,
           const float* bias, const float* add, float* out, FoldDims d, int tokens, hipStream_t s) {
    constexpr int RPG = 64 / (4 * TKP) * WAVES;
    const int groups = (d.cols + RPG - 1) / RPG;
    // enough workgroups for three per CU; past that a workgroup takes more rows, so that the
    // token's activation rows are quantized by fewer of them
    int passes = (int)(((int64_t)tokens * groups + 3 * lk_device().cus - 1) / (3 * lk_device().cus));
    if (const int t = lk_tune_env("LK_TUNE_DOWN_FOLD_PASSES")) passes = t;
    passes = passes < 1 ? 1 : passes > 16 ? 16 : passes;
    d.passes = passes;
    d.slab_bytes = (int64_t)d.cols * NB * Q4K_BYTES;
    const dim3 grid((groups + passes - 1) / passes, tokens);
    hipLaunchKernelGGL((moe_down_fold_q4k_kernel<NB, TKP>), grid, dim3(WG), 0, s, w, acts, sti, eid, tkw, bias, add, out, d);
    return lk_launch_status();
}

template <int NB>
int launch_topk(const uint8_t* w, const float* acts, const int32_t* sti, const int32_t* eid, const float* tkw,
                const float* bias, const float* add, float* out, FoldDims d, int tokens, hipStream_t s) {
    return d.topk <= 4 ? launch<NB, 4>(w, acts, sti, eid, tkw, bias, add, out, d, tokens, s)
                       : launch<NB, 8>(w, acts, sti, eid, tkw, bias, add, out, d, tokens, s);
}

}  // namespace

// Down + fold of Q4_K experts in one launch. Returns -1 when this kernel does not serve the call
// (the caller then takes the two launches), else an LK_* status.
int lk_moe_down_fold_q4k(const float* inputs, const void* weights, const int32_t* sorted_token_ids,
                         const int32_t* expert_ids, const float* topk_weights, float* outputs, int num_experts, int topk,
                         int size_m, int size_n, int size_k, const float* down_bias, const float* add_after,
                         hipStream_t stream) {
    if (lk_tune_env("LK_TUNE_DOWN_FOLD_OFF")) return -1;
    if (size_k % 256 != 0 || topk < 1 || topk > 8 || size_m > MAX_PAIRS || size_m % topk != 0) return -1;
    if ((((uintptr_t)inputs) | ((uintptr_t)weights)) & 15) return -1;
    const int tokens = size_m / topk;
    if (tokens < 1 || tokens > 65535) return -1;
    FoldDims d{num_experts, topk, size_m, size_n, 1, 0};
    const uint8_t* w = (const uint8_t*)weights;
    switch (size_k / 256) {
        case 2: return launch_topk<2>(w, inputs, sorted_token_ids, expert_ids, topk_weights, down_bias, add_after, outputs, d, tokens, stream);
        case 3: return launch_topk<3>(w, inputs, sorted_token_ids, expert_ids, topk_weights, down_bias, add_after, outputs, d, tokens, stream);
        case 4: return launch_topk<4>(w, inputs, sorted_token_ids, expert_ids, topk_weights, down_bias, add_after, outputs, d, tokens, stream);
        default: return -1;
    }
}

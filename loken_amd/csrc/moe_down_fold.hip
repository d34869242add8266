// MoE decode, the down projection and the fold over a token's routed pairs in ONE launch, for Q4_K,
// Q5_K and Q6_K experts with short rows (k <= 1024) and a handful of tokens. What it replaces is the
// pair of launches of loken_moe_gemm_gguf_down_reduce (cuda/moe/moe_gguf.cu:755-860 of the reference
// and the sum after it, :591-625): a mat-vec per routed pair into a scratch of pair rows, then a
// kernel that sums each token's rows in slot order. At one to sixteen tokens both are a few
// microseconds of dependent memory round trips each, so a launch saved is a third of the down side's
// time.
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

// The activation rows in LDS: codes in value order, then the scale table of the format's engine
// (Q4_K / Q5_K: (d, d * sum of codes) per Q8_1 block; Q6_K: d, then -32 * the code sum of every
// block's first and of its last 16 values).
template <int SCF_>
struct FmtLinear {
    static constexpr int VPI = 1024;
    static constexpr int PLANES = 1, SCF = SCF_;
    static __device__ __forceinline__ int slot(int j, int lh) { return j * 32 + lh * 16; }
};

// What lane q (0..3) of a super-block loads, keeps of the activation and makes of the two.
template <bool Q5>
struct LaneQ4K {
    using Fmt = FmtLinear<2>;
    static constexpr int BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES, QS0 = Q5 ? 48 : 16, ALIGN = 16;
    struct W {
        uint4 hdr, q0, q1, h0, h1;   // h0 / h1: Q5_K's fifth bits over l 0..15 and 16..31
    };
    struct A {
        uint4 a00, a01, a10, a11;
        float4 s4;
    };
    static __device__ __forceinline__ void load(W& f, const uint8_t* bp, int q) {
        f.hdr = *(const uint4*)(bp);
        f.q0 = *(const uint4*)(bp + QS0 + 32 * q);
        f.q1 = *(const uint4*)(bp + QS0 + 16 + 32 * q);
        if (Q5) {
            f.h0 = *(const uint4*)(bp + 16);
            f.h1 = *(const uint4*)(bp + 32);
        }
    }
    static __device__ __forceinline__ void read(A& a, const uint8_t* rowl, int table, int total, int b, int q) {
        const uint8_t* codes = rowl + b * 256 + q * 64;
        a.a00 = *(const uint4*)(codes);
        a.a01 = *(const uint4*)(codes + 16);
        a.a10 = *(const uint4*)(codes + 32);
        a.a11 = *(const uint4*)(codes + 48);
        a.s4 = *(const float4*)(rowl + table + (b * 8 + 2 * q) * 8);
    }
    static __device__ __forceinline__ float share(const W& f, const A& a, int q) {
        const Q4KScaleSel sel(q);
        uint32_t sc, mn;
        sel.unpack(f.hdr.y, f.hdr.z, f.hdr.w, sc, mn);
        const float dd = f16_bits_to_f32(f.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(f.hdr.x >> 16);
        int d_lo = 0, d_hi = 0;
        if (Q5) {
            q5k_dots(f.q0, shr4(f.h0, 2 * q), a.a00, a.a10, d_lo, d_hi);
            q5k_dots(f.q1, shr4(f.h1, 2 * q), a.a01, a.a11, d_lo, d_hi);
        } else {
            q4k_dots(f.q0, a.a00, a.a10, d_lo, d_hi);
            q4k_dots(f.q1, a.a01, a.a11, d_lo, d_hi);
        }
        return q4k_pair_share(dd, dmin, (float)(sc & 0xFFu), (float)(sc >> 8), (float)(mn & 0xFFu), (float)(mn >> 8),
                              a.s4.x, a.s4.z, a.s4.y, a.s4.w, (float)d_lo, (float)d_hi);
    }
};

struct LaneQ6K {   // q = 2 * (half of the super-block) + (which 16-byte run of the half's l range)
    using Fmt = FmtLinear<3>;
    static constexpr int BYTES = Q6K_BYTES, ALIGN = 2;
    struct W {
        uint4 ql0, ql1, qh;
        uint2 sc;
        uint32_t d;
    };
    struct A {
        uint4 a[4];
        float4 d8;
        int4 bias;
    };
    static __device__ __forceinline__ void load(W& f, const uint8_t* bp, int q) {
        const int h = q >> 1, lh = q & 1;
        f.ql0 = *(const uint4_a2*)(bp + 64 * h + 16 * lh);
        f.ql1 = *(const uint4_a2*)(bp + 64 * h + 16 * lh + 32);
        f.qh = *(const uint4_a2*)(bp + 128 + 32 * h + 16 * lh);
        f.sc = *(const uint2_a2*)(bp + 192 + 8 * h);
        f.d = *(const uint16_t*)(bp + 208);
    }
    static __device__ __forceinline__ void read(A& a, const uint8_t* rowl, int table, int total, int b, int q) {
        const int h = q >> 1, lh = q & 1;
        const int j0 = b * 8 + 4 * h;   // the half's four Q8_1 blocks
#pragma unroll
        for (int g = 0; g < 4; ++g) a.a[g] = *(const uint4*)(rowl + (j0 + g) * 32 + lh * 16);
        a.d8 = *(const float4*)(rowl + table + 4 * j0);
        a.bias = *(const int4*)(rowl + table + 4 * (total * (1 + lh) + j0));
    }
    static __device__ __forceinline__ float share(const W& f, const A& a, int q) {
        float ds[4];
        q6k_run_scales(f16_bits_to_f32(f.d), f.sc, q & 1, ds);
        int dot[4] = {a.bias.x, a.bias.y, a.bias.z, a.bias.w};
        q6k_dots_biased(f.ql0, f.ql1, f.qh, a.a, dot);
        float acc = 0.f;
        asm("" : "+v"(acc));   // a running sum to the compiler, as in the mat-vec engine: same contraction, same bits
        q6k_half_share(acc, ds, a.d8, dot);
        return acc;
    }
};

struct FoldDims {
    int experts, topk, pairs, cols, passes;
    int64_t slab_bytes;
};

constexpr int SCAN_ROUNDS = 2;              // routing entries a lane looks at: pairs <= 2 * 256
constexpr int MAX_PAIRS = SCAN_ROUNDS * WG;

template <class L, int NB>
struct FoldFrag {
    typename L::W w[NB];
    float prev, bias;
};

template <class L, int NB, int TKP>
__global__ __launch_bounds__(WG) void moe_down_fold_kernel(const uint8_t* __restrict__ w, const float* __restrict__ acts,
                                                           const int32_t* __restrict__ sorted_token_ids,
                                                           const int32_t* __restrict__ expert_ids,
                                                           const float* __restrict__ topk_weights,
                                                           const float* __restrict__ down_bias,
                                                           const float* __restrict__ add_after, float* __restrict__ out,
                                                           FoldDims d) {
    using Fmt = typename L::Fmt;
    constexpr int LPR = 4 * TKP;            // lanes per output row
    constexpr int RPW = 64 / LPR;           // output rows per wave and pass
    constexpr int RPG = RPW * WAVES;        // per workgroup and pass
    constexpr int K = NB * 256, K32 = NB * 8, QUADS = K / 4;
    constexpr int N_ITER = (K + Fmt::VPI - 1) / Fmt::VPI;
    constexpr int TABLE = N_ITER * Fmt::VPI, TOTAL = N_ITER * (Fmt::VPI / 32);
    // 16 bytes on top of a row keep activation rows j and j + 1 off each other's banks
    constexpr int PITCH = lds_bytes_per_row<Fmt>(N_ITER) + 16;
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
    auto load = [&](FoldFrag<L, NB>& f, int p) {
        const int row = min((group0 + p) * RPG + wave * RPW + r, d.cols - 1);
        const uint8_t* bp = (const uint8_t*)(slab + (size_t)row * (NB * L::BYTES));
#pragma unroll
        for (int b = 0; b < NB; ++b) L::load(f.w[b], bp + b * L::BYTES, q);
        f.prev = before[out_at + row];
        f.bias = down_bias ? down_bias[(size_t)(routed ? e : 0) * d.cols + row] : 0.f;
    };
    FoldFrag<L, NB> fa, fb;
    load(fa, 0);
    load_fence(w);

    // ---- the activation rows into LDS as Q8_1
#pragma unroll
    for (int u = 0; u < ACT_LOADS; ++u) {
        const int t = tid + u * WG;
        if (t / QUADS < d.topk) put_f32_quad<Fmt>(lds + (t / QUADS) * PITCH, N_ITER, K32, t % QUADS, x[u]);
    }
    __syncthreads();

    // ---- this lane's quarter of every super-block of activation row j, for the whole launch
    typename L::A act[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) L::read(act[b], lds + j * PITCH, TABLE, TOTAL, b, q);

    auto compute = [&](const FoldFrag<L, NB>& f, int p) {
        // Per super-block the four lanes' shares meet first, then the blocks add up as
        // (Q0 + Q1) + (Q2 + Q3): the order of the short-row mat-vec engines' fold over a row of 16
        // lanes, so a pair's total carries the same bits as the per-pair launch gives it.
        float quad[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float sh = L::share(f.w[b], act[b], q);
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

struct FoldCall {
    const uint8_t* w;
    const float* acts;
    const int32_t *sti, *eid;
    const float *tkw, *bias, *add;
    float* out;
    int tokens;
    hipStream_t s;
};

template <class L, int NB, int TKP>
int launch(const FoldCall& c, FoldDims d) {
    constexpr int RPG = 64 / (4 * TKP) * WAVES;
    const int groups = (d.cols + RPG - 1) / RPG;
    // enough workgroups for two per CU; past that a workgroup takes more rows, so that the token's
    // activation rows are quantized by fewer of them. An even count: the passes go two to a turn of
    // the loop, and an odd last turn loads a pass nobody computes (measured at 8 tokens: 3 passes
    // 35.5 us per block, 4 passes 32.9; at 16 tokens 6: 54.7, 8: 51.3).
    int passes = (int)(((int64_t)c.tokens * groups + 2 * lk_device().cus - 1) / (2 * lk_device().cus));
    passes = passes <= 1 ? 1 : passes <= 2 ? 2 : passes <= 5 ? 4 : 8;   // (12 passes: 57 us at 16 tokens, 88 at 24 against 81)
    if (const int t = lk_tune_env("LK_TUNE_DOWN_FOLD_PASSES")) passes = t;
    passes = passes < 1 ? 1 : passes > 16 ? 16 : passes;
    d.passes = passes;
    d.slab_bytes = (int64_t)d.cols * NB * L::BYTES;
    const dim3 grid((groups + passes - 1) / passes, c.tokens);
    hipLaunchKernelGGL((moe_down_fold_kernel<L, NB, TKP>), grid, dim3(WG), 0, c.s, c.w, c.acts, c.sti, c.eid, c.tkw, c.bias,
                       c.add, c.out, d);
    return lk_launch_status();
}

template <class L>
int launch_format(const FoldCall& c, const FoldDims& d, int nb) {
    if (((uintptr_t)c.w) & (L::ALIGN - 1)) return -1;
    const bool few = d.topk <= 4;
    switch (nb) {
        case 2: return few ? launch<L, 2, 4>(c, d) : launch<L, 2, 8>(c, d);
        case 3: return few ? launch<L, 3, 4>(c, d) : launch<L, 3, 8>(c, d);
        case 4: return few ? launch<L, 4, 4>(c, d) : launch<L, 4, 8>(c, d);
        default: return -1;
    }
}

}  // namespace

// Down + fold of Q4_K / Q5_K / Q6_K experts (wire ids 1, 4, 5) in one launch. Returns -1 when this
// kernel does not serve the call (the caller then takes the two launches), else an LK_* status.
int lk_moe_down_fold(int quant_type, const float* inputs, const void* weights, const int32_t* sorted_token_ids,
                     const int32_t* expert_ids, const float* topk_weights, float* outputs, int num_experts, int topk,
                     int size_m, int size_n, int size_k, const float* down_bias, const float* add_after,
                     hipStream_t stream) {
    if (lk_tune_env("LK_TUNE_DOWN_FOLD_OFF")) return -1;
    if (size_k % 256 != 0 || topk < 1 || topk > 8 || size_m > MAX_PAIRS || size_m % topk != 0) return -1;
    if (((uintptr_t)inputs) & 15) return -1;
    const int tokens = size_m / topk;
    if (tokens < 1 || tokens > 65535) return -1;
    const FoldDims d{num_experts, topk, size_m, size_n, 1, 0};
    const FoldCall c{(const uint8_t*)weights, inputs, sorted_token_ids, expert_ids, topk_weights, down_bias, add_after,
                     outputs, tokens, stream};
    switch (quant_type) {
        case 1: return launch_format<LaneQ4K<false>>(c, d, size_k / 256);
        case 4: return launch_format<LaneQ4K<true>>(c, d, size_k / 256);
        case 5: return launch_format<LaneQ6K>(c, d, size_k / 256);
        default: return -1;
    }
}

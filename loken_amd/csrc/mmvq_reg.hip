// Q4_K mat-vec over ONE activation row whose codes live in registers: the decode step's own
// shape (batch 1, rows of at most 16 super-blocks = 4096 values).
//
// A lane of the Q4_K engine serves one pair of sub-blocks (2p, 2p + 1) of one super-block slot of
// every weight row its wave meets, so the 64 activation codes and the two scales it needs never
// change over the launch: they are 72 contiguous bytes of the Q8_1 row, loaded once straight into
// registers. No LDS image of the activation, no barrier, nothing re-read per row; a wave depends
// on its own loads only. When the activation arrives as f32 the workgroup first quantizes the row
// together (the quantizer's steps, four values per thread) into 4.5 KB of LDS and every lane takes
// its slice from there.
//
// What a lane computes per weight row, and the order in which the lanes' shares are added, are
// those of the staged engine in mmvq_core.h (q4k_pair_share, group_sum), so a row carries the
// same bits whichever engine served it.

#include "mmvq_core.h"

#include <cstdlib>

using namespace mmvq;

namespace {

constexpr int RW = 8;          // waves per workgroup
constexpr int RT = RW * 64;    // threads per workgroup
constexpr int MAX_NB = 16;     // super-blocks per weight row the engine takes
constexpr int LDS_CODES = MAX_NB * 256;              // one quantized row
constexpr int LDS_BYTES = LDS_CODES + MAX_NB * 8 * 4;   // codes, then one f32 scale per Q8_1 block

struct RegArgs {
    const uint8_t* vx[4];
    void* dst[4];
    const float* bias[4];
    int n[4];
    int tile_end[4];   // matrix i owns the tiles [tile_end[i - 1], tile_end[i])
};

// The lane's 64 activation codes and what the share function needs of the two Q8_1 blocks.
struct Slice {
    uint4 a00, a01, a10, a11;   // sub-block 2p values 0..15, 16..31; sub-block 2p + 1 likewise
    float d8a, d8b16;           // d of block 2p; d of block 2p + 1 over 16
    float sa, sb;               // d * (sum of codes) of each block
    int hi_init;                // 128 * (sum of the codes of block 2p + 1)
};

static __device__ __forceinline__ void slice_finish(Slice& s, float d8a, float d8b) {
    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
    const int sum_a = dot16(ones, s.a01, dot16(ones, s.a00, 0));
    const int sum_b = dot16(ones, s.a11, dot16(ones, s.a10, 0));
    s.d8a = d8a;
    s.d8b16 = d8b * 0.0625f;
    s.sa = d8a * (float)sum_a;
    s.sb = d8b * (float)sum_b;
    s.hi_init = 128 * sum_b;
}

// One weight row's loads of a lane: the 16-byte block header and the 32 bytes of its pair.
struct RowFrag {
    uint4 h, q0, q1;
};
static __device__ __forceinline__ void row_load(RowFrag& f, gbytes_t row, uint32_t hdr_off, uint32_t qs_off) {
    const uint8_t* bp = (const uint8_t*)row;
    f.h = *(const uint4*)(bp + hdr_off);
    f.q0 = *(const uint4*)(bp + qs_off);
    f.q1 = *(const uint4*)(bp + qs_off + 16);
}
static __device__ __forceinline__ float row_share(const RowFrag& f, const Slice& s, const Q4KScaleSel& sel, bool valid,
                                                  uint32_t flip) {
    uint32_t sc, mn;
    sel.unpack(f.h.y, f.h.z, f.h.w, sc, mn);
    const uint32_t dd = valid ? f.h.x : 0u;   // a lane past the row's end adds nothing
    int d_lo = 0, x_hi = s.hi_init;
    q4k_dots_biased(f.q0, s.a00, s.a10, flip, d_lo, x_hi);
    q4k_dots_biased(f.q1, s.a01, s.a11, flip, d_lo, x_hi);
    return q4k_pair_share(f16_bits_to_f32(dd & 0xFFFFu), f16_bits_to_f32(dd >> 16), (float)(sc & 0xFFu), (float)(sc >> 8),
                          (float)(mn & 0xFFu), (float)(mn >> 8), s.d8a, s.d8b16, s.sa, s.sb, (float)d_lo, (float)x_hi);
}

// The activation row into the lane's slice, with `first_loads` (the wave's first weight loads)
// issued behind the activation's loads and ahead of everything that waits for them: loads return in
// issue order, so the small activation must go first and must not wait for weights.
// unit = 4 * slot + p: which 72 bytes of the Q8_1 row (64 bytes of the LDS image) are the lane's.
// B activation rows, `act_stride` bytes apart, into B slices (the f32 form: B images of LDS_BYTES).
template <bool ACT_F32, int B, class First>
static __device__ __forceinline__ void slice_load(Slice (&s)[B], gbytes_t act, size_t act_stride, int nb, int unit, bool valid,
                                                  uint8_t* lds, First&& first_loads) {
#pragma clang fp contract(off)
    if (!ACT_F32) {
        // (cast back from the global address space: the compiler keeps track of where it came from)
        uint32_t head0[B], head1[B];
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const uint8_t* ap = (const uint8_t*)(act + b * act_stride + (valid ? 72 * unit : 0));
            head0[b] = *(const uint32_t*)ap;
            s[b].a00 = *(const uint4_a4*)(ap + 4);
            s[b].a01 = *(const uint4_a4*)(ap + 20);
            head1[b] = *(const uint32_t*)(ap + 36);
            s[b].a10 = *(const uint4_a4*)(ap + 40);
            s[b].a11 = *(const uint4_a4*)(ap + 56);
        }
        load_fence((const void*)lds);
        first_loads();
        load_fence((const void*)lds);
#pragma unroll
        for (int b = 0; b < B; ++b) slice_finish(s[b], f16_bits_to_f32(head0[b] & 0xFFFFu), f16_bits_to_f32(head1[b] & 0xFFFFu));
        return;
    }
    // f32 row: item t is four values, eight consecutive items (lanes) are one Q8_1 block
    const int items = nb * 64;
    float4 v[B][2];
#pragma unroll
    for (int b = 0; b < B; ++b)
#pragma unroll
        for (int u = 0; u < 2; ++u)
            v[b][u] = *(const float4*)(const uint8_t*)(act + b * act_stride + 16 * min((int)threadIdx.x + u * RT, items - 1));
    load_fence((const void*)lds);
    first_loads();
    load_fence((const void*)lds);
#pragma unroll
    for (int b = 0; b < B; ++b) {
        uint8_t* img = lds + b * LDS_BYTES;
        float* scales = (float*)(img + LDS_CODES);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int item = threadIdx.x + u * RT;
            if (item < items) {   // whole waves: items is a multiple of 64
                const float4 x = v[b][u];
                const float amax = max8(fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w))));
                const float d = amax / 127.0f;
                const float inv = d != 0.0f ? 1.0f / d : 0.0f;
                const int q0 = (int)roundf(x.x * inv), q1 = (int)roundf(x.y * inv);
                const int q2 = (int)roundf(x.z * inv), q3 = (int)roundf(x.w * inv);
                *(uint32_t*)(img + 4 * item) = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) |
                                               ((uint32_t)(q2 & 0xFF) << 16) | ((uint32_t)(q3 & 0xFF) << 24);
                if ((item & 7) == 0) scales[item >> 3] = __half2float(__float2half_rn(d));
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < B; ++b) {
        const uint8_t* img = lds + b * LDS_BYTES;
        const uint8_t* ap = img + (valid ? 64 * unit : 0);
        s[b].a00 = *(const uint4*)(ap);
        s[b].a01 = *(const uint4*)(ap + 16);
        s[b].a10 = *(const uint4*)(ap + 32);
        s[b].a11 = *(const uint4*)(ap + 48);
        const float2 dd = *(const float2*)((const float*)(img + LDS_CODES) + (valid ? 2 * unit : 0));
        slice_finish(s[b], dd.x, dd.y);
    }
}

static __device__ __forceinline__ void store_out(void* dst, int dst_type, size_t at, float v) {
    if (dst_type == LK_TYPE_F32) ((float*)dst)[at] = v;
    else if (dst_type == LK_TYPE_F16) ((__half*)dst)[at] = __float2half_rn(v);
    else ((__hip_bfloat16*)dst)[at] = __float2bfloat16(v);
}

// Lane geometry: RP weight rows side by side in a wave pass, each in 64 / RP lanes = 16 / RP
// super-block slots of four lanes.
template <int RP>
struct Geo {
    static constexpr int S = 16 / RP, GROUP = 64 / RP;
    int lane, p, slot, rp, unit;
    bool valid;
    uint32_t hdr_off, qs_off;
    __device__ __forceinline__ Geo(int nb) {
        lane = threadIdx.x & 63;
        p = lane & 3;
        const int lb = lane >> 2;
        slot = lb & (S - 1);
        rp = lb / S;
        unit = 4 * slot + p;
        valid = slot < nb;
        hdr_off = (valid ? slot : nb - 1) * Q4K_BYTES;   // past the row's end: re-read its last block
        qs_off = hdr_off + 16 + 32 * p;
    }
};

// Up to four matrices over one activation row. A tile is R * RP consecutive rows of one matrix;
// wave g of the grid takes tiles g, g + waves, ...
// B: activation rows (1 or 2), act_stride bytes apart; their outputs dst_stride elements apart.
template <int R, int RP, bool ACT_F32, int B>
__global__ __launch_bounds__(RT) void q4k_reg_kernel(RegArgs a, const uint8_t* __restrict__ act, int nb, int dst_type,
                                                     int waves, int act_stride, int dst_stride) {
    __shared__ __align__(16) uint8_t lds[ACT_F32 ? B * LDS_BYTES : 16];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int TR = R * RP;
    uint32_t flip = 0x80808080u;
    asm volatile("" : "+v"(flip));   // kept in a register: the bit instruction takes no literal

    // Every argument the first loads need arrives in ONE round of scalar loads: each field is read
    // at a fixed index here and picked by mask later (an index computed from the tile, or a read
    // under a branch, costs further dependent rounds in front of the first weight load).
    uintptr_t vxs[4], dsts[4], biases[4], act_bits = (uintptr_t)act;
    int ns[4], ends[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        vxs[i] = (uintptr_t)a.vx[i];
        dsts[i] = (uintptr_t)a.dst[i];
        biases[i] = (uintptr_t)a.bias[i];
        ns[i] = a.n[i];
        ends[i] = a.tile_end[i];
    }
    asm volatile("" : "+s"(vxs[0]), "+s"(vxs[1]), "+s"(vxs[2]), "+s"(vxs[3]), "+s"(ns[0]), "+s"(ns[1]), "+s"(ns[2]), "+s"(ns[3]),
                 "+s"(ends[0]), "+s"(ends[1]), "+s"(ends[2]), "+s"(ends[3]), "+s"(act_bits), "+s"(nb), "+s"(dst_type), "+s"(waves));
    asm volatile("" : "+s"(dsts[0]), "+s"(dsts[1]), "+s"(dsts[2]), "+s"(dsts[3]), "+s"(biases[0]), "+s"(biases[1]),
                 "+s"(biases[2]), "+s"(biases[3]));
    const gbytes_t act_g = to_gbytes((uint64_t)act_bits);
    const Geo<RP> g(nb);
    const Q4KScaleSel sel(g.p);
    const int total = ends[3], step = (int)gridDim.x * waves;
    const size_t row_stride = (size_t)nb * Q4K_BYTES;
    // The matrix the wave's current tile belongs to. A wave's tiles only move forward, so this is
    // worked out again only when a tile passes the end of the current matrix (never, with one matrix).
    gbytes_t cur_vx;
    uintptr_t cur_dst, cur_bias;
    int cur_n, cur_begin, cur_end;
    auto relocate = [&](int t) {
        const int m = t >= ends[2] ? 3 : t >= ends[1] ? 2 : t >= ends[0] ? 1 : 0;
        uintptr_t vx_bits = 0, dst_bits = 0, bias_bits = 0;
        uint32_t n_bits = 0, begin_bits = 0, end_bits = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t pick = 0u - (uint32_t)(m == i);
            const uintptr_t pick64 = (uintptr_t)(int64_t)(int32_t)pick;
            vx_bits |= vxs[i] & pick64;
            dst_bits |= dsts[i] & pick64;
            bias_bits |= biases[i] & pick64;
            n_bits |= (uint32_t)ns[i] & pick;
            begin_bits |= (uint32_t)(i ? ends[i - 1] : 0) & pick;
            end_bits |= (uint32_t)ends[i] & pick;
        }
        cur_vx = to_gbytes((uint64_t)vx_bits);
        cur_dst = dst_bits;
        cur_bias = bias_bits;
        cur_n = (int)n_bits;
        cur_begin = (int)begin_bits;
        cur_end = (int)end_bits;
    };
    RowFrag f[R];
    auto load = [&](int t) {
        const int row0 = (t - cur_begin) * TR + g.rp * R;
#pragma unroll
        for (int r = 0; r < R; ++r) row_load(f[r], cur_vx + min(row0 + r, cur_n - 1) * row_stride, g.hdr_off, g.qs_off);
    };

    int t = (int)blockIdx.x * waves + wave;
    Slice s[B];
    // (a wave without a tile loads the last one rather than nothing: the count of loads ahead of
    // the weights stays the same for every wave)
    relocate(min(t, total - 1));
    slice_load<ACT_F32, B>(s, act_g, (size_t)act_stride, nb, g.unit, g.valid, lds, [&] { load(min(t, total - 1)); });
    const bool odd = g.lane & 1;
    while (t < total) {
        void* dst = (void*)(uint8_t*)to_gbytes((uint64_t)cur_dst);
        const float* bias = (const float*)to_gbytes((uint64_t)cur_bias);
        const int row = (t - cur_begin) * TR + g.rp * R, n = cur_n;   // the lane group's first row of the tile
#pragma unroll
        for (int b = 0; b < B; ++b) {
            if (R == 2) {
                // even lanes end with the first row's total, odd lanes with the second's
                float v = group_sum2<Geo<RP>::GROUP>(row_share(f[0], s[b], sel, g.valid, flip),
                                                     row_share(f[R - 1], s[b], sel, g.valid, flip), odd);
                const int mine = row + (int)odd;
                if ((g.lane & (Geo<RP>::GROUP - 1)) < 2 && mine < n) {
                    if (bias) v += bias[mine];
                    store_out(dst, dst_type, (size_t)b * dst_stride + mine, v);
                }
            } else {
                float v = group_sum<Geo<RP>::GROUP>(row_share(f[0], s[b], sel, g.valid, flip));
                if ((g.lane & (Geo<RP>::GROUP - 1)) == 0 && row < n) {
                    if (bias) v += bias[row];
                    store_out(dst, dst_type, (size_t)b * dst_stride + row, v);
                }
            }
        }
        t += step;
        if (t < total) {
            if (t >= cur_end) relocate(t);
            load(t);
        }
    }
}

static __device__ __forceinline__ float act_silu(float g) { return g / (1.0f + expf(-g)); }
static __device__ __forceinline__ float act_gelu_tanh(float g) {
    return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * g * (1.0f + 0.044715f * g * g)));
}

// The gate / up pair: a tile is RP rows (one per lane group) of both matrices; the two shares of a
// row are summed together (even lanes gate, odd lanes up) and lane 0 of the group combines them.
// Q81_OUT: a workgroup owns whole blocks of 32 consecutive rows (wave w rows 4w .. 4w + 3),
// the 32 results meet in LDS and eight lanes write them as one Q8_1 block with the quantizer's steps.
// (the two-row forms with Q8_1 output take 135-169 registers, one workgroup per CU; bounded to 128 they
// spill and measured slower: Llama step at two rows 1.70 against 1.62 ms)
template <int RP, bool ACT_F32, bool Q81_OUT, int B>
__global__ __launch_bounds__(RT) void q4k_reg_pair_kernel(const uint8_t* __restrict__ gate, const uint8_t* __restrict__ up,
                                                          const uint8_t* __restrict__ act, void* __restrict__ dst, int nb,
                                                          int n, int dst_type, int act_fn, int waves, int act_stride,
                                                          int dst_stride) {
#pragma clang fp contract(off)
    __shared__ __align__(16) uint8_t lds[(ACT_F32 ? B * LDS_BYTES : 0) + (Q81_OUT ? B * 2 * 32 * 4 : 16)];
    float* meet = (float*)(lds + (ACT_F32 ? B * LDS_BYTES : 0));   // [B][2][32]: two blocks in flight
    const Geo<RP> g(nb);
    const Q4KScaleSel sel(g.p);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t row_stride = (size_t)nb * Q4K_BYTES;
    const gbytes_t wg = to_gbytes(gate), wu = to_gbytes(up);
    uint32_t flip = 0x80808080u;
    asm volatile("" : "+v"(flip));
    const bool odd = g.lane & 1;
    RowFrag fg, fu;
    auto load = [&](int row) {
        const size_t at = (size_t)min(row, n - 1) * row_stride;
        row_load(fg, wg + at, g.hdr_off, g.qs_off);
        row_load(fu, wu + at, g.hdr_off, g.qs_off);
    };
    // the row's value in lane 0 of its group
    auto value = [&](const Slice& s) {
        const float both = group_sum2<Geo<RP>::GROUP>(row_share(fg, s, sel, g.valid, flip), row_share(fu, s, sel, g.valid, flip), odd);
        const float u = dpp_f32<0xB1>(both);   // the odd neighbour's total
        return (act_fn == 0 ? act_silu(both) : act_gelu_tanh(both)) * u;
    };
    Slice s[B];
    if (!Q81_OUT) {
        // tiles of RP rows, wave-strided
        const int tiles = (n + RP - 1) / RP, step = (int)gridDim.x * waves;
        int t = (int)blockIdx.x * waves + wave;
        slice_load<ACT_F32, B>(s, to_gbytes(act), (size_t)act_stride, nb, g.unit, g.valid, lds,
                               [&] { load(min(t, tiles - 1) * RP + g.rp); });
        while (t < tiles) {
            const int row = t * RP + g.rp;
#pragma unroll
            for (int b = 0; b < B; ++b) {
                const float v = value(s[b]);
                if ((g.lane & (Geo<RP>::GROUP - 1)) == 0 && row < n) store_out(dst, dst_type, (size_t)b * dst_stride + row, v);
            }
            t += step;
            if (t < tiles) load(t * RP + g.rp);
        }
        return;
    }
    // A wave's four rows of a block go through in PASSES = 4 / RP passes of RP rows side by side, with
    // the loads of D passes in flight (two rows of both matrices at RP = 1: more would cost the second
    // workgroup per CU its registers): a pass's loads go out D passes ahead, into the registers of the
    // pass just consumed, across block boundaries too.
    constexpr int PASSES = 4 / RP, D = PASSES < 2 ? PASSES : 2;
    const int blocks = n / 32;
    int b = blockIdx.x;
    RowFrag bg[D], bu[D];
    auto load_pass = [&](int slot, int blk, int i) {
        const size_t at = (size_t)min(32 * blk + 4 * wave + i * RP + g.rp, n - 1) * row_stride;
        row_load(bg[slot], wg + at, g.hdr_off, g.qs_off);
        row_load(bu[slot], wu + at, g.hdr_off, g.qs_off);
    };
    slice_load<ACT_F32, B>(s, to_gbytes(act), (size_t)act_stride, nb, g.unit, g.valid, lds, [&] {
#pragma unroll
        for (int i = 0; i < D; ++i) load_pass(i, min(b, blocks - 1), i);
    });
    int half = 0;
    for (; b < blocks; b += gridDim.x) {
        float val[B][PASSES];
        const int nb_next = b + (int)gridDim.x;
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
#pragma unroll
            for (int r = 0; r < B; ++r) {
                const float both = group_sum2<Geo<RP>::GROUP>(row_share(bg[i % D], s[r], sel, g.valid, flip),
                                                              row_share(bu[i % D], s[r], sel, g.valid, flip), odd);
                const float u = dpp_f32<0xB1>(both);   // the odd neighbour's total
                val[r][i] = (act_fn == 0 ? act_silu(both) : act_gelu_tanh(both)) * u;
            }
            if (i + D < PASSES) load_pass(i % D, b, i + D);
            else if (nb_next < blocks) load_pass(i % D, nb_next, i + D - PASSES);
        }
        if ((g.lane & (Geo<RP>::GROUP - 1)) == 0) {
#pragma unroll
            for (int r = 0; r < B; ++r)
#pragma unroll
                for (int i = 0; i < PASSES; ++i) meet[(r * 2 + half) * 32 + 4 * wave + i * RP + g.rp] = val[r][i];
        }
        __syncthreads();   // every wave of the workgroup has delivered its four
        if (wave == 0 && g.lane < 8 * B) {
            const int l8 = g.lane & 7, r = g.lane >> 3;
            const float4 v = *(const float4*)(meet + (r * 2 + half) * 32 + 4 * l8);
            const float amax = max8(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
            const float d = amax / 127.0f;
            const float inv = d != 0.0f ? 1.0f / d : 0.0f;
            const int q0 = (int)roundf(v.x * inv), q1 = (int)roundf(v.y * inv);
            const int q2 = (int)roundf(v.z * inv), q3 = (int)roundf(v.w * inv);
            int quad;
            const int sum = sum8(q0 + q1 + q2 + q3, quad);
            uint32_t* out = (uint32_t*)dst + ((size_t)r * dst_stride + b) * 9;
            out[1 + l8] = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
                          ((uint32_t)(q3 & 0xFF) << 24);
            if (l8 == 0) {
                const uint32_t dh = __half_as_ushort(__float2half_rn(d));
                float scaled_sum = (float)sum * d;
                asm volatile("" : "+v"(scaled_sum));   // two roundings, as the quantizer's
                out[0] = dh | ((uint32_t)__half_as_ushort(__float2half_rn(scaled_sum)) << 16);
            }
        }
        half ^= 1;   // the next block meets in the other buffer: a wave may run one block ahead
    }
}

// The gate / up pair per routed (token, expert) pair of an MoE layer: grid.y names the pair, whose
// expert picks the two slabs, whose token picks the f32 activation row and whose slot picks the
// output row (the conventions of loken_moe_gemm_gguf_gate_up_silu_mul, cuda/moe/moe_gguf.cu:896-1060
// of the reference). Everything else is the pair kernel above.
struct RegMoeArgs {
    const int32_t* sorted_token_ids;
    const int32_t* expert_ids;
    int experts, topk, pairs;
    int64_t slab_bytes;
    LkGateAct act;
};
template <int RP>
__global__ __launch_bounds__(RT) void q4k_reg_moe_pair_kernel(const uint8_t* __restrict__ gate, const uint8_t* __restrict__ up,
                                                              const float* __restrict__ acts, float* __restrict__ out, int nb,
                                                              int n, RegMoeArgs m, int waves) {
#pragma clang fp contract(off)
    __shared__ __align__(16) uint8_t lds[LDS_BYTES];
    const int pair = blockIdx.y;
    const int slot = m.sorted_token_ids[pair], e = m.expert_ids[pair];
    asm volatile("" ::"s"(slot), "s"(e), "s"(m.pairs), "s"(m.experts), "s"(m.topk), "s"(m.slab_bytes), "s"(gate), "s"(up),
                 "s"(acts), "s"(out), "s"(nb), "s"(n), "s"(waves), "s"(m.act.kind));
    if (slot < 0 || slot >= m.pairs || e < 0 || e >= m.experts) return;   // a pair the routing leaves out writes nothing
    const Geo<RP> g(nb);
    const Q4KScaleSel sel(g.p);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t row_stride = (size_t)nb * Q4K_BYTES;
    const gbytes_t wg = to_gbytes(gate) + (int64_t)e * m.slab_bytes, wu = to_gbytes(up) + (int64_t)e * m.slab_bytes;
    const gbytes_t act = to_gbytes(acts) + (size_t)(slot / m.topk) * nb * (256 * sizeof(float));
    float* dst = out + (size_t)slot * n;
    uint32_t flip = 0x80808080u;
    asm volatile("" : "+v"(flip));
    const bool odd = g.lane & 1;
    RowFrag fg, fu;
    auto load = [&](int row) {
        const size_t at = (size_t)min(row, n - 1) * row_stride;
        row_load(fg, wg + at, g.hdr_off, g.qs_off);
        row_load(fu, wu + at, g.hdr_off, g.qs_off);
    };
    const int tiles = (n + RP - 1) / RP, step = (int)gridDim.x * waves;
    int t = (int)blockIdx.x * waves + wave;
    Slice s[1];
    slice_load<true, 1>(s, act, 0, nb, g.unit, g.valid, lds, [&] { load(min(t, tiles - 1) * RP + g.rp); });
    while (t < tiles) {
        const int row = t * RP + g.rp;
        const float both = group_sum2<Geo<RP>::GROUP>(row_share(fg, s[0], sel, g.valid, flip), row_share(fu, s[0], sel, g.valid, flip), odd);
        const float u = dpp_f32<0xB1>(both);   // the odd neighbour's total
        if ((g.lane & (Geo<RP>::GROUP - 1)) == 0 && row < n) dst[row] = lk_gated(m.act, both, u, (size_t)e * n + row);
        t += step;
        if (t < tiles) load(t * RP + g.rp);
    }
}

// Launch shape. f32 activation: workgroups of RW waves (the row is quantized once per workgroup), two
// per CU. Q8_1 activation: nothing is shared inside a workgroup, four waves each, four per CU.
// LK_TUNE_REG_WAVES / LK_TUNE_REG_WGS_PER_CU override both for measurement runs.
struct Shape {
    int waves, cap;   // waves per workgroup, most workgroups launched
};
static Shape shape_for(bool act_f32) {
    const int forced_waves = lk_tune_env("LK_TUNE_REG_WAVES"), forced_per_cu = lk_tune_env("LK_TUNE_REG_WGS_PER_CU");
    const int waves = act_f32 ? RW : (forced_waves == 4 || forced_waves == 8 ? forced_waves : 4);
    const int per_cu = forced_per_cu > 0 ? forced_per_cu : 16 / waves;
    return Shape{waves, lk_device().cus * per_cu};
}

template <int R, int RP, int B>
static int launch_multi(const LkRegMulti& m, const void* act, int act_f32, int nb, int dst_type, int act_stride, int dst_stride,
                        hipStream_t s) {
    RegArgs a{};
    int total = 0;
    for (int i = 0; i < 4; ++i) {
        if (i < m.count) {
            a.vx[i] = m.vx[i];
            a.dst[i] = m.dst[i];
            a.bias[i] = m.bias[i];
            a.n[i] = m.n[i];
            total += (m.n[i] + R * RP - 1) / (R * RP);
        }
        a.tile_end[i] = total;
    }
    const Shape sh = shape_for(act_f32 != 0);
    const int need = (total + sh.waves - 1) / sh.waves;
    const int forced_grid = lk_tune_env("LK_TUNE_REG_GRID");
    const dim3 grid(forced_grid > 0 ? (forced_grid < need ? forced_grid : need) : need < sh.cap ? need : sh.cap), block(sh.waves * 64);
    if (act_f32)
        hipLaunchKernelGGL((q4k_reg_kernel<R, RP, true, B>), grid, block, 0, s, a, (const uint8_t*)act, nb, dst_type, sh.waves,
                           act_stride, dst_stride);
    else
        hipLaunchKernelGGL((q4k_reg_kernel<R, RP, false, B>), grid, block, 0, s, a, (const uint8_t*)act, nb, dst_type, sh.waves,
                           act_stride, dst_stride);
    return lk_launch_status();
}

template <int RP, int B>
static int launch_pair(const uint8_t* gate, const uint8_t* up, const void* act, int act_f32, void* dst, int dst_type,
                       bool q81, int nb, int n, int act_fn, int act_stride, int dst_stride, hipStream_t s) {
    const uint8_t* y = (const uint8_t*)act;
    if (q81) {
        // a workgroup of RW waves per block of 32 rows
        const Shape sh = shape_for(true);
        const int blocks = n / 32, cap = sh.cap;
        const dim3 grid(blocks < cap ? blocks : cap);
        if (act_f32)
            hipLaunchKernelGGL((q4k_reg_pair_kernel<RP, true, true, B>), grid, dim3(RT), 0, s, gate, up, y, dst, nb, n, dst_type, act_fn, sh.waves,
                               act_stride, dst_stride);
        else
            hipLaunchKernelGGL((q4k_reg_pair_kernel<RP, false, true, B>), grid, dim3(RT), 0, s, gate, up, y, dst, nb, n, dst_type, act_fn, sh.waves,
                               act_stride, dst_stride);
        return lk_launch_status();
    }
    const Shape sh = shape_for(act_f32 != 0);
    const int tiles = (n + RP - 1) / RP, need = (tiles + sh.waves - 1) / sh.waves;
    const dim3 grid(need < sh.cap ? need : sh.cap), block(sh.waves * 64);
    if (act_f32)
        hipLaunchKernelGGL((q4k_reg_pair_kernel<RP, true, false, B>), grid, block, 0, s, gate, up, y, dst, nb, n, dst_type, act_fn, sh.waves,
                           act_stride, dst_stride);
    else
        hipLaunchKernelGGL((q4k_reg_pair_kernel<RP, false, false, B>), grid, block, 0, s, gate, up, y, dst, nb, n, dst_type, act_fn, sh.waves,
                           act_stride, dst_stride);
    return lk_launch_status();
}

}  // namespace

bool lk_q4k_reg_serves(int nb) {
    const int off = lk_tune_env("LK_TUNE_NO_REG");   // measurement runs: the staged engine for everything
    return nb >= 1 && nb <= MAX_NB && !off;
}

template <int B>
static int multi_rows(const LkRegMulti& m, const void* act, int act_f32, int nb, int dst_type, int act_bytes, int dst_stride,
                      hipStream_t stream) {
    const int rp = q4k_rows_per_pass(nb);
    // Two rows per wave tile while every wave still gets at most one tile (the launch is one round
    // of loads and a tail: fewer, fatter waves), one row per tile when waves stream several.
    int rows = 0;
    for (int i = 0; i < m.count; ++i) rows += m.n[i];
    const int forced = lk_tune_env("LK_TUNE_REG_R");
    const Shape sh = shape_for(act_f32 != 0);
    // (from f32 rows the bound is one workgroup per CU: q + k + v of a Llama-sized layer, 6144 rows, is
    // faster as single rows over two workgroups per CU, 5.7 against 6.1 us; o, 4096 rows, as pairs)
    const int waves_at_once = (act_f32 ? lk_device().cus : sh.cap) * sh.waves;
    // (rows short enough to go side by side already give a wave two or four rows per pass: two such
    // tiles per wave measured slower, Qwen3-1.7B step 0.598 against 0.586 ms)
    const bool two = forced ? forced == 2 : rp == 1 && rows <= waves_at_once * 2;
    switch (rp) {
        case 1: return two ? launch_multi<2, 1, B>(m, act, act_f32, nb, dst_type, act_bytes, dst_stride, stream)
                           : launch_multi<1, 1, B>(m, act, act_f32, nb, dst_type, act_bytes, dst_stride, stream);
        case 2: return two ? launch_multi<2, 2, B>(m, act, act_f32, nb, dst_type, act_bytes, dst_stride, stream)
                           : launch_multi<1, 2, B>(m, act, act_f32, nb, dst_type, act_bytes, dst_stride, stream);
        default: return launch_multi<1, 4, B>(m, act, act_f32, nb, dst_type, act_bytes, dst_stride, stream);
    }
}

int lk_q4k_reg_multi(const LkRegMulti& m, const void* act, int act_f32, int nb, int dst_type, int batch, int act_stride,
                     int dst_stride, hipStream_t stream) {
    if (!lk_q4k_reg_serves(nb) || m.count < 1 || m.count > 4 || batch < 1 || batch > LK_REG_MAX_BATCH) return LK_ERR_ARG;
    const int act_bytes = act_stride * (act_f32 ? (int)sizeof(float) : Q81_BYTES);
    return batch == 1 ? multi_rows<1>(m, act, act_f32, nb, dst_type, act_bytes, dst_stride, stream)
                      : multi_rows<2>(m, act, act_f32, nb, dst_type, act_bytes, dst_stride, stream);
}

template <int RP>
static int launch_moe_pair(const uint8_t* gate, const uint8_t* up, const float* acts, float* out, int nb, int n,
                           const RegMoeArgs& m, hipStream_t s) {
    const int forced_per_cu = lk_tune_env("LK_TUNE_REG_MOE_PER_CU");
    const int tiles = (n + RP - 1) / RP, need = (tiles + RW - 1) / RW;
    int share = lk_device().cus * (forced_per_cu > 0 ? forced_per_cu : 4) / m.pairs;
    if (share < 1) share = 1;
    const dim3 grid(need < share ? need : share, m.pairs);
    hipLaunchKernelGGL((q4k_reg_moe_pair_kernel<RP>), grid, dim3(RT), 0, s, gate, up, acts, out, nb, n, m, RW);
    return lk_launch_status();
}

int lk_q4k_reg_moe_pair(const uint8_t* gate, const uint8_t* up, const float* acts, const int32_t* sorted_token_ids,
                        const int32_t* expert_ids, float* out, int experts, int topk, int pairs, int n, int nb,
                        int64_t slab_bytes, const LkGateAct& act, hipStream_t stream) {
    const int off = lk_tune_env("LK_TUNE_NO_REG_MOE");
    if (off || !lk_q4k_reg_serves(nb) || pairs < 1 || pairs > 65535 || n < 1) return -1;
    if ((((uintptr_t)gate) | ((uintptr_t)up) | ((uintptr_t)acts)) & 15) return -1;
    const RegMoeArgs m{sorted_token_ids, expert_ids, experts, topk, pairs, slab_bytes, act};
    switch (q4k_rows_per_pass(nb)) {
        case 1: return launch_moe_pair<1>(gate, up, acts, out, nb, n, m, stream);
        case 2: return launch_moe_pair<2>(gate, up, acts, out, nb, n, m, stream);
        default: return launch_moe_pair<4>(gate, up, acts, out, nb, n, m, stream);
    }
}

template <int B>
static int pair_rows(const uint8_t* gate, const uint8_t* up, const void* act, int act_f32, void* dst, int dst_type, bool dst_q8_1,
                     int nb, int n, int act_fn, int act_bytes, int dst_stride, hipStream_t stream) {
    switch (q4k_rows_per_pass(nb)) {
        case 1: return launch_pair<1, B>(gate, up, act, act_f32, dst, dst_type, dst_q8_1, nb, n, act_fn, act_bytes, dst_stride, stream);
        case 2: return launch_pair<2, B>(gate, up, act, act_f32, dst, dst_type, dst_q8_1, nb, n, act_fn, act_bytes, dst_stride, stream);
        default: return launch_pair<4, B>(gate, up, act, act_f32, dst, dst_type, dst_q8_1, nb, n, act_fn, act_bytes, dst_stride, stream);
    }
}

int lk_q4k_reg_pair(const uint8_t* gate, const uint8_t* up, const void* act, int act_f32, void* dst, int dst_type,
                    bool dst_q8_1, int nb, int n, int act_fn, int batch, int act_stride, int dst_stride, hipStream_t stream) {
    if (!lk_q4k_reg_serves(nb) || n < 1 || (dst_q8_1 && n % 32 != 0) || batch < 1 || batch > LK_REG_MAX_BATCH) return LK_ERR_ARG;
    const int act_bytes = act_stride * (act_f32 ? (int)sizeof(float) : Q81_BYTES);
    return batch == 1 ? pair_rows<1>(gate, up, act, act_f32, dst, dst_type, dst_q8_1, nb, n, act_fn, act_bytes, dst_stride, stream)
                      : pair_rows<2>(gate, up, act, act_f32, dst, dst_type, dst_q8_1, nb, n, act_fn, act_bytes, dst_stride, stream);
}

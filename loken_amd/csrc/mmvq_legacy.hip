// Mat-vec for the 32-value nibble formats Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, MXFP4 and the two-bit
// K-quants Q2_K, Q3_K (and IQ4_XS) against Q8_1 activation rows.
//
// Formats as loken states them (src/tensor/quant_cpu/format/q4_0.rs, q4_1.rs, q5_0.rs, q5_1.rs): byte
// j of `qs` holds value j in its low nibble and value j + 16 in its high one; the five-bit formats
// keep bit v of the little-endian word `qh` as value v's fifth bit. Q4_0 {d, qs} and Q5_0 {d, qh,
// qs} mean (code - 8 / 16) * d; Q4_1 {d, m, qs} and Q5_1 {d, m, qh, qs} mean code * d + m.
// Per block the product with a Q8_1 block {d8, codes a} is, as the reference's mat-vec forms it
// (cuda/moe/gguf.cuh:392-441: total_biased_codes, total_with_minimum), with the sum of the
// activation codes taken as the integer it is (as every kernel of this library takes it):
//     d * d8 * (sum code * a - bias * sum a)            Q4_0 (bias 8), Q5_0 (bias 16)
//     d * d8 * (sum code * a) + m * (d8 * sum a)        Q4_1, Q5_1
// IQ4_NL {d, qs} and MXFP4 {e, qs} pack their nibbles the same way, but a code names a level of a
// 16-entry int8 table (src/tensor/quant_cpu/format/iq4_nl.rs:11-13; KVALUES_MXFP4 and the E8M0 scale
// 0.5 * 2^(e - 127), src/tensor/quant_cpu/blocks.rs:24-42): scale * d8 * (sum level * a). Four
// levels at a time come out of the table with two byte permutes (entries 0..7, 8..15) and a select
// on the code's top bit.
// Replaces kernels `mmvq_gguf_{q4_0,q4_1,q5_0,q5_1,iq4_nl,mxfp4}_{f32,f16,bf16}_plain_cuda{1..8}`
// (src/inference/cuda/mmvq_gguf.cu:338-363) behind lk_mmvq.
//
// Shape: a wave owns a weight row; its lanes walk the row's blocks 64 at a time (consecutive lanes
// read consecutive 18..24-byte blocks, so a wave's loads cover one contiguous run), each lane forms
// its block's integers against every activation row of the batch and the wave folds once per row.
// The workgroup first copies the activation rows into LDS (codes in two planes of 16-byte halves,
// scales as f32, the halves' code sums as integers), so the load unit carries weight bytes only: a
// two-bit format has four activation bytes to the weight byte. Rows too long for 48 KB of LDS are
// read from memory block by block instead. These formats are the long tail of the reference's
// table; the kernels are plain statements without the register pipelines of the K-quant engines.

#include "legacy_blocks.h"
#include "codebook_blocks.h"

namespace {

constexpr int LWG = 256, LWAVES = 4;

// One Q8_1 block of the activation as the dots take it: the two halves of its codes, its scale and
// the integer sums of the halves.
struct ActBlock {
    uint4 lo, hi;
    float d8;
    int sum0, sum1;
};

static __device__ __forceinline__ ActBlock act_from_memory(const uint8_t* __restrict__ yb) {
    ActBlock a;
    a.lo = *(const uint4_a4*)(yb + 4);
    a.hi = *(const uint4_a4*)(yb + 20);
    a.d8 = f16_bits_to_f32(*(const uint16_t*)yb);
    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
    a.sum0 = dot16(ones, a.lo, 0);
    a.sum1 = dot16(ones, a.hi, 0);
    return a;
}

// LDS copy of `batch` activation rows of `k32` blocks: plane of low halves, plane of high halves
// (16 bytes per block each, so consecutive lanes read consecutive 16-byte slots), the scales as
// f32, the two sums packed as 16-bit halves of a dword (|sum| <= 16 * 127).
constexpr int ACT_LDS_PER_BLOCK = 40;

static __device__ __forceinline__ void stage_acts(uint8_t* lds, const uint8_t* __restrict__ vy, int batch, int k32,
                                                  int stride_col_y) {
    const int total = batch * k32;
    for (int i = threadIdx.x; i < total; i += LWG) {
        const int c = i / k32, b = i - c * k32;
        const ActBlock a = act_from_memory(vy + ((size_t)c * stride_col_y + b) * Q81_BYTES);
        ((uint4*)lds)[i] = a.lo;
        ((uint4*)lds)[total + i] = a.hi;
        ((float*)(lds + (size_t)total * 32))[i] = a.d8;
        ((int*)(lds + (size_t)total * 36))[i] = (a.sum0 & 0xFFFF) | (a.sum1 << 16);
    }
    __syncthreads();
}

template <bool STAGED>
static __device__ __forceinline__ ActBlock act_block(const uint8_t* lds, const uint8_t* __restrict__ vy, int total, int k32,
                                                     int stride_col_y, int c, int b) {
    if (!STAGED) return act_from_memory(vy + ((size_t)c * stride_col_y + b) * Q81_BYTES);
    const int i = c * k32 + b;
    ActBlock a;
    a.lo = ((const uint4*)lds)[i];
    a.hi = ((const uint4*)lds)[total + i];
    a.d8 = ((const float*)(lds + (size_t)total * 32))[i];
    const int packed = ((const int*)(lds + (size_t)total * 36))[i];
    a.sum0 = (packed << 16) >> 16;
    a.sum1 = packed >> 16;
    return a;
}

// The block's integer against one Q8_1 block: sum (code - bias) * a.
static __device__ __forceinline__ int block_dot(const uint4& lo, const uint4& hi, const ActBlock& a, int bias) {
    return dot16(hi, a.hi, dot16(lo, a.lo, 0)) - bias * (a.sum0 + a.sum1);
}

template <int ID, int B, typename T, bool STAGED>
__global__ __launch_bounds__(LWG) void mmvq_legacy_kernel(const uint8_t* __restrict__ vx, const uint8_t* __restrict__ vy,
                                                          T* __restrict__ dst, const float* __restrict__ bias, int nb, int n,
                                                          int stride_col_y, int stride_col_dst) {
    using F = Legacy<ID>;
    extern __shared__ __align__(16) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (STAGED) stage_acts(lds, vy, B, nb, stride_col_y);
    for (int row = blockIdx.x * LWAVES + wave; row < n; row += gridDim.x * LWAVES) {
        const uint8_t* wrow = vx + (size_t)row * nb * F::BYTES;
        float acc[B];
#pragma unroll
        for (int c = 0; c < B; ++c) acc[c] = 0.f;
        for (int b = lane; b < nb; b += 64) {
            const uint8_t* bp = wrow + (size_t)b * F::BYTES;
            uint4 lo, hi;
            block_codes<F>(bp, lo, hi);
            const float d = block_scale<F>(bp);
            const float m = F::M_AT >= 0 ? f16_bits_to_f32(*(const uint16_t*)(bp + (F::M_AT >= 0 ? F::M_AT : 0))) : 0.f;
#pragma unroll
            for (int c = 0; c < B; ++c) {
                const ActBlock a = act_block<STAGED>(lds, vy, B * nb, nb, stride_col_y, c, b);
                float part = d * a.d8 * (float)block_dot(lo, hi, a, F::BIAS);
                if (F::M_AT >= 0) part += m * (a.d8 * (float)(a.sum0 + a.sum1));
                acc[c] += part;
            }
        }
#pragma unroll
        for (int c = 0; c < B; ++c) {
            const float total = wave_sum(acc[c]);
            if (lane == 0) dst[(size_t)c * stride_col_dst + row] = from_f32<T>(bias ? total + bias[row] : total);
        }
    }
}

// The parity probe: every block's integer (sum (code - bias) * a) against ONE Q8_1 row.
template <int ID>
__global__ __launch_bounds__(64) void subdots_legacy_kernel(const uint8_t* __restrict__ vx, const uint8_t* __restrict__ vy,
                                                            int32_t* __restrict__ dots, int nb) {
    using F = Legacy<ID>;
    const int row = blockIdx.y, b = blockIdx.x * 64 + threadIdx.x;
    if (b >= nb) return;
    uint4 lo, hi;
    block_codes<F>(vx + ((size_t)row * nb + b) * F::BYTES, lo, hi);
    dots[(size_t)row * nb + b] = block_dot(lo, hi, act_from_memory(vy + (size_t)b * Q81_BYTES), F::BIAS);
}

// ---------------------------------------------------------------------------------------------
// Q2_K {scales[16], qs[64], d, dmin} (84 bytes) and Q3_K {hmask[32], qs[64], scales[12], d} (110
// bytes): sixteen sub-blocks of sixteen two-bit codes (src/tensor/quant_cpu/format/q2_k.rs:15-33,
// q3_k.rs:10-37, 127-146). The 32 values of Q8_1 block j of a super-block are sub-blocks 2 j and
// 2 j + 1: bytes 32 (j / 4) .. + 32 of qs at shift 2 (j % 4), and for Q3_K bit j of the 32 hmask
// bytes (clear = the value is four less). Q2_K: d * (sc & 15) * q - dmin * (sc >> 4); Q3_K:
// d * (six-bit scale - 32) * (q - 4 * !h). Combined as the reference's mat-vec combines them
// (cuda/moe/gguf.cuh:524-546, 937-959). A lane owns one Q8_1 block of the row; eight lanes share a
// super-block (and re-read its header bytes from cache). The plain statement, as above.
// IQ4_XS {d, scales_h, scales_l[4], qs[128]} (136 bytes, iq4_xs.rs:5-37) rides the same kernel: run
// j = bytes 16 j .. + 16 of qs as IQ4_NL levels (low nibbles values 0..15, high 16..31), one
// six-bit scale less 32 for the run.
// ---------------------------------------------------------------------------------------------
// Bytes of a block and runs of 32 values in it, by ggml type id: Q2_K, Q3_K, IQ4_XS and the codebook formats
// (IQ2_XXS 16, IQ3_XXS 18, IQ3_S 21, IQ2_S 22, Q2_0 42: codebook_blocks.h), which ride the same kernels: a run
// decodes to 32 int8 weights, an odd integer scale per half and the block's float.
template <int ID> struct Lowbit { static constexpr int BYTES = codebook::Fmt<ID>::BYTES, RUNS = codebook::Fmt<ID>::RUNS; };
template <> struct Lowbit<10> { static constexpr int BYTES = 84, RUNS = 8; };
template <> struct Lowbit<11> { static constexpr int BYTES = 110, RUNS = 8; };
template <> struct Lowbit<23> { static constexpr int BYTES = 136, RUNS = 8; };
static constexpr bool is_lowbit(int id) { return id == 10 || id == 11 || id == 23 || codebook::is_codebook(id); }

struct LowbitBlock {
    uint4 lo, hi;         // the block's codes 0..3, values 0..15 and 16..31
    uint4 nlo, nhi;       // Q3_K: 1 where the high bit is clear
    int sc0, sc1, mn0, mn1;
    float d, dmin;
};

// 32 bytes at a 2-byte-aligned address, made from the enclosing dwords like a Run16: two 16-byte
// loads and the dword that holds the run's last two bytes. Q3_K's 110-byte super-blocks put every
// other one two bytes off a dword, and its mat-vec ran at half the rate of Q2_K's on 16-byte loads
// from such addresses.
static __device__ __forceinline__ void load_run32(const uint8_t* p, uint4& lo, uint4& hi) {
    const uintptr_t a = (uintptr_t)p;
    const uint8_t* b = (const uint8_t*)(a & ~(uintptr_t)3);
    const uint4 x = *(const uint4_a4*)b, y = *(const uint4_a4*)(b + 16);
    const uint32_t e = *(const uint32_t*)(b + 28 + 2 * (a & 2));
    const uint32_t sh = 8 * (uint32_t)(a & 3);
    lo = make_uint4(__builtin_amdgcn_alignbit(x.y, x.x, sh), __builtin_amdgcn_alignbit(x.z, x.y, sh),
                    __builtin_amdgcn_alignbit(x.w, x.z, sh), __builtin_amdgcn_alignbit(y.x, x.w, sh));
    hi = make_uint4(__builtin_amdgcn_alignbit(y.y, y.x, sh), __builtin_amdgcn_alignbit(y.z, y.y, sh),
                    __builtin_amdgcn_alignbit(y.w, y.z, sh), __builtin_amdgcn_alignbit(e, y.w, sh));
}

template <int ID>
static __device__ __forceinline__ LowbitBlock lowbit_block(const uint8_t* __restrict__ bp, int j) {
    LowbitBlock r;
    if constexpr (codebook::is_codebook(ID)) {
        const codebook::Run run = codebook::decode<ID>(codebook::fetch<ID>(bp, j), j);
        r.lo = run.lo;
        r.hi = run.hi;
        r.sc0 = run.sc0;
        r.sc1 = run.sc1;
        r.mn0 = r.mn1 = 0;
        r.d = run.d;
        r.dmin = 0.f;
        r.nlo = r.nhi = make_uint4(0, 0, 0, 0);
        return r;
    }
    if (ID == 23) {
        const uint4 q = *(const uint4_a4*)(bp + 8 + 16 * j);
        r.lo = make_uint4(levels_of<1>(q.x & 0x0F0F0F0Fu), levels_of<1>(q.y & 0x0F0F0F0Fu), levels_of<1>(q.z & 0x0F0F0F0Fu),
                          levels_of<1>(q.w & 0x0F0F0F0Fu));
        r.hi = make_uint4(levels_of<1>((q.x >> 4) & 0x0F0F0F0Fu), levels_of<1>((q.y >> 4) & 0x0F0F0F0Fu),
                          levels_of<1>((q.z >> 4) & 0x0F0F0F0Fu), levels_of<1>((q.w >> 4) & 0x0F0F0F0Fu));
        const uint2 head = *(const uint2_a2*)bp;   // d, scales_h | scales_l[4]
        const uint32_t low = (head.y >> (4 * j)) & 15u;
        const uint32_t high = (head.x >> (16 + 2 * j)) & 3u;
        r.sc0 = r.sc1 = (int)(low | (high << 4)) - 32;
        r.mn0 = r.mn1 = 0;
        r.d = f16_bits_to_f32(head.x & 0xFFFFu);
        r.dmin = 0.f;
        r.nlo = r.nhi = make_uint4(0, 0, 0, 0);
        return r;
    }
    const int shift = 2 * (j & 3);
    const uint8_t* qs = bp + (ID == 10 ? 16 : 32) + 32 * (j >> 2);
    uint4 q0, q1;
    if (ID == 11) {
        load_run32(qs, q0, q1);
    } else {
        q0 = *(const uint4_a4*)qs;
        q1 = *(const uint4_a4*)(qs + 16);
    }
    r.lo = make_uint4((q0.x >> shift) & 0x03030303u, (q0.y >> shift) & 0x03030303u, (q0.z >> shift) & 0x03030303u, (q0.w >> shift) & 0x03030303u);
    r.hi = make_uint4((q1.x >> shift) & 0x03030303u, (q1.y >> shift) & 0x03030303u, (q1.z >> shift) & 0x03030303u, (q1.w >> shift) & 0x03030303u);
    if (ID == 10) {
        const uint32_t sm = *(const uint16_t*)(bp + 2 * j);   // scale | min << 4 of sub-blocks 2 j, 2 j + 1
        r.sc0 = sm & 15; r.mn0 = (sm >> 4) & 15; r.sc1 = (sm >> 8) & 15; r.mn1 = sm >> 12;
        const uint32_t dm = *(const uint32_a2*)(bp + 80);
        r.d = f16_bits_to_f32(dm & 0xFFFFu);
        r.dmin = f16_bits_to_f32(dm >> 16);
        r.nlo = r.nhi = make_uint4(0, 0, 0, 0);
    } else {
        uint4 h0, h1;
        load_run32(bp, h0, h1);
        r.nlo = make_uint4((~h0.x >> j) & 0x01010101u, (~h0.y >> j) & 0x01010101u, (~h0.z >> j) & 0x01010101u, (~h0.w >> j) & 0x01010101u);
        r.nhi = make_uint4((~h1.x >> j) & 0x01010101u, (~h1.y >> j) & 0x01010101u, (~h1.z >> j) & 0x01010101u, (~h1.w >> j) & 0x01010101u);
        // scales 2 j and 2 j + 1 of the sixteen packed in twelve bytes
        // (scale i: low four bits = nibble i / 8 of byte i % 8, top two = bits 2 (i / 4) of byte 8 + i % 4)
        const uintptr_t sa = (uintptr_t)(bp + 96);
        const uint32_t* sb = (const uint32_t*)(sa & ~(uintptr_t)3);
        const uint32_t x0 = sb[0], x1 = sb[1], x2 = sb[2], x3 = sb[2 + ((sa & 2) >> 1)], sh = 8 * (uint32_t)(sa & 3);
        const uint32_t w0 = __builtin_amdgcn_alignbit(x1, x0, sh), w1 = __builtin_amdgcn_alignbit(x2, x1, sh),
                       w2 = __builtin_amdgcn_alignbit(x3, x2, sh);
        const int group = j >> 1, jj = 2 * (j & 1);
        const uint32_t low = ((group & 1) ? w1 : w0) >> (8 * jj + (group < 2 ? 0 : 4));
        const uint32_t top = w2 >> (8 * jj + 2 * group);
        r.sc0 = (int)((low & 15u) | ((top & 3u) << 4)) - 32;
        r.sc1 = (int)(((low >> 8) & 15u) | (((top >> 8) & 3u) << 4)) - 32;
        r.mn0 = r.mn1 = 0;
        r.d = f16_bits_to_f32(*(const uint16_t*)(bp + 108));
        r.dmin = 0.f;
    }
    return r;
}

// The two sub-block integers of the block against a Q8_1 block.
template <int ID>
static __device__ __forceinline__ void lowbit_dots(const LowbitBlock& w, const ActBlock& a, int& dot0, int& dot1) {
    dot0 = dot16(w.lo, a.lo, 0);
    dot1 = dot16(w.hi, a.hi, 0);
    if (ID == 11) {
        dot0 -= 4 * dot16(w.nlo, a.lo, 0);
        dot1 -= 4 * dot16(w.nhi, a.hi, 0);
    }
}

// The block's share of the row's result.
template <int ID>
static __device__ __forceinline__ float lowbit_share(const LowbitBlock& w, const ActBlock& a) {
    int dot0, dot1;
    lowbit_dots<ID>(w, a, dot0, dot1);
    float part = w.d * (a.d8 * (float)(dot0 * w.sc0 + dot1 * w.sc1));
    if (ID == 10) part -= w.dmin * (a.d8 * (float)(a.sum0 * w.mn0 + a.sum1 * w.mn1));
    return part;
}

template <int ID, int B, typename T, bool STAGED>
__global__ __launch_bounds__(LWG) void mmvq_lowbit_kernel(const uint8_t* __restrict__ vx, const uint8_t* __restrict__ vy,
                                                          T* __restrict__ dst, const float* __restrict__ bias, int nb, int n,
                                                          int stride_col_y, int stride_col_dst) {
    constexpr int BYTES = Lowbit<ID>::BYTES, RUNS = Lowbit<ID>::RUNS;
    extern __shared__ __align__(16) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int k32 = nb * RUNS;
    if (STAGED) stage_acts(lds, vy, B, k32, stride_col_y);
    for (int row = blockIdx.x * LWAVES + wave; row < n; row += gridDim.x * LWAVES) {
        const uint8_t* wrow = vx + (size_t)row * nb * BYTES;
        float acc[B];
#pragma unroll
        for (int c = 0; c < B; ++c) acc[c] = 0.f;
        for (int idx = lane; idx < k32; idx += 64) {
            const LowbitBlock w = lowbit_block<ID>(wrow + (size_t)(idx / RUNS) * BYTES, idx % RUNS);
#pragma unroll
            for (int c = 0; c < B; ++c)
                acc[c] += lowbit_share<ID>(w, act_block<STAGED>(lds, vy, B * k32, k32, stride_col_y, c, idx));
        }
#pragma unroll
        for (int c = 0; c < B; ++c) {
            const float total = wave_sum(acc[c]);
            if (lane == 0) dst[(size_t)c * stride_col_dst + row] = from_f32<T>(bias ? total + bias[row] : total);
        }
    }
}

template <int ID>
__global__ __launch_bounds__(64) void subdots_lowbit_kernel(const uint8_t* __restrict__ vx, const uint8_t* __restrict__ vy,
                                                            int32_t* __restrict__ dots, int nb) {
    constexpr int BYTES = Lowbit<ID>::BYTES, RUNS = Lowbit<ID>::RUNS;
    const int row = blockIdx.y, idx = blockIdx.x * 64 + threadIdx.x;
    if (idx >= nb * RUNS) return;
    const LowbitBlock w = lowbit_block<ID>(vx + ((size_t)row * nb + (idx / RUNS)) * BYTES, idx % RUNS);
    int dot0, dot1;
    lowbit_dots<ID>(w, act_from_memory(vy + (size_t)idx * Q81_BYTES), dot0, dot1);
    if (ID == 23) {   // one integer per run of 32
        dots[(size_t)row * nb * 8 + idx] = dot0 + dot1;
        return;
    }
    int32_t* out = dots + (size_t)row * nb * 2 * RUNS + 2 * idx;
    out[0] = dot0;
    out[1] = dot1;
}

// ---------------------------------------------------------------------------------------------
// MoE decode over these formats: the per-pair mat-vec of loken's expert launchers
// (cuda/moe/moe_gguf.cu:476-511, 755-860, 1049-1061) for the rows of its format table that the
// K-quant engines do not serve. Workgroups (x, pair): the pair's Q8_1 row goes to LDS once, each
// wave then takes weight rows of the pair's expert. MODE 0: out = w . x (times the routing weight
// when given), 1: the gated activation of (gate . x, up . x), 2: routing weight * (w . x + bias).
// ---------------------------------------------------------------------------------------------
struct MoeLegacyDims {
    int experts, topk, pairs, cols, nb, k32, k32_stride;
    int64_t slab_bytes;
    int slab_rows;
    LkGateAct act;
    const unsigned int* live;
    LkMoeAlt alt;
};

// A lane's share of one weight row against the activation row in LDS.
template <int ID>
static __device__ __forceinline__ float staged_row_share(const uint8_t* __restrict__ wrow, int nb, const uint8_t* lds,
                                                         int k32, int lane) {
    float acc = 0.f;
    if constexpr (is_lowbit(ID)) {
        constexpr int BYTES = Lowbit<ID>::BYTES, RUNS = Lowbit<ID>::RUNS;
        for (int idx = lane; idx < k32; idx += 64) {
            const LowbitBlock w = lowbit_block<ID>(wrow + (size_t)(idx / RUNS) * BYTES, idx % RUNS);
            acc += lowbit_share<ID>(w, act_block<true>(lds, nullptr, k32, k32, 0, 0, idx));
        }
    } else {
        using F = Legacy<ID>;
        for (int b = lane; b < nb; b += 64) {
            const uint8_t* bp = wrow + (size_t)b * F::BYTES;
            uint4 lo, hi;
            block_codes<F>(bp, lo, hi);
            const float d = block_scale<F>(bp);
            const float m = F::M_AT >= 0 ? f16_bits_to_f32(*(const uint16_t*)(bp + (F::M_AT >= 0 ? F::M_AT : 0))) : 0.f;
            const ActBlock a = act_block<true>(lds, nullptr, nb, nb, 0, 0, b);
            float part = d * a.d8 * (float)block_dot(lo, hi, a, F::BIAS);
            if (F::M_AT >= 0) part += m * (a.d8 * (float)(a.sum0 + a.sum1));
            acc += part;
        }
    }
    return acc;
}

template <int ID, bool LOW = is_lowbit(ID)> struct BytesOf { static constexpr int V = Legacy<ID>::BYTES, RUNS = 1; };
template <int ID> struct BytesOf<ID, true> { static constexpr int V = Lowbit<ID>::BYTES, RUNS = Lowbit<ID>::RUNS; };

template <int ID, int MODE>
__global__ __launch_bounds__(LWG) void moe_rows_legacy_kernel(const uint8_t* __restrict__ w0, const uint8_t* __restrict__ w1,
                                                              const uint8_t* __restrict__ acts,
                                                              const int32_t* __restrict__ sorted_token_ids,
                                                              const int32_t* __restrict__ expert_ids,
                                                              const float* __restrict__ topk_weights,
                                                              const float* __restrict__ down_bias, float* __restrict__ out,
                                                              MoeLegacyDims d) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int pair = blockIdx.y;
    // the pair's routing and the live count in one round of scalar loads, the launch's fields in the
    // round before it (asked for where each is first used they arrive in many dependent rounds)
    const int slot = sorted_token_ids[pair];
    const int e = expert_ids[pair];
    const unsigned int live = d.live != nullptr ? *d.live : 0xFFFFFFFFu;
    asm volatile("" ::"s"(slot), "s"(e), "s"(live), "s"(d.pairs), "s"(d.experts), "s"(d.cols), "s"(d.nb), "s"(d.k32),
                 "s"(d.k32_stride), "s"(d.topk), "s"(w0), "s"(w1), "s"(acts), "s"(out), "s"(topk_weights),
                 "s"(d.slab_bytes), "s"(d.alt.alt0), "s"(d.alt.alt_at), "s"(d.alt.alt_from), "s"(d.act.kind));
    if ((unsigned int)pair >= live) return;
    if (slot < 0 || slot >= d.pairs) return;   // the whole workgroup leaves together
    float* out_row = out + (size_t)slot * d.cols;
    if (e < 0 || e >= d.experts) {
        // a pair the routing leaves out adds nothing: its row of the fold's input reads zero
        if (MODE == 2)
            for (int r = blockIdx.x * LWG + threadIdx.x; r < d.cols; r += gridDim.x * LWG) out_row[r] = 0.f;
        return;
    }
    const bool own_row = MODE == 2 || (MODE == 0 && topk_weights != nullptr);
    const int act_row = own_row ? slot : slot / d.topk;
    stage_acts(lds, acts + (size_t)act_row * d.k32_stride * Q81_BYTES, 1, d.k32, 0);
    const float scale = (MODE != 1 && topk_weights) ? topk_weights[slot] : 1.0f;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t row_bytes = (size_t)d.nb * BytesOf<ID>::V;
    const uint8_t* slab0 = lk_expert_slab(w0, 0, d.alt, e, d.slab_bytes);
    for (int row = blockIdx.x * LWAVES + wave; row < d.cols; row += gridDim.x * LWAVES) {
        const float first = wave_sum(staged_row_share<ID>(slab0 + row * row_bytes, d.nb, lds, d.k32, lane));
        if (MODE == 1) {
            const uint8_t* slab1 = lk_expert_slab(w1, 1, d.alt, e, d.slab_bytes);
            const float second = wave_sum(staged_row_share<ID>(slab1 + row * row_bytes, d.nb, lds, d.k32, lane));
            if (lane == 0) out_row[row] = lk_gated(d.act, first, second, (size_t)e * d.cols + row);
        } else {
            float v = first * scale;
            if (MODE == 2 && down_bias) v += scale * down_bias[(size_t)e * d.cols + row];
            if (lane == 0) out_row[row] = v;
        }
    }
}

template <int ID>
static int launch_moe(int mode, const uint8_t* w0, const uint8_t* w1, const uint8_t* acts, const int32_t* sti,
                      const int32_t* eid, const float* tw, const float* bias, float* out, MoeLegacyDims d, hipStream_t s) {
    d.k32 = d.nb * BytesOf<ID>::RUNS;
    d.slab_bytes = (int64_t)d.slab_rows * d.nb * BytesOf<ID>::V;
    const size_t lds_bytes = (size_t)d.k32 * ACT_LDS_PER_BLOCK;
    if (lds_bytes > 48 * 1024 || d.pairs > 65535) return LK_ERR_ARG;
    const int need = (d.cols + LWAVES - 1) / LWAVES;
    int share = lk_device().cus * 8 / d.pairs;
    if (share < 1) share = 1;
    const dim3 grid(need < share ? need : share, d.pairs);
    const auto run = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(LWG), lds_bytes, s, w0, w1, acts, sti, eid, tw, bias, out, d);
    };
    switch (mode) {
        case 0: run(moe_rows_legacy_kernel<ID, 0>); break;
        case 1: run(moe_rows_legacy_kernel<ID, 1>); break;
        case 2: run(moe_rows_legacy_kernel<ID, 2>); break;
        default: return LK_ERR_ARG;
    }
    return lk_launch_status();
}

template <int ID, int B, typename T>
static int launch(const void* vx, const void* vy, void* dst, const float* bias, int nb, int n, int stride_col_y,
                  int stride_col_dst, hipStream_t s) {
    const int need = (n + LWAVES - 1) / LWAVES, cap = lk_device().cus * 8;
    const dim3 grid(need < cap ? need : cap);
    constexpr bool LOWBIT = is_lowbit(ID);
    const int k32 = nb * BytesOf<ID>::RUNS;
    const size_t lds_bytes = (size_t)B * k32 * ACT_LDS_PER_BLOCK;
    const auto run = [&](auto kernel, size_t lds) {
        hipLaunchKernelGGL(kernel, grid, dim3(LWG), lds, s, (const uint8_t*)vx, (const uint8_t*)vy, (T*)dst, bias, nb, n,
                           stride_col_y, stride_col_dst);
    };
    // the activation rows in LDS while they fit the 48 KB every kernel may ask for; from memory beyond
    if (lds_bytes <= 48 * 1024) {
        if constexpr (LOWBIT) run(mmvq_lowbit_kernel<ID, B, T, true>, lds_bytes);
        else run(mmvq_legacy_kernel<ID, B, T, true>, lds_bytes);
    } else {
        if constexpr (LOWBIT) run(mmvq_lowbit_kernel<ID, B, T, false>, 0);
        else run(mmvq_legacy_kernel<ID, B, T, false>, 0);
    }
    return lk_launch_status();
}

template <int ID, typename T>
static int by_batch(int batch, const void* vx, const void* vy, void* dst, const float* bias, int nb, int n,
                    int stride_col_y, int stride_col_dst, hipStream_t s) {
    // batches above four go out as two launches: the per-lane accumulators stay few
    if (batch > 4) {
        if (int rc = by_batch<ID, T>(4, vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s)) return rc;
        return by_batch<ID, T>(batch - 4, vx, (const uint8_t*)vy + (size_t)4 * stride_col_y * Q81_BYTES,
                               (T*)dst + (size_t)4 * stride_col_dst, bias, nb, n, stride_col_y, stride_col_dst, s);
    }
    switch (batch) {
        case 1: return launch<ID, 1, T>(vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s);
        case 2: return launch<ID, 2, T>(vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s);
        case 3: return launch<ID, 3, T>(vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s);
        default: return launch<ID, 4, T>(vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s);
    }
}

template <int ID>
static int by_type(int dst_type, int batch, const void* vx, const void* vy, void* dst, const float* bias, int nb, int n,
                   int stride_col_y, int stride_col_dst, hipStream_t s) {
    switch (dst_type) {
        case LK_TYPE_F32: return by_batch<ID, float>(batch, vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s);
        case LK_TYPE_F16: return by_batch<ID, __half>(batch, vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s);
        case LK_TYPE_BF16: return by_batch<ID, __hip_bfloat16>(batch, vx, vy, dst, bias, nb, n, stride_col_y, stride_col_dst, s);
        default: return LK_ERR_TYPE;
    }
}

}  // namespace

bool lk_is_legacy_type(int wtype) {
    return wtype == LK_TYPE_Q4_0 || wtype == LK_TYPE_Q4_1 || wtype == LK_TYPE_Q5_0 || wtype == LK_TYPE_Q5_1 ||
           wtype == LK_TYPE_IQ4_NL || wtype == LK_TYPE_MXFP4 || wtype == LK_TYPE_Q2_K || wtype == LK_TYPE_Q3_K ||
           wtype == LK_TYPE_IQ4_XS || codebook::is_codebook(wtype);
}

// lk_mmvq for the 32-value nibble formats (the caller has told them apart with lk_is_legacy_type).
int lk_mmvq_legacy(int wtype, const void* vx, const void* vy_q8_1, void* dst, int dst_type, int ncols_x, int nrows_x,
                   int batch, int stride_col_y, int stride_col_dst, const float* bias, hipStream_t s) {
    if (nrows_x == 0) return LK_OK;
    const int block_len = wtype == LK_TYPE_Q2_0 ? 64
                          : wtype == LK_TYPE_Q2_K || wtype == LK_TYPE_Q3_K || wtype == LK_TYPE_IQ4_XS || codebook::is_codebook(wtype) ? 256 : 32;
    if (!vx || !vy_q8_1 || !dst || ncols_x <= 0 || ncols_x % block_len != 0 || nrows_x < 0) return LK_ERR_ARG;
    if (batch < 1 || batch > 8 || stride_col_y < ncols_x / 32 || stride_col_dst < nrows_x) return LK_ERR_ARG;
    if ((wtype != LK_TYPE_MXFP4 && ((uintptr_t)vx & 1) != 0) || ((uintptr_t)vy_q8_1 & 3) != 0) return LK_ERR_ARG;
    // super-blocks of 84 and 136 bytes are read with dword-aligned 16-byte loads
    if ((wtype == LK_TYPE_Q2_K || wtype == LK_TYPE_IQ4_XS) && ((uintptr_t)vx & 3) != 0) return LK_ERR_ARG;
    const int nb = ncols_x / block_len;
    switch (wtype) {
        case LK_TYPE_Q2_K: return by_type<10>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_Q3_K: return by_type<11>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_IQ4_XS: return by_type<23>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_IQ2_XXS: return by_type<16>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_IQ3_XXS: return by_type<18>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_IQ3_S: return by_type<21>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_IQ2_S: return by_type<22>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_Q2_0: return by_type<42>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_Q4_0: return by_type<2>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_Q4_1: return by_type<3>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_Q5_0: return by_type<6>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_Q5_1: return by_type<7>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_IQ4_NL: return by_type<20>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        case LK_TYPE_MXFP4: return by_type<39>(dst_type, batch, vx, vy_q8_1, dst, bias, nb, nrows_x, stride_col_y, stride_col_dst, s);
        default: return LK_ERR_TYPE;
    }
}

int lk_mmvq_subdots_legacy(int wtype, const void* vx, const void* vy_q8_1, int32_t* dots, int ncols_x, int nrows_x,
                           hipStream_t s) {
    if (!vx || !vy_q8_1 || !dots || ncols_x <= 0 || ncols_x % 32 != 0 || nrows_x <= 0 || nrows_x > 65535) return LK_ERR_ARG;
    const uint8_t *w = (const uint8_t*)vx, *y = (const uint8_t*)vy_q8_1;
    if (wtype == LK_TYPE_Q2_K || wtype == LK_TYPE_Q3_K || wtype == LK_TYPE_IQ4_XS) {
        // sixteen sub-block integers per super-block (IQ4_XS: eight, one per run of 32)
        if (ncols_x % 256 != 0 || ((uintptr_t)vx & (wtype == LK_TYPE_Q3_K ? 1 : 3)) != 0) return LK_ERR_ARG;
        const int nbk = ncols_x / 256;
        const dim3 gridk((nbk * 8 + 63) / 64, nrows_x);
        if (wtype == LK_TYPE_Q2_K) hipLaunchKernelGGL(subdots_lowbit_kernel<10>, gridk, dim3(64), 0, s, w, y, dots, nbk);
        else if (wtype == LK_TYPE_Q3_K) hipLaunchKernelGGL(subdots_lowbit_kernel<11>, gridk, dim3(64), 0, s, w, y, dots, nbk);
        else hipLaunchKernelGGL(subdots_lowbit_kernel<23>, gridk, dim3(64), 0, s, w, y, dots, nbk);
        return lk_launch_status();
    }
    if (codebook::is_codebook(wtype)) {
        // two integers per run of 32: its halves
        const int len = wtype == LK_TYPE_Q2_0 ? 64 : 256;
        if (ncols_x % len != 0 || ((uintptr_t)vx & 1) != 0) return LK_ERR_ARG;
        const int nbc = ncols_x / len;
        const dim3 gridc((ncols_x / 32 + 63) / 64, nrows_x);
        switch (wtype) {
            case LK_TYPE_IQ2_XXS: hipLaunchKernelGGL(subdots_lowbit_kernel<16>, gridc, dim3(64), 0, s, w, y, dots, nbc); break;
            case LK_TYPE_IQ3_XXS: hipLaunchKernelGGL(subdots_lowbit_kernel<18>, gridc, dim3(64), 0, s, w, y, dots, nbc); break;
            case LK_TYPE_IQ3_S: hipLaunchKernelGGL(subdots_lowbit_kernel<21>, gridc, dim3(64), 0, s, w, y, dots, nbc); break;
            case LK_TYPE_IQ2_S: hipLaunchKernelGGL(subdots_lowbit_kernel<22>, gridc, dim3(64), 0, s, w, y, dots, nbc); break;
            default: hipLaunchKernelGGL(subdots_lowbit_kernel<42>, gridc, dim3(64), 0, s, w, y, dots, nbc); break;
        }
        return lk_launch_status();
    }
    const int nb = ncols_x / 32;
    const dim3 grid((nb + 63) / 64, nrows_x);
    switch (wtype) {
        case LK_TYPE_Q4_0: hipLaunchKernelGGL(subdots_legacy_kernel<2>, grid, dim3(64), 0, s, w, y, dots, nb); break;
        case LK_TYPE_Q4_1: hipLaunchKernelGGL(subdots_legacy_kernel<3>, grid, dim3(64), 0, s, w, y, dots, nb); break;
        case LK_TYPE_Q5_0: hipLaunchKernelGGL(subdots_legacy_kernel<6>, grid, dim3(64), 0, s, w, y, dots, nb); break;
        case LK_TYPE_Q5_1: hipLaunchKernelGGL(subdots_legacy_kernel<7>, grid, dim3(64), 0, s, w, y, dots, nb); break;
        case LK_TYPE_IQ4_NL: hipLaunchKernelGGL(subdots_legacy_kernel<20>, grid, dim3(64), 0, s, w, y, dots, nb); break;
        case LK_TYPE_MXFP4: hipLaunchKernelGGL(subdots_legacy_kernel<39>, grid, dim3(64), 0, s, w, y, dots, nb); break;
        default: return LK_ERR_TYPE;
    }
    return lk_launch_status();
}

// Wire ids of the reference's expert table (src/inference/moe_cuda/gemm.rs:23-39) served here.
int lk_moe_wire_block_len_legacy(int quant_type) {
    switch (quant_type) {
        case 2: case 3: case 10: return 256;       // Q2_K, Q3_K, IQ4_XS
        case 11: case 12: case 13: case 15: return 256;   // IQ3_XXS, IQ3_S, IQ2_S, IQ2_XXS
        case 14: return 64;                        // Q2_0
        case 6: case 7: case 8: case 9: return 32; // Q5_0, MXFP4, Q5_1, IQ4_NL
        default: return 0;
    }
}

int lk_moe_rows_legacy(int mode, int quant_type, const uint8_t* w0, const uint8_t* w1, const uint8_t* acts_q8_1,
                       const int32_t* sorted_token_ids, const int32_t* expert_ids, const float* topk_weights,
                       const float* down_bias, float* out, int experts, int topk, int pairs, int cols, int size_k,
                       int k32_stride, const LkGateAct& act, int slab_rows, const unsigned int* live,
                       const LkMoeAlt& alt, hipStream_t s) {
    const int bl = lk_moe_wire_block_len_legacy(quant_type);
    if (bl == 0) return LK_ERR_TYPE;
    if (size_k % bl != 0 || ((uintptr_t)acts_q8_1 & 3) != 0) return LK_ERR_ARG;
    const uintptr_t both = (uintptr_t)w0 | (uintptr_t)w1 | (uintptr_t)alt.alt0 | (uintptr_t)alt.alt1;
    const uintptr_t mask = (quant_type == 2 || quant_type == 10) ? 3 : quant_type == 7 ? 0 : 1;
    if ((both & mask) != 0) return LK_ERR_ARG;
    MoeLegacyDims d{experts, topk, pairs, cols, size_k / bl, 0, k32_stride, 0, slab_rows, act, live, alt};
    switch (quant_type) {
        case 2: return launch_moe<10>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 3: return launch_moe<11>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 6: return launch_moe<6>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 7: return launch_moe<39>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 8: return launch_moe<7>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 9: return launch_moe<20>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 11: return launch_moe<18>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 12: return launch_moe<21>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 13: return launch_moe<22>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 14: return launch_moe<42>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        case 15: return launch_moe<16>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
        default: return launch_moe<23>(mode, w0, w1, acts_q8_1, sorted_token_ids, expert_ids, topk_weights, down_bias, out, d, s);
    }
}

// Decode mat-vec launchers: GGUF weight rows (Q4_K / Q6_K / Q8_0) against 1..8 Q8_1 activation
// rows, plus the fused neighbours that share its engine (several matrices over one activation,
// gate/up pairs with the activation function applied in the store, grouped launches).
//
// Bandwidth work, so the design is about bytes in flight, not arithmetic:
//   * a lane loads 16 weight bytes per instruction (global_load_dwordx4); a wave takes whole
//     super-blocks side by side (Q4_K 4 lanes per 256-value block and 16 blocks = 4096 values
//     per pass; Q6_K 8 lanes per block; Q8_0 2 lanes per 32-value block);
//   * a wave owns R consecutive weight rows end to end (no cross-wave reduction) and persists
//     over row tiles, with the next tile's loads in flight while the current one is consumed;
//   * the Q8_1 activation is staged ONCE per workgroup into LDS, re-laid so that the 16 bytes a
//     lane needs sit at lane*16 of a plane (conflict-free ds_read_b128), with its f16 scales
//     widened to f32 and, for Q4_K, d8 * sum(codes) precomputed for the min term;
//   * 6-bit scales / mins are unpacked in registers from the 16-byte block header;
//   * integer products are v_dot4_i32_i8; per-lane f32 partials meet in one wave64 DPP
//     reduction per row.
// The engines live in mmvq_core.h.

#include "mmvq_launch.h"

using namespace mmvq;

namespace {

// --------------------------------------------------------------------------------------------
// Sub-block-dot probe: one wave per (row, pass), activation read straight from global memory.
// --------------------------------------------------------------------------------------------
static __device__ __forceinline__ void load_act16(const uint8_t* vy, int q81_block, int lh, uint4& a) {
    const uint32_t* src = (const uint32_t*)(vy + (size_t)q81_block * Q81_BYTES) + 1 + 4 * lh;
    a = make_uint4(src[0], src[1], src[2], src[3]);
}

__global__ __launch_bounds__(64) void subdots_q4k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7, p = ch >> 1, lh = ch & 1;
    int d_lo = 0, d_hi = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q4K_BYTES;
        const uint4 q = *(const uint4*)(bp + 16 + 16 * ch);
        uint4 a_lo, a_hi;
        load_act16(vy, blk * 8 + 2 * p, lh, a_lo);
        load_act16(vy, blk * 8 + 2 * p + 1, lh, a_hi);
        // the integer core of the register-resident engine: the high nibbles stay in place and the
        // accumulator starts at 128 * (sum of the activation codes), which leaves 16 * d_hi
        const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
        d_hi = 128 * dot16(ones, a_hi, 0);
        uint32_t flip = 0x80808080u;
        asm volatile("" : "+v"(flip));
        q4k_dots_biased(q, a_lo, a_hi, flip, d_lo, d_hi);
        int plain_lo = 0, plain_hi = 0;
        q4k_dots(q, a_lo, a_hi, plain_lo, plain_hi);   // the staged engine's core: must agree
        if (plain_lo != d_lo || 16 * plain_hi != d_hi) d_lo = d_hi = 0x7FFFFFF0;
        d_hi >>= 4;
    }
    d_lo += __shfl_xor(d_lo, 1);
    d_hi += __shfl_xor(d_hi, 1);
    if (blk < nb && lh == 0) {
        int32_t* out = dots + (size_t)row * nb * 8 + blk * 8 + 2 * p;
        out[0] = d_lo;
        out[1] = d_hi;
    }
}

__global__ __launch_bounds__(64) void subdots_q5k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7, p = ch >> 1, lh = ch & 1;
    int d_lo = 0, d_hi = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q5K_BYTES;
        const uint4 q = *(const uint4*)(bp + 48 + 16 * ch);
        const uint4 qh = *(const uint4*)(bp + 16 + 16 * lh);
        uint4 a_lo, a_hi;
        load_act16(vy, blk * 8 + 2 * p, lh, a_lo);
        load_act16(vy, blk * 8 + 2 * p + 1, lh, a_hi);
        q5k_dots(q, shr4(qh, 2 * p), a_lo, a_hi, d_lo, d_hi);
    }
    d_lo += __shfl_xor(d_lo, 1);
    d_hi += __shfl_xor(d_hi, 1);
    if (blk < nb && lh == 0) {
        int32_t* out = dots + (size_t)row * nb * 8 + blk * 8 + 2 * p;
        out[0] = d_lo;
        out[1] = d_hi;
    }
}

__global__ __launch_bounds__(64) void subdots_q6k_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 8 + (lane >> 3), ch = lane & 7;
    const int h = ch >> 2, g0 = (ch >> 1) & 1, lh = ch & 1;
    if (blk >= nb) return;
    const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q6K_BYTES;
    const uint4 ql = *(const uint4_a2*)(bp + 16 * ch);
    const uint4 qh = *(const uint4_a2*)(bp + 128 + 16 * (2 * h + lh));
    uint4 a_a, a_b;
    load_act16(vy, blk * 8 + 4 * h + g0, lh, a_a);
    load_act16(vy, blk * 8 + 4 * h + g0 + 2, lh, a_b);
    int d_a, d_b;
    q6k_dots(ql, qh, g0, a_a, a_b, d_a, d_b);
    int32_t* out = dots + (size_t)row * nb * 16 + blk * 16;
    out[8 * h + 2 * g0 + lh] = d_a;
    out[8 * h + 2 * (g0 + 2) + lh] = d_b;
}

__global__ __launch_bounds__(64) void subdots_q80_kernel(const uint8_t* __restrict__ vx,
                                                         const uint8_t* __restrict__ vy,
                                                         int32_t* __restrict__ dots, int nb) {
    const int row = blockIdx.y, lane = threadIdx.x;
    const int blk = blockIdx.x * 32 + (lane >> 1), lh = lane & 1;
    int d = 0;
    if (blk < nb) {
        const uint8_t* bp = vx + ((size_t)row * nb + blk) * Q80_BYTES;
        const uint4 q = *(const uint4_a2*)(bp + 2 + 16 * lh);
        uint4 a;
        load_act16(vy, blk, lh, a);
        d = dot16(q, a, 0);
    }
    d += __shfl_xor(d, 1);
    if (blk < nb && lh == 0) dots[(size_t)row * nb + blk] = d;
}

__global__ void act_sums_kernel(const uint8_t* __restrict__ vy, int32_t* __restrict__ sums, int k32) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= k32) return;
    uint4 lo, hi;
    load_act16(vy, j, 0, lo);
    load_act16(vy, j, 1, hi);
    const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
    sums[j] = dot16(ones, hi, dot16(ones, lo, 0));
}

static int dispatch_plain(int wtype, int dst_type, int batch, MmvqCall& a) {
    switch (wtype) {
        case LK_TYPE_Q4_K: return a.nb <= 8 ? lk_eng_plain_q4k_short(batch, dst_type, a) : lk_eng_plain_q4k(batch, dst_type, a);
        case LK_TYPE_Q5_K: return a.nb <= 8 ? lk_eng_plain_q5k_short(batch, dst_type, a) : lk_eng_plain_q5k(batch, dst_type, a);
        case LK_TYPE_Q6_K: return a.nb <= 8 ? lk_eng_plain_q6k_short(batch, dst_type, a) : lk_eng_plain_q6k(batch, dst_type, a);
        case LK_TYPE_Q8_0: return lk_eng_plain_q80(batch, dst_type, a);
        default: return LK_ERR_TYPE;
    }
}

static int check_common(int wtype, const void* vy, int ncols_x, int batch, int stride_col_y) {
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (!vy || ncols_x <= 0 || ncols_x % bl != 0) return LK_ERR_ARG;
    if (batch < 1 || batch > 8 || stride_col_y < ncols_x / 32) return LK_ERR_ARG;
    if (((uintptr_t)vy & 3) != 0) return LK_ERR_ARG;
    return LK_OK;
}
static int check_weight(int wtype, const void* vx) {
    if (!vx) return LK_ERR_ARG;
    if ((wtype == LK_TYPE_Q4_K || wtype == LK_TYPE_Q5_K) && ((uintptr_t)vx & 15) != 0) return LK_ERR_ARG;
    if (((uintptr_t)vx & 1) != 0) return LK_ERR_ARG;
    return LK_OK;
}

static int run_multi(int wtype, int count, const void* const* vx, const void* vy, void* const* dst, int dst_type,
                     int ncols_x, const int* nrows_x, int batch, int stride_col_y, int stride_col_dst,
                     const float* const* bias, void* stream, int act_stride_f32 = 0) {
    if (int rc = check_common(wtype, vy, ncols_x, batch, act_stride_f32 ? ncols_x / 32 : stride_col_y)) return rc;
    if (act_stride_f32 && (act_stride_f32 < ncols_x || act_stride_f32 % 4 != 0 || ((uintptr_t)vy & 15) != 0)) return LK_ERR_ARG;
    if (count < 1 || count > MAX_MULTI) return LK_ERR_ARG;
    MmvqCall a{};
    a.vy = (const uint8_t*)vy;
    a.nb = ncols_x / block_len_of(wtype);
    a.stride_col_y = stride_col_y;
    a.stride_col_dst = stride_col_dst;
    a.act_stride_f32 = act_stride_f32;
    a.stream = (hipStream_t)stream;
    int live = 0;
    for (int i = 0; i < count; ++i) {
        if (nrows_x[i] < 0) return LK_ERR_ARG;
        if (nrows_x[i] == 0) continue;
        if (int rc = check_weight(wtype, vx[i])) return rc;
        if (!dst[i] || stride_col_dst < nrows_x[i]) return LK_ERR_ARG;
        a.m.vx[live] = (const uint8_t*)vx[i];
        a.m.dst[live] = dst[i];
        a.m.bias[live] = bias ? bias[i] : nullptr;
        a.m.n[live] = nrows_x[i];
        ++live;
    }
    if (live == 0) return LK_OK;
    a.m.count = live;
    if (dst_type != LK_TYPE_F32 && dst_type != LK_TYPE_F16 && dst_type != LK_TYPE_BF16) return LK_ERR_TYPE;
    // one or two activation rows over Q4_K rows of at most 16 super-blocks: the register-resident engine
    if (wtype == LK_TYPE_Q4_K && batch <= LK_REG_MAX_BATCH && lk_q4k_reg_serves(a.nb)) {
        LkRegMulti m{};
        m.count = live;
        for (int i = 0; i < live; ++i) {
            m.vx[i] = a.m.vx[i];
            m.dst[i] = a.m.dst[i];
            m.bias[i] = a.m.bias[i];
            m.n[i] = a.m.n[i];
        }
        return lk_q4k_reg_multi(m, vy, act_stride_f32 != 0, a.nb, dst_type, batch, act_stride_f32 ? act_stride_f32 : stride_col_y,
                                stride_col_dst, a.stream);
    }
    // A launch stages all its activation rows in LDS; a batch that does not fit (long rows) goes
    // out as several launches over equal shares of the rows.
    const int fit = lk_device().lds_bytes / lds_bytes_of(wtype, a.nb, 1);
    if (fit < 1) return LK_ERR_ARG;
    const int launches = (batch + fit - 1) / fit, share = (batch + launches - 1) / launches;
    const size_t dst_elem = dst_type == LK_TYPE_F32 ? 4 : 2;
    for (int b0 = 0; b0 < batch; b0 += share) {
        const int b = batch - b0 < share ? batch - b0 : share;
        MmvqCall c = a;
        c.vy = a.vy + (act_stride_f32 ? (size_t)b0 * act_stride_f32 * sizeof(float) : (size_t)b0 * stride_col_y * Q81_BYTES);
        for (int i = 0; i < live; ++i) c.m.dst[i] = (uint8_t*)a.m.dst[i] + (size_t)b0 * stride_col_dst * dst_elem;
        if (int rc = dispatch_plain(wtype, dst_type, b, c)) return rc;
    }
    return LK_OK;
}

}  // namespace

extern "C" int lk_mmvq(int wtype, const void* vx, const void* vy_q8_1, void* dst, int dst_type,
                       int ncols_x, int nrows_x, int batch, int stride_col_y, int stride_col_dst,
                       const float* bias, int decode_order, void* stream) {
    (void)decode_order;  // a row's sum never depends on batch here
    if (lk_is_legacy_type(wtype))   // Q4_0, Q4_1, Q5_0, Q5_1: the plain kernel of mmvq_legacy.hip
        return lk_mmvq_legacy(wtype, vx, vy_q8_1, dst, dst_type, ncols_x, nrows_x, batch, stride_col_y, stride_col_dst,
                              bias, (hipStream_t)stream);
    if (block_len_of(wtype) == 0) return LK_ERR_TYPE;
    if (nrows_x == 0) return LK_OK;
    return run_multi(wtype, 1, &vx, vy_q8_1, &dst, dst_type, ncols_x, &nrows_x, batch, stride_col_y, stride_col_dst,
                     bias ? &bias : nullptr, stream);
}

// The reference's batch-1 Q4_K mat-vec on the matrix unit (cuda/q4k_mmvq_imma.cu:149-175, AMD twin
// cuda/moe/imma_amd.cu:476; declared src/inference/quantized_cuda/mod.rs:29-40). One activation row
// gives a matrix instruction one useful column in thirty-two, and the reference itself no longer
// takes that path (src/inference/quantized_cuda/quantize.rs:35-47): here the name is the Q4_K
// mat-vec launch, which computes the same sums.
extern "C" void q4k_mmvq_imma(const void* vx, const void* vy, void* dst, int ncols_x, int nrows_x, void* stream) {
    if (ncols_x <= 0 || nrows_x <= 0 || ncols_x % 256 != 0) return;
    (void)lk_mmvq(LK_TYPE_Q4_K, vx, vy, dst, LK_TYPE_F32, ncols_x, nrows_x, 1, ncols_x / 32, nrows_x, nullptr, 0, stream);
}

extern "C" int lk_mmvq_multi(int wtype, int count, const void* const* vx, const void* vy_q8_1, void* const* dst,
                             int dst_type, int ncols_x, const int* nrows_x, int batch, int stride_col_y,
                             int stride_col_dst, const float* const* bias, void* stream) {
    if (!vx || !dst || !nrows_x) return LK_ERR_ARG;
    return run_multi(wtype, count, vx, vy_q8_1, dst, dst_type, ncols_x, nrows_x, batch, stride_col_y, stride_col_dst,
                     bias, stream);
}

extern "C" int lk_mmvq_fused(int wtype, int count, const void* const* vx, const float* x, int stride_x,
                             void* const* dst, int dst_type, int ncols_x, const int* nrows_x, int batch,
                             int stride_col_dst, const float* const* bias, void* stream) {
    if (!vx || !dst || !nrows_x || stride_x <= 0) return LK_ERR_ARG;
    return run_multi(wtype, count, vx, x, dst, dst_type, ncols_x, nrows_x, batch, 0, stride_col_dst, bias, stream,
                     stride_x);
}

extern "C" int lk_mmvq_pair_act(int wtype, const void* gate, const void* up, const void* vy_q8_1, void* dst,
                                int dst_type, int ncols_x, int nrows_x, int batch, int stride_col_y,
                                int stride_col_dst, int act, void* stream) {
    if (int rc = check_common(wtype, vy_q8_1, ncols_x, batch, stride_col_y)) return rc;
    if (nrows_x == 0) return LK_OK;
    if (int rc = check_weight(wtype, gate)) return rc;
    if (int rc = check_weight(wtype, up)) return rc;
    if (!dst || nrows_x < 0 || stride_col_dst < nrows_x || (act != 0 && act != 1)) return LK_ERR_ARG;
    if (batch > 4) return LK_ERR_ARG;
    const int nb = ncols_x / block_len_of(wtype);
    if (dst_type != LK_TYPE_F32 && dst_type != LK_TYPE_BF16) return LK_ERR_TYPE;
    const int fit = lk_device().lds_bytes / lds_bytes_of(wtype, nb, 1);
    if (fit < 1) return LK_ERR_ARG;
    if (batch > fit) {   // rows too long to stage the whole batch: one launch per share of it
        for (int b0 = 0; b0 < batch; b0 += fit) {
            const int b = batch - b0 < fit ? batch - b0 : fit;
            const int rc = lk_mmvq_pair_act(wtype, gate, up, (const uint8_t*)vy_q8_1 + (size_t)b0 * stride_col_y * Q81_BYTES,
                                            (uint8_t*)dst + (size_t)b0 * stride_col_dst * (dst_type == LK_TYPE_F32 ? 4 : 2),
                                            dst_type, ncols_x, nrows_x, b, stride_col_y, stride_col_dst, act, stream);
            if (rc != LK_OK) return rc;
        }
        return LK_OK;
    }
    if (wtype == LK_TYPE_Q4_K && batch <= LK_REG_MAX_BATCH && lk_q4k_reg_serves(nb))
        return lk_q4k_reg_pair((const uint8_t*)gate, (const uint8_t*)up, vy_q8_1, 0, dst, dst_type, false, nb, nrows_x, act,
                               batch, stride_col_y, stride_col_dst, (hipStream_t)stream);
    const PairCall c{(const uint8_t*)gate, (const uint8_t*)up, (const uint8_t*)vy_q8_1, dst, nb, nrows_x, stride_col_y,
                     stride_col_dst, act, 0, (hipStream_t)stream};
    switch (wtype) {
        case LK_TYPE_Q4_K: return nb <= 8 ? lk_eng_pair_q4k_short(batch, dst_type, c) : lk_eng_pair_q4k(batch, dst_type, c);
        case LK_TYPE_Q5_K: return lk_eng_pair_q5k(batch, dst_type, c);
        case LK_TYPE_Q6_K: return nb <= 8 ? lk_eng_pair_q6k_short(batch, dst_type, c) : lk_eng_pair_q6k(batch, dst_type, c);
        case LK_TYPE_Q8_0: return lk_eng_pair_q80(batch, dst_type, c);
        default: return LK_ERR_TYPE;
    }
}

extern "C" int lk_mmvq_pair_act_q8_1(int wtype, const void* gate, const void* up, const void* act, int act_is_f32,
                                     int stride_act, void* dst_q8_1, int stride_dst_blocks, int ncols_x, int nrows_x,
                                     int batch, int act_fn, void* stream) {
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (nrows_x == 0) return LK_OK;
    if (!act || !dst_q8_1 || ncols_x <= 0 || ncols_x % bl != 0 || nrows_x < 0 || nrows_x % 32 != 0) return LK_ERR_ARG;
    if (batch < 1 || batch > 4 || stride_dst_blocks < nrows_x / 32 || (act_fn != 0 && act_fn != 1)) return LK_ERR_ARG;
    if (((uintptr_t)dst_q8_1 & 3) != 0) return LK_ERR_ARG;
    if (act_is_f32 ? (stride_act < ncols_x || stride_act % 4 != 0 || ((uintptr_t)act & 15) != 0)
                   : (stride_act < ncols_x / 32 || ((uintptr_t)act & 3) != 0))
        return LK_ERR_ARG;
    if (int rc = check_weight(wtype, gate)) return rc;
    if (int rc = check_weight(wtype, up)) return rc;
    const int nb = ncols_x / bl;
    if (lds_bytes_of(wtype, nb, batch) + 2 * batch * 32 * (int)sizeof(float) > lk_device().lds_bytes) return LK_ERR_ARG;
    // (at two rows the register engine's form of this launch holds one workgroup per CU: it pays while
    // the blocks of 32 output rows fit one round of them; Llama-sized 448 blocks measured 20.5 us against
    // 19.1 on the staged engine)
    if (wtype == LK_TYPE_Q4_K && lk_q4k_reg_serves(nb) && (batch == 1 || (batch == 2 && nrows_x / 32 <= lk_device().cus)))
        return lk_q4k_reg_pair((const uint8_t*)gate, (const uint8_t*)up, act, act_is_f32, dst_q8_1, LK_TYPE_F32, true, nb,
                               nrows_x, act_fn, batch, stride_act, stride_dst_blocks, (hipStream_t)stream);
    const PairCall c{(const uint8_t*)gate, (const uint8_t*)up, (const uint8_t*)act, dst_q8_1, nb, nrows_x,
                     act_is_f32 ? 0 : stride_act, stride_dst_blocks, act_fn, act_is_f32 ? stride_act : 0, (hipStream_t)stream};
    switch (wtype) {
        case LK_TYPE_Q4_K: return lk_eng_pair_q8_1_q4k(batch, c);
        case LK_TYPE_Q5_K: return lk_eng_pair_q8_1_q5k(batch, c);
        case LK_TYPE_Q6_K: return nb <= 8 ? lk_eng_pair_q8_1_q6k_short(batch, c) : lk_eng_pair_q8_1_q6k(batch, c);
        case LK_TYPE_Q8_0: return lk_eng_pair_q8_1_q80(batch, c);
        default: return LK_ERR_TYPE;
    }
}

extern "C" int lk_mmvq_grouped(int wtype, const uint64_t* table, int groups, const void* vy_q8_1, float* dst,
                               int ncols_x, int nrows_x, void* stream) {
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (groups == 0 || nrows_x == 0) return LK_OK;
    if (!table || !vy_q8_1 || !dst || groups < 0 || groups > 65535 || nrows_x < 0 || ncols_x <= 0) return LK_ERR_ARG;
    if (ncols_x % LK_ROW_PADDING != 0 || ncols_x % bl != 0 || ((uintptr_t)vy_q8_1 & 3) != 0) return LK_ERR_ARG;
    const int nb = ncols_x / bl, k32 = ncols_x / 32;
    hipStream_t s = (hipStream_t)stream;
    const uint8_t* y = (const uint8_t*)vy_q8_1;
    switch (wtype) {
        case LK_TYPE_Q4_K:
            return nb <= 8 ? lk_eng_grouped_q4k_short(table, groups, y, dst, nb, nrows_x, k32, s)
                           : lk_eng_grouped_q4k(table, groups, y, dst, nb, nrows_x, k32, s);
        case LK_TYPE_Q5_K: return lk_eng_grouped_q5k(table, groups, y, dst, nb, nrows_x, k32, s);
        case LK_TYPE_Q6_K:
            return nb <= 8 ? lk_eng_grouped_q6k_short(table, groups, y, dst, nb, nrows_x, k32, s)
                           : lk_eng_grouped_q6k(table, groups, y, dst, nb, nrows_x, k32, s);
        default: return lk_eng_grouped_q80(table, groups, y, dst, nb, nrows_x, k32, s);
    }
}

extern "C" int lk_mmvq_subdots(int wtype, const void* vx, const void* vy_q8_1, int32_t* dots,
                               int32_t* sums, int ncols_x, int nrows_x, void* stream) {
    if (lk_is_legacy_type(wtype)) {
        if (int rc = lk_mmvq_subdots_legacy(wtype, vx, vy_q8_1, dots, ncols_x, nrows_x, (hipStream_t)stream)) return rc;
        if (sums) {
            const int k32 = ncols_x / 32;
            hipLaunchKernelGGL(act_sums_kernel, dim3((k32 + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                               (const uint8_t*)vy_q8_1, sums, k32);
        }
        return lk_launch_status();
    }
    const int bl = block_len_of(wtype);
    if (bl == 0) return LK_ERR_TYPE;
    if (!vx || !vy_q8_1 || !dots || ncols_x <= 0 || nrows_x <= 0 || ncols_x % bl != 0) return LK_ERR_ARG;
    if (nrows_x > 65535) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int nb = ncols_x / bl;
    const uint8_t* w = (const uint8_t*)vx;
    const uint8_t* y = (const uint8_t*)vy_q8_1;
    if (wtype == LK_TYPE_Q4_K) {
        hipLaunchKernelGGL(subdots_q4k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else if (wtype == LK_TYPE_Q5_K) {
        hipLaunchKernelGGL(subdots_q5k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else if (wtype == LK_TYPE_Q6_K) {
        hipLaunchKernelGGL(subdots_q6k_kernel, dim3((nb + 7) / 8, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    } else {
        hipLaunchKernelGGL(subdots_q80_kernel, dim3((nb + 31) / 32, nrows_x), dim3(64), 0, s, w, y, dots, nb);
    }
    if (sums) {
        const int k32 = ncols_x / 32;
        hipLaunchKernelGGL(act_sums_kernel, dim3((k32 + 255) / 256), dim3(256), 0, s, y, sums, k32);
    }
    return lk_launch_status();
}

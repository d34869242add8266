// What the tiled-matmul kernels share: the problem record and the one-time kernel set-up.
#pragma once

#include "lk_common.h"

#include <mutex>
#include <unordered_map>

constexpr int MMQ_REC_BYTES = 288;   // workspace record: 256 codes + 8 f16 scales + 8 i16 sums

// One problem = one weight slab against a contiguous run of workspace rows.
struct MmqProblem {
    const uint8_t* w;      // [n][nb] blocks
    const uint8_t* y;      // workspace records
    float* dst;
    const int32_t* ids_dst;  // nullable: destination row of workspace row c
    int64_t nb;            // K steps: 256-value blocks per weight row
    int64_t row_blocks;    // format blocks between consecutive weight rows
    int64_t rows_total;    // rows the workspace was quantized with (record stride)
    int64_t ldd;           // floats between destination rows
    int n, m_begin, m_end;
};

// Raises a kernel's dynamic LDS limit once per process; LK_ERR_ARG when the device has less.
template <typename K>
static int mmq_prepare_kernel(K kernel, int lds_bytes) {
    static std::mutex mu;
    static std::unordered_map<const void*, bool> done;
    std::lock_guard<std::mutex> lock(mu);
    if (done.count((const void*)kernel)) return LK_OK;
    if (lds_bytes > lk_device().lds_bytes) return LK_ERR_ARG;
    if (lds_bytes > 48 * 1024 &&
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        return LK_ERR_LAUNCH;
    }
    done[(const void*)kernel] = true;
    return LK_OK;
}

// What the caller's tmp_fixup holds (FIXUP_BYTES, src/tensor/quantized/kernel_matmul/mmq.rs:42): the
// reference's kernels keep their stream-k partial tiles there, these the partial products of a cut K.
constexpr int64_t MMQ_FIXUP_BYTES = 256ll * 128 * 128 * 4;

// A dense product whose tiles alone leave most of the chip idle is launched with K cut into ranges of
// blocks: a workgroup walks one range and writes its partial tile to part[range] ([token][n] floats in
// the caller's tmp_fixup), and lk_mmq_split_sum adds the ranges in ascending order, so a result does
// not depend on which workgroup finished when. mmq_splits: how many ranges, for `tiles` tiles on a chip
// that holds `slots` workgroups of the kernel at once: as many as bring tiles x ranges to the slots,
// while a range keeps at least two blocks and every partial product fits the buffer. 1 = the plain launch.
static inline int mmq_splits(const MmqProblem& pb, int64_t tiles, int64_t slots, const void* fixup) {
    const int forced = lk_tune_env("LK_TUNE_MMQ_SPLITS");   // measurement runs: -1 never, n > 0 that many where they fit
    if (!fixup || forced < 0 || pb.ids_dst || pb.m_begin != 0) return 1;
    if (pb.n % 4 != 0 || pb.ldd % 4 != 0 || (uintptr_t)pb.dst % 16 != 0 || (uintptr_t)fixup % 16 != 0) return 1;
    const int64_t fit = MMQ_FIXUP_BYTES / ((int64_t)pb.m_end * pb.n * 4);
    int64_t want = forced > 0 ? forced : slots / tiles;
    if (want > fit) want = fit;
    if (want > pb.nb / 2) want = pb.nb / 2;
    return want < 2 ? 1 : (int)want;
}
// dst[token][c] = part[0][token][c] + part[1][token][c] + ..., part[i] m_end x n floats; LK_* status.
int lk_mmq_split_sum(const float* part, int splits, const MmqProblem& pb, hipStream_t s);

// Q4_K against 33 or more token rows (mmq_q4k_f16.hip); `fixup`: the caller's tmp_fixup or null. Return the token-tile width launched,
// 0 when the launch failed, -1 when the operands do not suit these kernels (16-byte alignment,
// 32-bit record offsets) and the caller should take the int8 tiles.
int lk_mmq_q4k_f16_dense(const MmqProblem& pb, hipStream_t s, void* fixup);
// Q4_K against 129 or more token rows on the f16 tiles with four token tiles per wave (mmq_q4k_wide.hip); same returns.
int lk_mmq_q4k_wide_dense(const MmqProblem& pb, hipStream_t s);
void lk_mmq_q4k_wide_release(int device);
int lk_mmq_q4k_f16_moe(const MmqProblem& pb, const uint8_t* w_second, int64_t dst_second, const int32_t* bounds,
                       int64_t stride_expert, int n_experts, int64_t ncols_max, hipStream_t s);

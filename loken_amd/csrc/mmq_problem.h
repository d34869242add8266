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

// Q4_K against 65 or more token rows (mmq_q4k_f16.hip). Return the token-tile width launched,
// 0 when the launch failed, -1 when the operands do not suit these kernels (16-byte alignment,
// 32-bit record offsets) and the caller should take the int8 tiles.
int lk_mmq_q4k_f16_dense(const MmqProblem& pb, hipStream_t s);
// Q4_K against 129 or more token rows on the f16 tiles with four token tiles per wave (mmq_q4k_wide.hip); same returns.
int lk_mmq_q4k_wide_dense(const MmqProblem& pb, hipStream_t s);
void lk_mmq_q4k_wide_release(int device);
int lk_mmq_q4k_f16_moe(const MmqProblem& pb, const uint8_t* w_second, int64_t dst_second, const int32_t* bounds,
                       int64_t stride_expert, int n_experts, int64_t ncols_max, hipStream_t s);

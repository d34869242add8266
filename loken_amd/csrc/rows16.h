// Q4_K / Q5_K x at most sixteen Q8_1 rows in 16-row tiles on the matrix unit (rows16_mfma.hip).
#pragma once
#include "lk_common.h"

struct LkRows16 {
    const uint8_t* w[3];   // matrices sharing the activation (gate and up when `dual`)
    float* dst[3];         // their outputs (`dual`: dst[0] alone)
    int n[3];              // weight rows of each
    int ldd[3];            // floats between output rows
    int count;
    const uint8_t* y;      // Q8_1 rows, stride_y blocks apart
    int nb, m, stride_y;
    int gelu;              // `dual`: 0 SiLU, 1 tanh-form GELU
    uint8_t* q81_dst;      // `dual` only, when given: the result as Q8_1 rows (blocks of 32 consecutive output
    int q81_stride;        // rows, q81_stride blocks between rows) instead of f32 in dst[0]; n a multiple of 32
};
// True when the launch takes `size_m` activation rows of `nb` super-blocks (their codes fit in LDS).
bool lk_rows16_serves(int size_m, int nb);
int lk_rows16_launch(const LkRows16& a, bool dual, bool q5, hipStream_t stream);

// Q4_K per expert over a sorted routing, a wave per 16-row tile (rows16_moe.hip): expert e's matrices are
// a.w[..] + e * expert_bytes (a.n[0] rows each, a.w[1] with `dual`), its rows the sorted rows
// [bounds[e], bounds[e + 1]) (`src`: sorted row -> row of a.y, `dst_map`: sorted row -> output row; either
// may be null: the sorted row itself). `rows_hint`: the rows an expert is expected to own (up to 8: passes
// of 8; up to 16: passes of 16). LK_* status, or -1 when the launch does not serve the call (rows of a
// super-block count it is not compiled for, more rows expected).
struct LkRows16Experts {
    const int32_t* bounds;
    const int32_t* src;
    const int32_t* dst_map;
    int64_t expert_bytes;
};
int lk_rows16_launch_experts(const LkRows16& a, const LkRows16Experts& m, int n_experts, bool dual, int rows_hint,
                             hipStream_t stream);

// Q6_K x at most 64 Q8_1 rows in 16-row tiles (rows16_q6k.hip; above eight rows possibly as sets of eight rows
// over the same weights). LK_* status, or -1 when the launch does not serve the call (more rows, k not a
// multiple of 2048, rows whose codes do not fit in LDS, above 16 rows a matrix of more than 64 MB or of more 16-row tiles than CUs, above 32 rows
// anything but whole rounds of resident workgroups).
int lk_rows16_q6k(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k, int stride_y, int ldd,
                  hipStream_t stream);

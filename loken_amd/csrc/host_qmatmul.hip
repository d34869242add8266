// Host mirror of loken's QKernelMatMul for the card path: see include/loken_host.hpp.

#include "../../include/loken_host.hpp"

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <map>
#include <type_traits>
#include <mutex>

namespace loken {
namespace {

constexpr int Q81_BLOCK = 36;
constexpr size_t MMQ_RECORD = 144;                      // bytes per 128 padded values per row
constexpr size_t FIXUP_BYTES = 256u * 128u * 128u * 4u;  // kernel_matmul/mmq.rs:42

size_t pad_to(size_t v, size_t m) { return (v + m - 1) / m * m; }

// One device's buffers. `mu` is held across a quantize -> consume pair so that two host threads
// sharing the card's stream cannot interleave their pairs (fast_mmvq.rs:15-32,
// kernel_matmul/mmq.rs:43-86); `last_use` orders a later user on ANOTHER stream behind the
// kernels enqueued here (the host mutex alone orders only the enqueueing).
struct Slot {
    std::mutex mu;
    void* act = nullptr;      // Q8_1 rows / tiled-matmul workspace
    size_t act_bytes = 0;
    void* fixup = nullptr;
    void* out32 = nullptr;    // f32 result rows of a call whose rows came in f16 / bf16 (the matrix-unit kernels write f32)
    size_t out32_bytes = 0;
    hipEvent_t last_use = nullptr;
    bool used = false;
};

std::mutex g_slots_mu;
std::map<int, Slot*> g_slots;

Slot& slot_of(int device) {
    std::lock_guard<std::mutex> lock(g_slots_mu);
    auto it = g_slots.find(device);
    if (it != g_slots.end()) return *it->second;
    Slot* s = new Slot();
    g_slots.emplace(device, s);
    return *s;
}

bool capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

// Grow-only, zero-filled. Never grows while `stream` records a graph (an allocation is not a
// capturable operation): the caller warms the size up outside the capture, as with the MoE scratch.
int reserve(Slot& slot, size_t bytes, bool want_fixup, hipStream_t stream) {
    const bool rec = capturing(stream);
    if (slot.act_bytes < bytes) {
        if (rec) return LK_ERR_NOMEM;
        if (slot.act) {   // release the smaller one first: no double peak (kernel_matmul/mmq.rs:49-53)
            if (hipStreamSynchronize(stream) != hipSuccess || hipFree(slot.act) != hipSuccess) (void)hipGetLastError();
            slot.act = nullptr;
            slot.act_bytes = 0;
        }
        if (hipMalloc(&slot.act, bytes) != hipSuccess) {
            (void)hipGetLastError();
            slot.act = nullptr;
            return LK_ERR_NOMEM;
        }
        slot.act_bytes = bytes;
        if (hipMemsetAsync(slot.act, 0, bytes, stream) != hipSuccess) (void)hipGetLastError();
    }
    if (want_fixup && !slot.fixup) {
        if (rec) return LK_ERR_NOMEM;
        if (hipMalloc(&slot.fixup, FIXUP_BYTES) != hipSuccess) {
            (void)hipGetLastError();
            slot.fixup = nullptr;
            return LK_ERR_NOMEM;
        }
        if (hipMemsetAsync(slot.fixup, 0, FIXUP_BYTES, stream) != hipSuccess) (void)hipGetLastError();
    }
    if (!slot.last_use && !rec) {
        if (hipEventCreateWithFlags(&slot.last_use, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            slot.last_use = nullptr;
        }
    }
    // queue behind whoever used the buffers last; a graph being recorded neither waits nor marks
    if (slot.used && slot.last_use && !rec && hipStreamWaitEvent(stream, slot.last_use, 0) != hipSuccess)
        (void)hipGetLastError();
    return LK_OK;
}

// The f32 rows a half-precision call's kernels write before they are narrowed into the caller's buffer.
int reserve_out32(Slot& slot, size_t bytes, hipStream_t stream) {
    if (slot.out32_bytes >= bytes) return LK_OK;
    if (capturing(stream)) return LK_ERR_NOMEM;
    if (slot.out32) {
        if (hipStreamSynchronize(stream) != hipSuccess || hipFree(slot.out32) != hipSuccess) (void)hipGetLastError();
        slot.out32 = nullptr;
        slot.out32_bytes = 0;
    }
    if (hipMalloc(&slot.out32, bytes) != hipSuccess) {
        (void)hipGetLastError();
        slot.out32 = nullptr;
        return LK_ERR_NOMEM;
    }
    slot.out32_bytes = bytes;
    return LK_OK;
}

template <typename T>
__global__ __launch_bounds__(256) void narrow_rows_kernel(const float* __restrict__ from, T* __restrict__ to, size_t count) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    if constexpr (sizeof(T) == 2 && std::is_same<T, __half>::value) to[i] = __float2half_rn(from[i]);
    else to[i] = __float2bfloat16(from[i]);
}

// out (f16 / bf16) = the f32 rows, rounded to nearest: the conversion the reference applies to the
// f32 rows mmq_forward returns (src/tensor/quantized/kernel_matmul.rs:1086-1714, output dtype follows input).
int narrow_rows(const float* from, void* to, int type, size_t count, hipStream_t stream) {
    const unsigned grid = (unsigned)((count + 255) / 256);
    if (type == LK_TYPE_F16) hipLaunchKernelGGL(narrow_rows_kernel<__half>, dim3(grid), dim3(256), 0, stream, from, (__half*)to, count);
    else hipLaunchKernelGGL(narrow_rows_kernel<__hip_bfloat16>, dim3(grid), dim3(256), 0, stream, from, (__hip_bfloat16*)to, count);
    return hipGetLastError() == hipSuccess ? LK_OK : LK_ERR_LAUNCH;
}

void mark_used(Slot& slot, hipStream_t stream) {
    if (slot.last_use && !capturing(stream)) {
        if (hipEventRecord(slot.last_use, stream) != hipSuccess) (void)hipGetLastError();
        slot.used = true;
    }
}

// The 32-value nibble formats and the two-bit K-quants: served by the plain mat-vec (four of them by the
// tiled matmul as well, and Q2_K / Q3_K, from the row counts of nibble_tiles_pay below).
bool matvec_only(int dtype) {
    return dtype == LK_TYPE_Q4_0 || dtype == LK_TYPE_Q4_1 || dtype == LK_TYPE_Q5_0 || dtype == LK_TYPE_Q5_1 ||
           dtype == LK_TYPE_IQ4_NL || dtype == LK_TYPE_MXFP4 || dtype == LK_TYPE_Q2_K || dtype == LK_TYPE_Q3_K ||
           dtype == LK_TYPE_IQ4_XS;
}

bool nibble_tiles(int dtype) {
    return dtype == LK_TYPE_Q4_0 || dtype == LK_TYPE_Q4_1 || dtype == LK_TYPE_Q5_0 || dtype == LK_TYPE_Q5_1 || dtype == LK_TYPE_Q3_K ||
           dtype == LK_TYPE_Q2_K;
}

bool tiled_serves(int dtype, int k) {
    return (dtype == LK_TYPE_Q4_K || dtype == LK_TYPE_Q5_K || dtype == LK_TYPE_Q6_K || dtype == LK_TYPE_Q8_0 || nibble_tiles(dtype)) &&
           k % 256 == 0;
}

// Q4_0 / Q4_1 / Q5_0 / Q5_1, Q3_K and Q2_K above eight rows: one tiled launch (with K cut into ranges
// where its tiles are few, mmq_problem.h) against mat-vec launches of eight rows each. Measured on MI355X,
// quantizer included, mat-vec against tiled: Q4_0 4096 x 4096 at 9 / 16 / 32 rows 29 / 35 / 55 us against
// 31 / 27 / 29; 14336 x 4096 at 9 / 16 rows 42 / 58 against 37 / 38; 4096 x 14336 at 9 rows 57 against 41;
// 1024 x 4096 at 9 / 16 rows 27 / 31 against 33 / 26. Q5_1, Q3_K and Q2_K alike (Q3_K 4096 x 4096 at 9 / 16
// rows 31 / 40 against 29 / 27). So: from 16 rows, and from 9 on a matrix of 48 M weights or more.
bool nibble_tiles_pay(int dtype, int n, int k, int rows) {
    if (!nibble_tiles(dtype) || k % 256 != 0) return false;
    return rows >= 16 || (long long)n * k >= (48ll << 20);
}

size_t elem_bytes(int type) { return type == LK_TYPE_F32 ? 4 : 2; }

}  // namespace

int matvec_rows(int dtype, int k) {
    if ((dtype == LK_TYPE_Q4_K || dtype == LK_TYPE_Q5_K || dtype == LK_TYPE_Q6_K) && k % 256 == 0) return 8;
    // Q8_0, mat-vec launches of eight rows against the tiled matmul: 4096 x 4096 at 16 / 24 / 32 rows 32 / 40 /
    // 49 us against 32 / 32 / 32; 14336 x 4096 51 / 70 / 89 against 56 / 56 / 58
    return dtype == LK_TYPE_Q8_0 && tiled_serves(dtype, k) ? 16 : 8;
}

// Rows the matrix-unit rows kernels take before the tiled matmul does. Measured on MI355X over
// n = 2048 ... 151936 and k = 2048 ... 14336: a rows kernel re-reads the weights for every 32
// activation rows but fills the chip from the first pass; a tiled launch holds a 128- or 256-row weight
// block per workgroup, cuts K into ranges while its tiles are fewer than the chip's workgroup slots
// (mmq_problem.h) and pays one more pass over the partial products for that. Up to 16 rows the 16-row
// tiles stay; above, the two meet near n x rows = 450 K at k <= 4096 and in proportion earlier for
// longer rows (quantizer + kernel, rows kernel against tiled):
//   Q4_K  4096 x 4096: 128 rows 36 us against 39, 256 rows 49 against 43; 14336 x 4096: 32 rows 36
//         against 36, 128 rows 75 against 53; 4096 x 14336: 32 rows 52 against 39, 512 rows 207 against 127
//   Q6_K  4096 x 4096: 64 rows 32 against 35, 256 rows 64 against 51; 14336 x 4096: 32 rows 44 against 40,
//         256 rows 161 against 114; 4096 x 14336: 32 rows 54 against 42, 1024 rows 568 against 360
//   Q5_K  4096 x 4096: 128 rows 37 against 41, 256 rows 52 against 48; 4096 x 14336: 128 rows 80 against 63
// `bench.py --workload rows-sweep` prints the table for a shape.
static bool rows_kernel_serves(int dtype, int n, int k, int rows) {
    if (dtype != LK_TYPE_Q4_K && dtype != LK_TYPE_Q5_K && dtype != LK_TYPE_Q6_K) return false;
    // (a matrix of fewer than 2048 rows yields few tiles whatever the cut: Q4_K 1024 x 4096 at 512 rows 38 us
    // against 38, at 1024 rows 55 against 49)
    const long long few = n < 2048 ? 2048 / (n > 0 ? n : 1) : 1;
    // (Q4_K / Q5_K rows of 8192 values or more at 9 to 16 activation rows: the 16-row tiles' second set of eight
    // costs them more than the cut K costs the tiled launch: 4096 x 14336 at 9 / 16 rows 42 / 46 us against 37,
    // Q5_K 44 / 48 against 38; 4096 x 8192 31 / 33 against 30. Q6_K keeps its 16-row tiles: 38 against 40)
    if (dtype != LK_TYPE_Q6_K && rows > 8 && rows <= 16 && k >= 8192 && n >= 2048) return false;
    return rows <= 16 || (long long)n * rows * (k > 4096 ? k : 4096) <= 450000ll * 4096 * few;
}

// The K-quants at 3 to 8 f32 rows: the 16-row tiles of the matrix-unit kernels (their time hardly moves
// with the row count) against mat-vec launches (whose dot work grows with every row). Every workgroup of
// a rows kernel stages all the rows, so the matrix has to be large enough to pay for that. Measured on
// MI355X, Q4_K / Q5_K, k = 4096: 14336 rows from 4 activation rows, 4096 rows from 8, 1024 rows never;
// k = 2048: 2048 rows from 4, 6144 and 151936 rows from 3. Q6_K (k a multiple of 2048: its rows are loaded
// in granules of eight super-blocks): 4096 x 14336 and 151936 x 2048 from 3 rows, 14336 x 4096 from 4,
// 4096 x 4096 and 2048 x 6144 from 7 (as two sets of four rows: 8.9 us against 9.5 at 8 rows, 8.1 as mat-vec at 6).
static bool small_rows_kernel_pays(int dtype, int n, int k, int rows) {
    if (rows < 3 || rows > 8 || k % 256 != 0) return false;
    if (dtype == LK_TYPE_Q6_K) return k % 2048 == 0 && ((long long)n * k >= (48ll << 20) || (rows >= 7 && n >= 1024));
    if (dtype != LK_TYPE_Q4_K && dtype != LK_TYPE_Q5_K) return false;
    return (long long)n * rows >= (k <= 2048 ? 8192 : 57344);
}

QKernelMatMul::QKernelMatMul(int dtype, int n, int k, const void* blob, int device)
    : dtype_(dtype), n_(n), k_(k), device_(device), blob_(blob) {}

int QKernelMatMul::forward(const void* x, int x_type, int rows, void* out, void* stream_ptr, bool decode_order) {
    last_path_ = Path::None;
    hipStream_t stream = (hipStream_t)stream_ptr;
    const bool plain = matvec_only(dtype_);
    if (!plain && dtype_ != LK_TYPE_Q4_K && dtype_ != LK_TYPE_Q5_K && dtype_ != LK_TYPE_Q6_K && dtype_ != LK_TYPE_Q8_0) return LK_ERR_TYPE;
    if (x_type != LK_TYPE_F32 && x_type != LK_TYPE_F16 && x_type != LK_TYPE_BF16) return LK_ERR_TYPE;
    if (rows == 0) return LK_OK;
    if (!x || !out || !blob_ || rows < 0 || n_ <= 0 || k_ <= 0) return LK_ERR_ARG;
    const int block_len = dtype_ == LK_TYPE_Q8_0 || (plain && dtype_ != LK_TYPE_Q2_K && dtype_ != LK_TYPE_Q3_K && dtype_ != LK_TYPE_IQ4_XS) ? 32 : 256;
    if (k_ % block_len != 0) return LK_ERR_ARG;
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current != device_) {
        (void)hipGetLastError();
        return LK_ERR_ARG;   // "input on a different device" (kernel_matmul.rs:1499-1503)
    }
    const int mv_max = matvec_rows(dtype_, k_);
    Slot& slot = slot_of(device_);

    // --- mat-vec family: up to matvec_rows, or any count when every row must sum like a one-row call
    const bool rows_kernel_fits = k_ % 256 == 0 && ((uintptr_t)blob_ & (dtype_ == LK_TYPE_Q6_K ? 1 : 15)) == 0;
    const bool to_rows_kernel = rows_kernel_fits && small_rows_kernel_pays(dtype_, n_, k_, rows);
    const bool to_nibble_tiles = !decode_order && nibble_tiles_pay(dtype_, n_, k_, rows) &&
                                 ((uintptr_t)blob_ & (dtype_ == LK_TYPE_Q2_K ? 3 : 1)) == 0;
    auto matvec = [&]() -> int {
        if (!plain && x_type == LK_TYPE_F32 && rows <= 2 && k_ <= 8192 && ((uintptr_t)x & 15) == 0 && k_ % 4 == 0) {
            const void* vx[1] = {blob_};
            void* dst[1] = {out};
            const int nn[1] = {n_};
            last_path_ = Path::MatVecFused;
            return lk_mmvq_fused(dtype_, 1, vx, (const float*)x, k_, dst, x_type, k_, nn, rows, n_, nullptr, stream);
        }
        const int k_padded = (int)pad_to((size_t)k_, 512), blocks = k_padded / 32;
        std::lock_guard<std::mutex> pair(slot.mu);
        if (int rc = reserve(slot, (size_t)rows * blocks * Q81_BLOCK, false, stream)) return rc;
        if (int rc = lk_quantize_q8_1(x, x_type, slot.act, k_, k_padded, rows, stream)) return rc;
        for (int r0 = 0; r0 < rows; r0 += 8) {
            const int b = rows - r0 < 8 ? rows - r0 : 8;
            const int rc = lk_mmvq(dtype_, blob_, (const uint8_t*)slot.act + (size_t)r0 * blocks * Q81_BLOCK,
                                   (uint8_t*)out + (size_t)r0 * n_ * elem_bytes(x_type), x_type, k_, n_, b, blocks, n_,
                                   nullptr, decode_order ? 1 : 0, stream);
            if (rc) return rc;
        }
        mark_used(slot, stream);
        last_path_ = Path::MatVec;
        return LK_OK;
    };
    if ((rows <= mv_max && !to_rows_kernel) || decode_order || (plain && !to_nibble_tiles)) return matvec();

    // The matrix-unit kernels write f32 rows. Rows that came in f16 / bf16 leave in that type, as the
    // reference's do (the f32 rows its mmq_forward returns are narrowed by the caller,
    // src/tensor/quantized/kernel_matmul.rs:1086-1714): the kernels write into a buffer of the
    // device's slot and one more launch rounds them into `out`.
    const bool half_rows = x_type != LK_TYPE_F32;
    const size_t out_count = (size_t)rows * n_;

    // --- a handful of rows (or a matrix too small to fill the chip with tiles): matrix unit, weights
    //     straight from HBM
    if (rows_kernel_serves(dtype_, n_, k_, rows) && rows_kernel_fits) {
        const int blocks = k_ / 32;
        int rc;
        {
            std::lock_guard<std::mutex> pair(slot.mu);
            if (int r = reserve(slot, (size_t)rows * blocks * Q81_BLOCK, false, stream)) return r;
            if (half_rows)
                if (int r = reserve_out32(slot, out_count * 4, stream)) return r;
            float* dst = half_rows ? (float*)slot.out32 : (float*)out;
            if (int r = lk_quantize_q8_1(x, x_type, slot.act, k_, k_, rows, stream)) return r;
            // the launchers with a status (the exported void forms drop it): rows too long for their scale
            // tables in LDS launch nothing, and the call goes on to the mat-vec or the tiled matmul below
            rc = dtype_ == LK_TYPE_Q4_K   ? lk_dense_q4k_rows(blob_, slot.act, dst, rows, n_, k_, stream)
                 : dtype_ == LK_TYPE_Q5_K ? lk_dense_q5k_rows(blob_, slot.act, dst, rows, n_, k_, stream)
                                          : lk_dense_q6k_rows(blob_, slot.act, dst, rows, n_, k_, stream);
            if (rc == LK_OK && half_rows) rc = narrow_rows(dst, out, x_type, out_count, stream);
            mark_used(slot, stream);
        }
        if (rc == LK_OK) {
            last_path_ = Path::RowsOnMatrixUnit;
            return LK_OK;
        }
        if (rc != LK_ERR_ARG) return rc;
        if (rows <= mv_max) return matvec();   // a few rows the rows kernel declined: not worth a tile
    }

    // --- tiled matmul (mmq_forward, kernel_matmul/mmq.rs:21-159)
    if (!tiled_serves(dtype_, k_)) return LK_ERR_TYPE;
    const size_t k_padded = pad_to(pad_to((size_t)k_, 512), 128);
    const size_t ws_bytes = (size_t)rows * (k_padded / 128) * MMQ_RECORD + 128 * MMQ_RECORD;
    std::lock_guard<std::mutex> pair(slot.mu);
    if (int rc = reserve(slot, ws_bytes, true, stream)) return rc;
    if (half_rows)
        if (int rc = reserve_out32(slot, out_count * 4, stream)) return rc;
    void* dst = half_rows ? slot.out32 : out;
    // the layouts of the reference's table (quantized/mmq.rs:274-285)
    auto quantizer = dtype_ == LK_TYPE_Q2_K ? launch_mmq_quantize_q8_1_D2S6
                     : dtype_ == LK_TYPE_Q6_K || dtype_ == LK_TYPE_Q8_0 || dtype_ == LK_TYPE_Q5_0 || dtype_ == LK_TYPE_Q3_K
                         ? launch_mmq_quantize_q8_1_D4
                         : launch_mmq_quantize_q8_1_DS4;
    quantizer(x, nullptr, slot.act, x_type, k_, k_, 0, 0, (int64_t)k_padded, rows, 1, 1, stream);
    auto launcher = dtype_ == LK_TYPE_Q4_K   ? launch_mmq_gguf_q4_k
                    : dtype_ == LK_TYPE_Q5_K ? launch_mmq_gguf_q5_k
                    : dtype_ == LK_TYPE_Q6_K ? launch_mmq_gguf_q6_k
                    : dtype_ == LK_TYPE_Q4_0 ? launch_mmq_gguf_q4_0
                    : dtype_ == LK_TYPE_Q4_1 ? launch_mmq_gguf_q4_1
                    : dtype_ == LK_TYPE_Q5_0 ? launch_mmq_gguf_q5_0
                    : dtype_ == LK_TYPE_Q5_1 ? launch_mmq_gguf_q5_1
                    : dtype_ == LK_TYPE_Q3_K ? launch_mmq_gguf_q3_k
                    : dtype_ == LK_TYPE_Q2_K ? launch_mmq_gguf_q2_k
                                             : launch_mmq_gguf_q8_0;
    int abi = 0, cus = 0, lds = 0, wave = 0;
    (void)lk_device_info(&abi, &cus, &lds, &wave);
    const int tile = launcher(slot.fixup, blob_, slot.act, dst, k_, n_, rows, k_ / block_len, n_, 0x1000950, cus, lds, wave,
                              stream);
    int narrowed = LK_OK;
    if (tile != 0 && half_rows) narrowed = narrow_rows((const float*)dst, out, x_type, out_count, stream);
    mark_used(slot, stream);
    if (tile == 0) return LK_ERR_ARG;   // "no tile fits, nothing ran": the reference falls back to dequantized
    if (narrowed != LK_OK) return narrowed;
    last_path_ = Path::Tiled;
    return LK_OK;
}

// takes_matvec of the reference (kernel_matmul.rs:1069-1075) with this mirror's own exceptions: the
// K-quants' few rows over a large matrix go to the 16-row tiles, and the formats with tiles leave the
// mat-vec launches from nibble_tiles_pay's row counts.
bool QKernelMatMul::takes_matvec(int rows, bool decode_order) const {
    if (!blob_ || rows < 1) return false;
    if (decode_order && rows > 1) return true;
    const bool plain = matvec_only(dtype_);
    if (plain) return !nibble_tiles_pay(dtype_, n_, k_, rows) || rows <= matvec_rows(dtype_, k_);
    if (rows > matvec_rows(dtype_, k_)) return false;
    const bool rows_kernel_fits = k_ % 256 == 0 && ((uintptr_t)blob_ & (dtype_ == LK_TYPE_Q6_K ? 1 : 15)) == 0;
    return !(rows_kernel_fits && small_rows_kernel_pays(dtype_, n_, k_, rows));
}

size_t QKernelMatMul::quantized_bytes(int k, int rows) {
    return k > 0 && rows > 0 ? (size_t)rows * (pad_to((size_t)k, 512) / 32) * Q81_BLOCK : 0;
}

int QKernelMatMul::quantize_for_matvec(const void* x, int x_type, int rows, void* q81, void* stream, QuantizedActivation* a,
                                       bool decode_order) const {
    if (!x || !q81 || !a || rows <= 0) return LK_ERR_ARG;
    if (x_type != LK_TYPE_F32 && x_type != LK_TYPE_F16 && x_type != LK_TYPE_BF16) return LK_ERR_TYPE;
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current != device_) {
        (void)hipGetLastError();
        return LK_ERR_ARG;
    }
    if (!takes_matvec(rows, decode_order)) return LK_NOT_TAKEN;
    const int k_padded = (int)pad_to((size_t)k_, 512);
    if (int rc = lk_quantize_q8_1(x, x_type, q81, k_, k_padded, rows, stream)) return rc;
    a->q81 = q81;
    a->k = k_;
    a->rows = rows;
    a->device = device_;
    a->x_type = x_type;
    return LK_OK;
}

int QKernelMatMul::forward_quantized(const QuantizedActivation& a, void* out, void* stream, bool decode_order) {
    last_path_ = Path::None;
    if (!a.q81 || !out) return LK_ERR_ARG;
    if (a.k != k_ || a.device != device_ || !takes_matvec(a.rows, decode_order)) return LK_NOT_TAKEN;
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current != device_) {
        (void)hipGetLastError();
        return LK_ERR_ARG;
    }
    const int blocks = (int)pad_to((size_t)k_, 512) / 32;
    for (int r0 = 0; r0 < a.rows; r0 += 8) {
        const int b = a.rows - r0 < 8 ? a.rows - r0 : 8;
        const int rc = lk_mmvq(dtype_, blob_, (const uint8_t*)a.q81 + (size_t)r0 * blocks * Q81_BLOCK,
                               (uint8_t*)out + (size_t)r0 * n_ * elem_bytes(a.x_type), a.x_type, k_, n_, b, blocks, n_,
                               nullptr, decode_order ? 1 : 0, stream);
        if (rc) return rc;
    }
    last_path_ = Path::MatVec;
    return LK_OK;
}

int QKernelMatMul::forward_quantized_pair(QKernelMatMul& other, const QuantizedActivation& a, void* out0, void* out1,
                                          void* stream) {
    last_path_ = other.last_path_ = Path::None;
    if (!a.q81 || !out0 || !out1) return LK_ERR_ARG;
    if (a.k != k_ || other.k_ != k_ || a.rows != 1 || a.x_type != LK_TYPE_F32 || dtype_ != other.dtype_ ||
        device_ != other.device_ || a.device != device_ || !takes_matvec(1, false) || !other.takes_matvec(1, false))
        return LK_NOT_TAKEN;
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current != device_) {
        (void)hipGetLastError();
        return LK_ERR_ARG;
    }
    const void* vx[2] = {blob_, other.blob_};
    void* dst[2] = {out0, out1};
    const int nn[2] = {n_, other.n_};
    const int blocks = (int)pad_to((size_t)k_, 512) / 32;
    const int rc = lk_mmvq_multi(dtype_, 2, vx, a.q81, dst, LK_TYPE_F32, k_, nn, 1, blocks, n_ > other.n_ ? n_ : other.n_, nullptr,
                                 stream);
    if (rc == LK_ERR_TYPE) return LK_NOT_TAKEN;   // a format without the several-matrices launch
    if (rc) return rc;
    last_path_ = other.last_path_ = Path::MatVec;
    return LK_OK;
}

void release_workspaces() {
    std::lock_guard<std::mutex> lock(g_slots_mu);
    int current = 0;
    (void)hipGetDevice(&current);
    for (auto& kv : g_slots) {
        Slot& s = *kv.second;
        std::lock_guard<std::mutex> pair(s.mu);
        if (hipSetDevice(kv.first) != hipSuccess) { (void)hipGetLastError(); continue; }
        (void)hipDeviceSynchronize();
        if (s.act) (void)hipFree(s.act);
        if (s.fixup) (void)hipFree(s.fixup);
        if (s.out32) (void)hipFree(s.out32);
        s.out32 = nullptr;
        s.out32_bytes = 0;
        if (s.last_use) (void)hipEventDestroy(s.last_use);
        s.act = s.fixup = nullptr;
        s.act_bytes = 0;
        s.last_use = nullptr;
        s.used = false;
    }
    (void)hipSetDevice(current);
    (void)hipGetLastError();
}

}  // namespace loken

extern "C" void* lkh_qkernel_matmul_new(int dtype, int n, int k, const void* blob, int device) {
    return new loken::QKernelMatMul(dtype, n, k, blob, device);
}
extern "C" void lkh_qkernel_matmul_free(void* handle) { delete (loken::QKernelMatMul*)handle; }
extern "C" int lkh_qkernel_matmul_forward(void* handle, const void* x, int x_type, int rows, void* out, void* stream,
                                          int decode_order) {
    if (!handle) return LK_ERR_ARG;
    return ((loken::QKernelMatMul*)handle)->forward(x, x_type, rows, out, stream, decode_order != 0);
}
extern "C" int lkh_qkernel_matmul_last_path(void* handle) {
    return handle ? (int)((loken::QKernelMatMul*)handle)->last_path() : 0;
}
extern "C" size_t lkh_quantized_activation_bytes(int k, int rows) { return loken::QKernelMatMul::quantized_bytes(k, rows); }
extern "C" int lkh_qkernel_matmul_quantize_for_matvec(void* handle, const void* x, int x_type, int rows, void* q81, void* stream,
                                                      int decode_order) {
    if (!handle) return LK_ERR_ARG;
    loken::QKernelMatMul::QuantizedActivation a;
    return ((loken::QKernelMatMul*)handle)->quantize_for_matvec(x, x_type, rows, q81, stream, &a, decode_order != 0);
}
namespace {
loken::QKernelMatMul::QuantizedActivation activation_of(const loken::QKernelMatMul& m, const void* q81, int x_type, int rows) {
    loken::QKernelMatMul::QuantizedActivation a;
    a.q81 = q81;
    a.k = m.k();
    a.rows = rows;
    a.x_type = x_type;
    (void)hipGetDevice(&a.device);   // the rows were quantized on the current card
    return a;
}
}  // namespace
extern "C" int lkh_qkernel_matmul_forward_quantized(void* handle, const void* q81, int x_type, int rows, void* out, void* stream,
                                                    int decode_order) {
    if (!handle) return LK_ERR_ARG;
    if (x_type != LK_TYPE_F32 && x_type != LK_TYPE_F16 && x_type != LK_TYPE_BF16) return LK_ERR_TYPE;
    auto* m = (loken::QKernelMatMul*)handle;
    return m->forward_quantized(activation_of(*m, q81, x_type, rows), out, stream, decode_order != 0);
}
extern "C" int lkh_qkernel_matmul_forward_quantized_pair(void* handle, void* other, const void* q81, void* out0, void* out1,
                                                         void* stream) {
    if (!handle || !other) return LK_ERR_ARG;
    auto* m = (loken::QKernelMatMul*)handle;
    return m->forward_quantized_pair(*(loken::QKernelMatMul*)other, activation_of(*m, q81, LK_TYPE_F32, 1), out0, out1, stream);
}
extern "C" int lkh_matvec_rows(int dtype, int k) { return loken::matvec_rows(dtype, k); }
extern "C" void lkh_release_workspaces(void) { loken::release_workspaces(); }

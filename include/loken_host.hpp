/* Host side of the quantized linear above the C ABI of loken_gfx950.h, in C++: the mirror of
 * loken's QKernelMatMul for the card path (src/tensor/quantized/kernel_matmul.rs:1086-1714,
 * kernel_matmul/mmq.rs:21-159): which kernel family a call takes by its row count, the grow-only
 * per-device workspaces with the host mutex held across a quantize -> consume pair of launches,
 * and the event that orders workspace reuse between streams. Rust is what the reference's host is
 * written in; this is the same logic for a C++ caller, and what the Rust shim of INTEGRATION.md
 * would keep doing on its own side.
 *
 * Device pointers in, device pointers out; nothing here synchronizes the host with the device. */
#ifndef LOKEN_HOST_HPP
#define LOKEN_HOST_HPP

#include <stdint.h>

#include "loken_gfx950.h"

namespace loken {

/* Which launchers a forward call went through. */
enum class Path : int {
    None = 0,
    MatVecFused = 1,   /* lk_mmvq_fused: f32 rows quantized inside the mat-vec launch */
    MatVec = 2,        /* lk_quantize_q8_1 + lk_mmvq (slices of eight rows) */
    RowsOnMatrixUnit = 3, /* lk_quantize_q8_1 + loken_dense_q4k_imma_m8_plain */
    Tiled = 4,         /* launch_mmq_quantize_q8_1_* + launch_mmq_gguf_* */
};

/* The most rows the mat-vec family takes for this weight before the call moves to a matrix-unit
 * kernel (matvec_rows of the reference, kernel_matmul.rs:27-33, with the crossovers measured on
 * MI355X: Q4_K 6 rows, then the rows kernel up to 64, then the tiled matmul; Q6_K / Q8_0 mat-vec
 * slices up to 32 rows, then the tiled matmul). */
int matvec_rows(int dtype, int k);

class QKernelMatMul {
public:
    /* `blob`: device address of `n` rows of `k` values in GGUF blocks of `dtype` (LK_TYPE_Q4_K /
     * Q6_K / Q8_0), owned by the caller, on device `device`. */
    QKernelMatMul(int dtype, int n, int k, const void* blob, int device);

    /* x [rows, k] (LK_TYPE_F32; F16 / BF16 for calls that stay on the mat-vec family) ->
     * out [rows, n] in x's type, on `stream`. `decode_order` keeps every row on the mat-vec
     * kernels whatever the count (DecodeOrder of the reference, kernel_matmul.rs:34-75).
     * Returns LK_OK or an LK_ERR_* code; never throws, never aborts. */
    int forward(const void* x, int x_type, int rows, void* out, void* stream, bool decode_order = false);

    Path last_path() const { return last_path_; }
    int n() const { return n_; }
    int k() const { return k_; }

private:
    int dtype_, n_, k_, device_;
    const void* blob_;
    Path last_path_ = Path::None;
};

/* Frees every workspace this layer holds on every device (synchronizes those devices). */
void release_workspaces();

}  // namespace loken

/* The same through plain C, for callers and tests that bind by symbol. */
extern "C" {
void* lkh_qkernel_matmul_new(int dtype, int n, int k, const void* blob, int device);
void lkh_qkernel_matmul_free(void* handle);
int lkh_qkernel_matmul_forward(void* handle, const void* x, int x_type, int rows, void* out, void* stream,
                               int decode_order);
int lkh_qkernel_matmul_last_path(void* handle);
int lkh_matvec_rows(int dtype, int k);
void lkh_release_workspaces(void);
}

#endif

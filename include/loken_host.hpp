/* Host side of the quantized linear above the C ABI of loken_gfx950.h, in C++: the mirror of
 * loken's QKernelMatMul for the card path (src/tensor/quantized/kernel_matmul.rs:1086-1714,
 * kernel_matmul/mmq.rs:21-159): which kernel family a call takes by its row count, the grow-only
 * per-device workspaces with the host mutex held across a quantize -> consume pair of launches,
 * and the event that orders workspace reuse between streams. Rust is what the reference's host is
 * written in; this is the same logic for a C++ caller, and what a Rust binding to this library
 * would keep doing on its own side.
 *
 * Device pointers in, device pointers out; nothing here synchronizes the host with the device. */
#ifndef LOKEN_HOST_HPP
#define LOKEN_HOST_HPP

#include <stdint.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "loken_gfx950.h"

namespace loken {

/* Which launchers a forward call went through. */
enum class Path : int {
    None = 0,
    MatVecFused = 1,   /* lk_mmvq_fused: f32 rows quantized inside the mat-vec launch */
    MatVec = 2,        /* lk_quantize_q8_1 + lk_mmvq (slices of eight rows) */
    RowsOnMatrixUnit = 3, /* lk_quantize_q8_1 + lk_dense_q4k_rows / lk_dense_q5k_rows / lk_dense_q6k_rows */
    Tiled = 4,         /* launch_mmq_quantize_q8_1_* + launch_mmq_gguf_* */
};

/* The most rows the mat-vec family takes for this weight before the call moves to a matrix-unit
 * kernel (matvec_rows of the reference, kernel_matmul.rs:27-33, with the crossovers measured on
 * MI355X: the K-quants 8 rows, except that matrices large enough to pay for it go to the 16-row tiles
 * of the matrix-unit rows kernels from 3 f32 rows on (Q4_K / Q5_K: n x rows of 57344, or 8192 at
 * k <= 2048; Q6_K: n x k of 48 Mi with k a multiple of 2048); then the matrix-unit rows kernels up to
 * 16 rows, or while n x rows x max(k, 4096) / 4096 <= 450 000 (twice that for a matrix of 1024 rows, and so
 * on: few rows yield few tiles; Q4_K / Q5_K rows of 8192 values or more leave them from 9 rows; below that even a tiled launch with K cut
 * into ranges does not beat them), then the tiled matmul; Q8_0 mat-vec slices up to 16 rows, then the
 * tiled matmul; the 32-value nibble formats, Q3_K and Q2_K mat-vec slices up to 15 rows, or 8 over a
 * matrix of 48 Mi weights or more, then the tiled matmul). */
int matvec_rows(int dtype, int k);

class QKernelMatMul {
public:
    /* `blob`: device address of `n` rows of `k` values in GGUF blocks of `dtype` (LK_TYPE_Q4_K /
     * Q6_K / Q8_0), owned by the caller, on device `device`. */
    QKernelMatMul(int dtype, int n, int k, const void* blob, int device);

    /* x [rows, k] (LK_TYPE_F32, F16 or BF16) -> out [rows, n] in x's type, on `stream`. The
     * matrix-unit kernels write f32 rows; for f16 / bf16 rows they write into a buffer of the device's
     * slot and one more launch rounds them into `out` (the reference narrows the f32 rows its
     * mmq_forward returns the same way, kernel_matmul.rs:1086-1714). `decode_order` keeps every row on the mat-vec
     * kernels whatever the count (DecodeOrder of the reference, kernel_matmul.rs:34-75).
     * Returns LK_OK or an LK_ERR_* code; never throws, never aborts. */
    int forward(const void* x, int x_type, int rows, void* out, void* stream, bool decode_order = false);

    /* An activation quantized to Q8_1 once, for every mat-vec over the same k on the same card
     * (QuantizedActivation of the reference, kernel_matmul.rs:105-117). The caller owns `q81`:
     * quantized_bytes(k, rows) bytes of device memory, 4-byte aligned. */
    struct QuantizedActivation {
        const void* q81 = nullptr;
        int k = 0, rows = 0, device = -1;
        int x_type = 0;   /* the type the rows were in, and so the type each product comes back in */
    };
    static size_t quantized_bytes(int k, int rows);

    /* quantize_for_matvec (kernel_matmul.rs:695-748): x [rows, k] into `q81` the way forward quantizes it
     * for the mat-vec kernels, so that several weights over the same rows quantize them once. LK_OK and `a`
     * filled, or LK_NOT_TAKEN where forward would not take those kernels for this row count (the
     * reference's None): more rows than matvec_rows without `decode_order`, or a matrix whose few rows go
     * to the matrix-unit rows kernels. */
    int quantize_for_matvec(const void* x, int x_type, int rows, void* q81, void* stream, QuantizedActivation* a,
                            bool decode_order = false) const;
    /* forward_quantized (kernel_matmul.rs:750-812): out [rows, n] in a.x_type, the bits forward gives on the
     * rows `a` was made from. LK_NOT_TAKEN where forward would take another path. */
    int forward_quantized(const QuantizedActivation& a, void* out, void* stream, bool decode_order = false);
    /* forward_quantized_pair (kernel_matmul.rs:814-876): this weight and `other` over ONE f32-born activation
     * row in one launch, each output with the bits of its own forward_quantized. LK_NOT_TAKEN where the pair
     * is not two weights of one format and one k on one card that the mat-vec family serves together. */
    int forward_quantized_pair(QKernelMatMul& other, const QuantizedActivation& a, void* out0, void* out1, void* stream);

    Path last_path() const { return last_path_; }
    int n() const { return n_; }
    int k() const { return k_; }

private:
    bool takes_matvec(int rows, bool decode_order) const;
    int dtype_, n_, k_, device_;
    const void* blob_;
    Path last_path_ = Path::None;
};

/* Frees every workspace this layer holds on every device (synchronizes those devices). */
void release_workspaces();

/* ------------------------------------------------------------------------------------------
 * GGUF container reader and weight upload (loken's src/tensor/quantized/gguf_file.rs; the upload
 * rule of kernel_matmul.rs:218-236 and cuda_storage.rs:27-39).
 * ---------------------------------------------------------------------------------------- */

/* Metadata value types, by the id the file stores (gguf_file.rs:45-60). */
enum class GgufType : int {
    U8 = 0, I8 = 1, U16 = 2, I16 = 3, U32 = 4, I32 = 5, F32 = 6, Bool = 7, String = 8, Array = 9,
    U64 = 10, I64 = 11, F64 = 12,
};

struct GgufValue {
    GgufType type = GgufType::U8;
    GgufType elem_type = GgufType::U8;   /* of an Array */
    uint64_t u = 0;                      /* unsigned kinds and Bool */
    int64_t i = 0;                       /* signed kinds */
    double f = 0;                        /* F32 (widened) and F64 */
    std::string s;
    std::vector<GgufValue> items;

    /* The reference's conversions (gguf_file.rs:314-357): any whole-number kind that fits; to_i64
     * refuses a U64 whatever its value; floats convert among themselves only. False = not that. */
    bool to_u64(uint64_t* out) const;
    bool to_i64(int64_t* out) const;
    bool to_f64(double* out) const;
};

struct GgufTensor {
    std::string name;
    std::vector<int64_t> dims;   /* row-major: the file's order reversed */
    int dtype = 0;               /* block type id, as LK_TYPE_* where those exist */
    uint64_t offset = 0;         /* from the aligned start of the payload */
    uint64_t bytes = 0;          /* elements / block values * block bytes */
    uint64_t elements() const;
};

/* What a model listing needs from a header without reading a tensor (gguf_file.rs:575-708).
 * -1 = the file does not say. */
struct GgufFacts {
    bool has_architecture = false;
    std::string architecture;
    int64_t file_type = -1;
    int64_t parameter_count = -1;   /* declared, else the sum over the tensor directory */
    bool pools = false;             /* `<architecture>.pooling_type` is present */
    int64_t split_parts = -1;
};

class GgufFile {
public:
    /* Maps `path` read-only and parses its header; nullptr and a message on any failure. */
    static GgufFile* open(const char* path, std::string* error);
    /* Parses an image the caller keeps alive (a mapping of its own, a test's bytes). */
    static GgufFile* over(const void* bytes, uint64_t len, std::string* error);
    ~GgufFile();

    int version() const { return version_; }
    uint64_t alignment() const { return alignment_; }
    uint64_t data_offset() const { return data_offset_; }   /* first multiple of alignment after the directory */

    int kv_count() const { return (int)keys_.size(); }       /* in file order */
    const std::string& key(int index) const { return keys_[index]; }
    const GgufValue& value(int index) const { return values_[index]; }
    int find_key(const char* key) const;                     /* -1: absent */

    int tensor_count() const { return (int)tensors_.size(); }
    const GgufTensor& tensor(int index) const { return tensors_[index]; }
    int find_tensor(const char* name) const;                 /* -1: absent */
    /* The tensor's blocks inside the image; nullptr when the directory points past its end. */
    const void* tensor_data(int index) const;

    GgufFacts facts() const;
    const GgufFacts& cached_facts() {
        if (!facts_ready_) { facts_ = facts(); facts_ready_ = true; }
        return facts_;
    }

    /* Device copy the kernels take: hipMalloc of bytes + 4096 on `device`, the tail zeroed, the
     * blocks copied on `stream`; returns after the copy has left the host. nullptr on failure.
     * The caller frees it (hipFree / lkh_gguf_free_blob). */
    void* upload(int index, int device, void* stream, uint64_t* blob_bytes) const;

private:
    GgufFile();
    bool parse(std::string* error);
    struct Image;
    Image* image_;
    int version_ = 0;
    uint64_t alignment_ = 32, data_offset_ = 0;
    std::vector<std::string> keys_;
    std::vector<GgufValue> values_;
    std::unordered_map<std::string, int> kv_index_, tensor_index_;
    std::vector<GgufTensor> tensors_;
    GgufFacts facts_;
    bool facts_ready_ = false;
};

}  // namespace loken

/* The same through plain C, for callers and tests that bind by symbol. */
extern "C" {
void* lkh_qkernel_matmul_new(int dtype, int n, int k, const void* blob, int device);
void lkh_qkernel_matmul_free(void* handle);
int lkh_qkernel_matmul_forward(void* handle, const void* x, int x_type, int rows, void* out, void* stream,
                               int decode_order);
int lkh_qkernel_matmul_last_path(void* handle);
/* QuantizedActivation through plain pointers: the caller keeps (q81, x_type, rows) and passes them back. */
size_t lkh_quantized_activation_bytes(int k, int rows);
int lkh_qkernel_matmul_quantize_for_matvec(void* handle, const void* x, int x_type, int rows, void* q81, void* stream,
                                           int decode_order);
int lkh_qkernel_matmul_forward_quantized(void* handle, const void* q81, int x_type, int rows, void* out, void* stream,
                                         int decode_order);
int lkh_qkernel_matmul_forward_quantized_pair(void* handle, void* other, const void* q81, void* out0, void* out1,
                                              void* stream);
int lkh_matvec_rows(int dtype, int k);
void lkh_release_workspaces(void);

/* GgufFile by handle. `err` (nullable, `err_len` bytes) receives the message when a call that
 * returns a handle returns NULL. Strings returned through `const char**` live as long as the
 * handle. Status returns are LK_OK or LK_ERR_ARG (no such handle / index) / LK_ERR_TYPE (the value
 * is not of the kind asked for). */
void* lkh_gguf_open(const char* path, char* err, int err_len);
void* lkh_gguf_over(const void* bytes, uint64_t len, char* err, int err_len);
void lkh_gguf_close(void* g);
int lkh_gguf_layout(void* g, int* version, uint64_t* alignment, uint64_t* data_offset, int* tensor_count,
                    int* kv_count);
int lkh_gguf_find_tensor(void* g, const char* name);
int lkh_gguf_tensor(void* g, int index, const char** name, int* dtype, int* n_dims, int64_t* dims, int max_dims,
                    uint64_t* offset, uint64_t* bytes);
void* lkh_gguf_tensor_data(void* g, int index);
int lkh_gguf_find_key(void* g, const char* key);
int lkh_gguf_kv(void* g, int index, const char** key, int* type, int* elem_type, uint64_t* count);
int lkh_gguf_kv_u64(void* g, int index, uint64_t* out);
int lkh_gguf_kv_i64(void* g, int index, int64_t* out);
int lkh_gguf_kv_f64(void* g, int index, double* out);
int lkh_gguf_kv_bool(void* g, int index, int* out);
int lkh_gguf_kv_str(void* g, int index, const char** out, uint64_t* len);
int lkh_gguf_kv_item_u64(void* g, int index, uint64_t i, uint64_t* out);
int lkh_gguf_kv_item_i64(void* g, int index, uint64_t i, int64_t* out);
int lkh_gguf_kv_item_f64(void* g, int index, uint64_t i, double* out);
int lkh_gguf_kv_item_str(void* g, int index, uint64_t i, const char** out, uint64_t* len);
int lkh_gguf_facts(void* g, const char** architecture, int64_t* file_type, int64_t* parameter_count, int* pools,
                   int64_t* split_parts);
void* lkh_gguf_upload(void* g, int index, int device, void* stream, uint64_t* blob_bytes);
void lkh_gguf_free_blob(void* blob);
/* Tensor `name` (2-D; Q4_K / Q5_K / Q6_K / Q8_0, or a 32-value nibble format, which runs as mat-vec launches at any row count) uploaded to `device` and wrapped as a QKernelMatMul
 * handle (QKernelMatMul::from_qtensor_on, kernel_matmul.rs:213-275); `*blob` receives the device
 * allocation, which the caller frees after the handle. */
void* lkh_gguf_linear(void* g, const char* name, int device, void* stream, void** blob, char* err, int err_len);
}

#endif

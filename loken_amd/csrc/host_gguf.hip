// GGUF container reader and weight upload: the on-disk format that feeds the quantized matmuls.
//
// Host-side mirror of loken's reader (src/tensor/quantized/gguf_file.rs): header v2 / v3
// (:868-901), metadata values (:223-284) with their conversions (:300-376), the tensor directory
// with dimensions stored innermost-first and restored to row-major (:135-204), the payload at the
// first multiple of `general.alignment` (default 32) after the directory (:139-144, :888-900),
// tensor byte size = elements / block values * block bytes (:391-393, table
// src/tensor/quantized/dtype.rs:66-96), the header facts walk (:608-708), and the upload rule of
// the card path: a zeroed device allocation of the tensor's bytes plus a 4096-byte tail the
// kernels may read into (src/tensor/quantized/mod.rs:35, kernel_matmul.rs:218-236,
// cuda_storage.rs:27-39). Files are memory-mapped read-only; tensor data is never copied on the
// host.

#include "../../include/loken_host.hpp"

#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <cstdio>
#include <exception>
#include <cstring>
#include <fcntl.h>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <unordered_map>
#include <vector>

namespace loken {

namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;   // "GGUF" little-endian
constexpr uint64_t DEFAULT_ALIGNMENT = 32;
constexpr uint64_t BLOB_TAIL_PAD_BYTES = 4096;

struct DtypeRow {
    int id, values, bytes;
    const char* name;
};
// id, values per block, bytes per block: the file's own table (dtype.rs:66-96)
const DtypeRow DTYPES[] = {
    {0, 1, 4, "f32"},       {1, 1, 2, "f16"},       {2, 32, 18, "q4_0"},     {3, 32, 20, "q4_1"},
    {6, 32, 22, "q5_0"},    {7, 32, 24, "q5_1"},    {8, 32, 34, "q8_0"},     {9, 32, 36, "q8_1"},
    {10, 256, 84, "q2_K"},  {11, 256, 110, "q3_K"}, {12, 256, 144, "q4_K"},  {13, 256, 176, "q5_K"},
    {14, 256, 210, "q6_K"}, {15, 256, 292, "q8_K"}, {16, 256, 66, "iq2_xxs"}, {20, 32, 18, "iq4_nl"},
    {18, 256, 98, "iq3_xxs"}, {21, 256, 110, "iq3_s"}, {22, 256, 82, "iq2_s"}, {23, 256, 136, "iq4_xs"},
    {42, 64, 18, "q2_0"},   {30, 1, 2, "bf16"},     {24, 1, 1, "i8"},        {39, 32, 17, "mxfp4"},
};

const DtypeRow* dtype_row(int id) {
    for (const DtypeRow& r : DTYPES)
        if (r.id == id) return &r;
    return nullptr;
}

struct Failure {
    std::string what;
};

// A bounded little-endian cursor over the file image.
struct Cursor {
    const uint8_t* base;
    uint64_t len, at = 0;

    void need(uint64_t n) const {
        if (n > len - at) throw Failure{"gguf read: failed to fill whole buffer"};
    }
    template <typename T>
    T scalar() {
        need(sizeof(T));
        T v;
        memcpy(&v, base + at, sizeof(T));
        at += sizeof(T);
        return v;
    }
    // a string is its byte length as a u64, then the bytes
    std::string string() {
        const uint64_t n = scalar<uint64_t>();
        need(n);
        std::string s((const char*)base + at, (size_t)n);
        at += n;
        return s;
    }
};

GgufValue read_value(Cursor& c, uint32_t type, int depth = 0) {
    GgufValue v;
    v.type = (GgufType)type;
    switch (type) {
        case 0: v.u = c.scalar<uint8_t>(); break;
        case 1: v.i = c.scalar<int8_t>(); break;
        case 2: v.u = c.scalar<uint16_t>(); break;
        case 3: v.i = c.scalar<int16_t>(); break;
        case 4: v.u = c.scalar<uint32_t>(); break;
        case 5: v.i = c.scalar<int32_t>(); break;
        case 6: v.f = c.scalar<float>(); break;
        case 7: v.u = c.scalar<uint8_t>() != 0; break;
        case 8: v.s = c.string(); break;
        case 9: {
            const uint32_t elem = c.scalar<uint32_t>();
            const uint64_t count = c.scalar<uint64_t>();
            if (depth > 8) throw Failure{"gguf: arrays nested too deep"};
            v.elem_type = (GgufType)elem;
            // an array cannot hold more items than the file has bytes left (every item is at least one)
            if (count > c.len - c.at) throw Failure{"gguf: array longer than the file"};
            v.items.reserve((size_t)(count < 4096 ? count : 4096));
            for (uint64_t i = 0; i < count; ++i) v.items.push_back(read_value(c, elem, depth + 1));
            break;
        }
        case 10: v.u = c.scalar<uint64_t>(); break;
        case 11: v.i = c.scalar<int64_t>(); break;
        case 12: v.f = c.scalar<double>(); break;
        default: throw Failure{"gguf: unknown value type " + std::to_string(type)};
    }
    return v;
}

}  // namespace

bool GgufValue::to_u64(uint64_t* out) const {
    switch (type) {
        case GgufType::U8: case GgufType::U16: case GgufType::U32: case GgufType::U64: *out = u; return true;
        case GgufType::I8: case GgufType::I16: case GgufType::I32: case GgufType::I64:
            if (i < 0) return false;
            *out = (uint64_t)i;
            return true;
        default: return false;
    }
}

bool GgufValue::to_i64(int64_t* out) const {
    switch (type) {
        case GgufType::U8: case GgufType::U16: case GgufType::U32: *out = (int64_t)u; return true;
        case GgufType::I8: case GgufType::I16: case GgufType::I32: case GgufType::I64: *out = i; return true;
        default: return false;   // a U64 is not an integer to this accessor, whatever its value
    }
}

bool GgufValue::to_f64(double* out) const {
    if (type != GgufType::F32 && type != GgufType::F64) return false;
    *out = f;
    return true;
}

uint64_t GgufTensor::elements() const {
    uint64_t n = 1;
    for (int64_t d : dims) n *= (uint64_t)d;
    return n;
}

struct GgufFile::Image {
    const uint8_t* bytes = nullptr;
    uint64_t len = 0;
    bool mapped = false;
    ~Image() {
        if (mapped && bytes) munmap((void*)bytes, len);
    }
};

GgufFile::GgufFile() : image_(new Image) {}
GgufFile::~GgufFile() { delete image_; }

bool GgufFile::parse(std::string* error) {
    try {
        Cursor c{image_->bytes, image_->len};
        const uint32_t magic = c.scalar<uint32_t>();
        const uint32_t version = c.scalar<uint32_t>();
        const uint64_t tensor_count = c.scalar<uint64_t>();
        const uint64_t kv_count = c.scalar<uint64_t>();
        if (magic != GGUF_MAGIC) {
            char buf[64];
            snprintf(buf, sizeof buf, "not a GGUF file (magic %#x)", magic);
            throw Failure{buf};
        }
        // version 1 sizes its counts and string lengths differently: named, not parsed
        if (version != 2 && version != 3) throw Failure{"unsupported GGUF version " + std::to_string(version)};
        version_ = (int)version;

        for (uint64_t i = 0; i < kv_count; ++i) {
            std::string key = c.string();
            const uint32_t type = c.scalar<uint32_t>();
            GgufValue v = read_value(c, type);
            kv_index_[key] = (int)keys_.size();   // a repeated key: the later value is the one found
            keys_.push_back(std::move(key));
            values_.push_back(std::move(v));
        }
        for (uint64_t i = 0; i < tensor_count; ++i) {
            GgufTensor t;
            t.name = c.string();
            const uint32_t n_dims = c.scalar<uint32_t>();
            if (n_dims > 8) throw Failure{"gguf: tensor `" + t.name + "` has " + std::to_string(n_dims) + " dimensions"};
            uint64_t elements = 1;
            for (uint32_t d = 0; d < n_dims; ++d) {
                const uint64_t dim = c.scalar<uint64_t>();
                if (dim == 0 || dim > (uint64_t)INT64_MAX || __builtin_mul_overflow(elements, dim, &elements) ||
                    elements > (uint64_t)INT64_MAX)
                    throw Failure{"gguf: tensor `" + t.name + "` has a dimension the format cannot mean"};
                t.dims.push_back((int64_t)dim);
            }
            // stored innermost-first; the rest of the stack states shapes row-major
            for (size_t a = 0, b = t.dims.size(); a + 1 < b; ++a, --b) std::swap(t.dims[a], t.dims[b - 1]);
            t.dtype = (int)c.scalar<uint32_t>();
            t.offset = c.scalar<uint64_t>();
            const DtypeRow* row = dtype_row(t.dtype);
            if (!row) throw Failure{"unsupported ggml dtype id " + std::to_string(t.dtype)};
            if (elements % (uint64_t)row->values != 0)
                throw Failure{"gguf: tensor `" + t.name + "` is not whole blocks of its type"};
            if (__builtin_mul_overflow(elements / (uint64_t)row->values, (uint64_t)row->bytes, &t.bytes))
                throw Failure{"gguf: tensor `" + t.name + "` is larger than an address"};
            tensor_index_[t.name] = (int)tensors_.size();
            tensors_.push_back(std::move(t));
        }
        alignment_ = DEFAULT_ALIGNMENT;
        auto it = kv_index_.find("general.alignment");
        uint64_t a;
        if (it != kv_index_.end() && values_[it->second].to_u64(&a)) alignment_ = a;
        if (alignment_ == 0) throw Failure{"gguf: general.alignment is zero"};
        if ((alignment_ & (alignment_ - 1)) != 0 || alignment_ > image_->len)
            throw Failure{"gguf: general.alignment " + std::to_string(alignment_) + " is not a power of two inside the file"};
        data_offset_ = (c.at + alignment_ - 1) / alignment_ * alignment_;
        return true;
    } catch (const Failure& f) {
        if (error) *error = f.what;
        return false;
    } catch (const std::exception& e) {   // a length the standard library refuses, or no memory: never out of an extern "C" call
        if (error) *error = std::string("gguf: ") + e.what();
        return false;
    }
}

GgufFile* GgufFile::open(const char* path, std::string* error) {
    const int fd = ::open(path, O_RDONLY);
    if (fd < 0) {
        if (error) *error = std::string("open ") + path + ": " + strerror(errno);
        return nullptr;
    }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        if (error) *error = std::string("gguf: cannot size ") + path;
        ::close(fd);
        return nullptr;
    }
    void* p = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_SHARED, fd, 0);
    ::close(fd);
    if (p == MAP_FAILED) {
        if (error) *error = std::string("gguf: cannot map ") + path;
        return nullptr;
    }
    GgufFile* g = new GgufFile;
    g->image_->bytes = (const uint8_t*)p;
    g->image_->len = (uint64_t)st.st_size;
    g->image_->mapped = true;
    if (!g->parse(error)) {
        delete g;
        return nullptr;
    }
    return g;
}

GgufFile* GgufFile::over(const void* bytes, uint64_t len, std::string* error) {
    GgufFile* g = new GgufFile;
    g->image_->bytes = (const uint8_t*)bytes;
    g->image_->len = len;
    if (!g->parse(error)) {
        delete g;
        return nullptr;
    }
    return g;
}

int GgufFile::find_tensor(const char* name) const {
    auto it = tensor_index_.find(name);
    return it == tensor_index_.end() ? -1 : it->second;
}

int GgufFile::find_key(const char* key) const {
    auto it = kv_index_.find(key);
    return it == kv_index_.end() ? -1 : it->second;
}

const void* GgufFile::tensor_data(int index) const {
    if (index < 0 || index >= (int)tensors_.size()) return nullptr;
    const GgufTensor& t = tensors_[index];
    const uint64_t at = data_offset_ + t.offset;
    if (at > image_->len || t.bytes > image_->len - at) return nullptr;   // a directory that points past the file
    return image_->bytes + at;
}

GgufFacts GgufFile::facts() const {
    // The walk of the reference, in file order: the listed keys precede the vocabulary, and with
    // the parameter count already read the walk stops at the first tokenizer key.
    GgufFacts f;
    for (size_t i = 0; i < keys_.size(); ++i) {
        const std::string& key = keys_[i];
        const GgufValue& v = values_[i];
        if (key.rfind("tokenizer.", 0) == 0 && f.parameter_count >= 0) return f;
        uint64_t u;
        if (key == "general.architecture") {
            f.has_architecture = v.type == GgufType::String;
            f.architecture = f.has_architecture ? v.s : std::string();
        } else if (key == "general.file_type") {
            f.file_type = v.to_u64(&u) ? (int64_t)u : -1;
        } else if (key == "general.parameter_count") {
            f.parameter_count = v.to_u64(&u) ? (int64_t)u : -1;
        } else if (key == "split.count") {
            f.split_parts = v.to_u64(&u) ? (int64_t)u : -1;
        } else if (f.has_architecture && key == f.architecture + ".pooling_type") {
            f.pools = true;
        }
    }
    // no declared count: the sum of what the directory lists; an empty directory leaves it absent
    if (f.parameter_count < 0) {
        uint64_t total = 0;
        for (const GgufTensor& t : tensors_) {
            uint64_t n = 1;
            for (int64_t d : t.dims) n = __builtin_mul_overflow(n, (uint64_t)d, &n) ? UINT64_MAX : n;
            total = __builtin_add_overflow(total, n, &total) ? UINT64_MAX : total;
        }
        if (total > 0) f.parameter_count = (int64_t)(total > (uint64_t)INT64_MAX ? INT64_MAX : total);
    }
    return f;
}

void* GgufFile::upload(int index, int device, void* stream, uint64_t* blob_bytes) const {
    const void* src = tensor_data(index);
    if (!src) return nullptr;
    const uint64_t n = tensors_[index].bytes;
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess || hipSetDevice(device) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    void* blob = nullptr;
    hipStream_t s = (hipStream_t)stream;
    bool ok = hipMalloc(&blob, n + BLOB_TAIL_PAD_BYTES) == hipSuccess;
    // the tail is what a kernel may read past the last row: zeros, whatever the allocator held
    ok = ok && hipMemsetAsync((uint8_t*)blob + n, 0, BLOB_TAIL_PAD_BYTES, s) == hipSuccess;
    ok = ok && (n == 0 || hipMemcpyAsync(blob, src, n, hipMemcpyHostToDevice, s) == hipSuccess);
    // the source is pageable (a file mapping): the copy has left the host when this returns
    ok = ok && hipStreamSynchronize(s) == hipSuccess;
    if (!ok) {
        (void)hipGetLastError();
        if (blob) (void)hipFree(blob);
        blob = nullptr;
    }
    (void)hipSetDevice(before);
    if (blob && blob_bytes) *blob_bytes = n + BLOB_TAIL_PAD_BYTES;
    return blob;
}

}  // namespace loken

// ------------------------------------------------------------------------------------------------
// The same through plain C.
// ------------------------------------------------------------------------------------------------
using loken::GgufFile;
using loken::GgufType;
using loken::GgufValue;

namespace {

void put_error(char* err, int err_len, const std::string& what) {
    if (err && err_len > 0) snprintf(err, (size_t)err_len, "%s", what.c_str());
}

const GgufValue* value_at(void* g, int index) {
    const GgufFile* f = (const GgufFile*)g;
    if (!f || index < 0 || index >= f->kv_count()) return nullptr;
    return &f->value(index);
}

const GgufValue* item_at(void* g, int index, uint64_t i) {
    const GgufValue* v = value_at(g, index);
    if (!v || v->type != GgufType::Array || i >= v->items.size()) return nullptr;
    return &v->items[(size_t)i];
}

}  // namespace

extern "C" void* lkh_gguf_open(const char* path, char* err, int err_len) {
    std::string what;
    GgufFile* g = path ? GgufFile::open(path, &what) : nullptr;
    if (!g) put_error(err, err_len, path ? what : "gguf: no path");
    return g;
}

extern "C" void* lkh_gguf_over(const void* bytes, uint64_t len, char* err, int err_len) {
    std::string what;
    GgufFile* g = bytes ? GgufFile::over(bytes, len, &what) : nullptr;
    if (!g) put_error(err, err_len, bytes ? what : "gguf: no bytes");
    return g;
}

extern "C" void lkh_gguf_close(void* g) { delete (GgufFile*)g; }

extern "C" int lkh_gguf_layout(void* g, int* version, uint64_t* alignment, uint64_t* data_offset, int* tensor_count,
                               int* kv_count) {
    const GgufFile* f = (const GgufFile*)g;
    if (!f) return LK_ERR_ARG;
    if (version) *version = f->version();
    if (alignment) *alignment = f->alignment();
    if (data_offset) *data_offset = f->data_offset();
    if (tensor_count) *tensor_count = f->tensor_count();
    if (kv_count) *kv_count = f->kv_count();
    return LK_OK;
}

extern "C" int lkh_gguf_find_tensor(void* g, const char* name) {
    return g && name ? ((const GgufFile*)g)->find_tensor(name) : -1;
}

extern "C" int lkh_gguf_tensor(void* g, int index, const char** name, int* dtype, int* n_dims, int64_t* dims,
                               int max_dims, uint64_t* offset, uint64_t* bytes) {
    const GgufFile* f = (const GgufFile*)g;
    if (!f || index < 0 || index >= f->tensor_count()) return LK_ERR_ARG;
    const loken::GgufTensor& t = f->tensor(index);
    if (name) *name = t.name.c_str();
    if (dtype) *dtype = t.dtype;
    if (n_dims) *n_dims = (int)t.dims.size();
    if (dims)
        for (int i = 0; i < max_dims && i < (int)t.dims.size(); ++i) dims[i] = t.dims[i];
    if (offset) *offset = t.offset;
    if (bytes) *bytes = t.bytes;
    return LK_OK;
}

extern "C" void* lkh_gguf_tensor_data(void* g, int index) {
    return g ? (void*)((const GgufFile*)g)->tensor_data(index) : nullptr;
}

extern "C" int lkh_gguf_find_key(void* g, const char* key) {
    return g && key ? ((const GgufFile*)g)->find_key(key) : -1;
}

extern "C" int lkh_gguf_kv(void* g, int index, const char** key, int* type, int* elem_type, uint64_t* count) {
    const GgufValue* v = value_at(g, index);
    if (!v) return LK_ERR_ARG;
    if (key) *key = ((const GgufFile*)g)->key(index).c_str();
    if (type) *type = (int)v->type;
    if (elem_type) *elem_type = v->type == GgufType::Array ? (int)v->elem_type : -1;
    if (count) *count = v->type == GgufType::Array ? v->items.size() : 1;
    return LK_OK;
}

extern "C" int lkh_gguf_kv_u64(void* g, int index, uint64_t* out) {
    const GgufValue* v = value_at(g, index);
    return v && out && v->to_u64(out) ? LK_OK : LK_ERR_TYPE;
}
extern "C" int lkh_gguf_kv_i64(void* g, int index, int64_t* out) {
    const GgufValue* v = value_at(g, index);
    return v && out && v->to_i64(out) ? LK_OK : LK_ERR_TYPE;
}
extern "C" int lkh_gguf_kv_f64(void* g, int index, double* out) {
    const GgufValue* v = value_at(g, index);
    return v && out && v->to_f64(out) ? LK_OK : LK_ERR_TYPE;
}
extern "C" int lkh_gguf_kv_bool(void* g, int index, int* out) {
    const GgufValue* v = value_at(g, index);
    if (!v || !out || v->type != GgufType::Bool) return LK_ERR_TYPE;
    *out = v->u != 0;
    return LK_OK;
}
extern "C" int lkh_gguf_kv_str(void* g, int index, const char** out, uint64_t* len) {
    const GgufValue* v = value_at(g, index);
    if (!v || !out || v->type != GgufType::String) return LK_ERR_TYPE;
    *out = v->s.c_str();
    if (len) *len = v->s.size();
    return LK_OK;
}
extern "C" int lkh_gguf_kv_item_u64(void* g, int index, uint64_t i, uint64_t* out) {
    const GgufValue* v = item_at(g, index, i);
    return v && out && v->to_u64(out) ? LK_OK : LK_ERR_TYPE;
}
extern "C" int lkh_gguf_kv_item_i64(void* g, int index, uint64_t i, int64_t* out) {
    const GgufValue* v = item_at(g, index, i);
    return v && out && v->to_i64(out) ? LK_OK : LK_ERR_TYPE;
}
extern "C" int lkh_gguf_kv_item_f64(void* g, int index, uint64_t i, double* out) {
    const GgufValue* v = item_at(g, index, i);
    return v && out && v->to_f64(out) ? LK_OK : LK_ERR_TYPE;
}
extern "C" int lkh_gguf_kv_item_str(void* g, int index, uint64_t i, const char** out, uint64_t* len) {
    const GgufValue* v = item_at(g, index, i);
    if (!v || !out || v->type != GgufType::String) return LK_ERR_TYPE;
    *out = v->s.c_str();
    if (len) *len = v->s.size();
    return LK_OK;
}

extern "C" int lkh_gguf_facts(void* g, const char** architecture, int64_t* file_type, int64_t* parameter_count,
                              int* pools, int64_t* split_parts) {
    GgufFile* f = (GgufFile*)g;
    if (!f) return LK_ERR_ARG;
    const loken::GgufFacts& facts = f->cached_facts();
    if (architecture) *architecture = facts.has_architecture ? facts.architecture.c_str() : nullptr;
    if (file_type) *file_type = facts.file_type;
    if (parameter_count) *parameter_count = facts.parameter_count;
    if (pools) *pools = facts.pools;
    if (split_parts) *split_parts = facts.split_parts;
    return LK_OK;
}

extern "C" void* lkh_gguf_upload(void* g, int index, int device, void* stream, uint64_t* blob_bytes) {
    return g ? ((const GgufFile*)g)->upload(index, device, stream, blob_bytes) : nullptr;
}

extern "C" void lkh_gguf_free_blob(void* blob) {
    if (blob) (void)hipFree(blob);
}

extern "C" void* lkh_gguf_linear(void* g, const char* name, int device, void* stream, void** blob, char* err,
                                 int err_len) {
    const GgufFile* f = (const GgufFile*)g;
    if (!f || !name || !blob) {
        put_error(err, err_len, "gguf: no file, name or blob slot");
        return nullptr;
    }
    const int index = f->find_tensor(name);
    if (index < 0) {
        put_error(err, err_len, std::string("gguf: no tensor `") + name + "`");
        return nullptr;
    }
    const loken::GgufTensor& t = f->tensor(index);
    if (t.dims.size() != 2) {
        put_error(err, err_len, "QKernelMatMul: weight must be 2-D, got " + std::to_string(t.dims.size()) + " dims");
        return nullptr;
    }
    const bool nibble32 = t.dtype == LK_TYPE_Q4_0 || t.dtype == LK_TYPE_Q4_1 || t.dtype == LK_TYPE_Q5_0 ||
                          t.dtype == LK_TYPE_Q5_1 || t.dtype == LK_TYPE_IQ4_NL || t.dtype == LK_TYPE_MXFP4 ||
                          t.dtype == LK_TYPE_Q2_K || t.dtype == LK_TYPE_Q3_K || t.dtype == LK_TYPE_IQ4_XS;   // (the mat-vec-only formats)
    if (!nibble32 && t.dtype != LK_TYPE_Q4_K && t.dtype != LK_TYPE_Q5_K && t.dtype != LK_TYPE_Q6_K && t.dtype != LK_TYPE_Q8_0) {
        put_error(err, err_len, "QKernelMatMul: block type " + std::to_string(t.dtype) + " is not served on the card");
        return nullptr;
    }
    if (t.dims[0] <= 0 || t.dims[1] <= 0 || t.dims[0] > INT32_MAX || t.dims[1] > INT32_MAX) {
        put_error(err, err_len, "QKernelMatMul: dimension beyond 2^31");
        return nullptr;
    }
    *blob = f->upload(index, device, stream, nullptr);
    if (!*blob) {
        put_error(err, err_len, std::string("QKernelMatMul upload: `") + name + "` did not reach device " + std::to_string(device));
        return nullptr;
    }
    return lkh_qkernel_matmul_new(t.dtype, (int)t.dims[0], (int)t.dims[1], *blob, device);
}

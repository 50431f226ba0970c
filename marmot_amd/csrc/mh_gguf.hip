// GGUF file reader for the weights of the path: maps a file read-only, parses the header, the key/value table (kept as
// views into the mapping for marmot_hip_gguf_find_kv; only general.alignment is interpreted here) and the tensor table,
// and exposes every tensor as a view into the mapping with the
// shape convention and the ggml-type -> quant-kind mapping of the reference's loader (src/graph/gguf/loader.cpp:
// map_ggml_type :300-490, set_tensor_data_views :492-575, load_file :577-770). Host code only. Tensor views are host
// pointers: the tensor-level backend mirrors them on first use; marmot_hip_gguf_upload copies one tensor to the device
// for callers of the raw-pointer ABI.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "mh_common.h"

struct marmot_hip_gguf {
    int fd = -1;
    uint8_t *data = nullptr;
    size_t size = 0;
    size_t alignment = 32;
    uint32_t version = 0;
    struct Entry {
        std::string name;
        uint32_t ggml_type = 0;
        int kind = 0;
        int dtype = 0;
        uint32_t ndim = 0;
        uint64_t shape[MARMOT_HIP_GGUF_MAX_DIMS] = {0};
        uint64_t offset = 0;
        size_t nbytes = 0;
    };
    std::vector<Entry> tensors;
    struct Kv {
        std::string key;
        uint32_t type = 0, elem_type = 0;
        uint64_t count = 1;
        size_t offset = 0, nbytes = 0;  // payload inside the mapping
    };
    std::vector<Kv> kv;
};

namespace {

using namespace mh;

struct Cursor {
    const uint8_t *p;
    size_t size, off = 0;
    template <class T>
    bool read(T &v) {
        if (off + sizeof(T) > size) {
            return false;
        }
        std::memcpy(&v, p + off, sizeof(T));
        off += sizeof(T);
        return true;
    }
    bool skip(uint64_t n) {
        if (n > size - off) {
            return false;
        }
        off += (size_t)n;
        return true;
    }
    bool read_string(std::string *out) {
        uint64_t len = 0;
        if (!read(len) || len > size - off) {
            return false;
        }
        if (out != nullptr) {
            out->assign((const char *)p + off, (size_t)len);
        }
        off += (size_t)len;
        return true;
    }
};

// GGUF value types: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string, 9 array, 10 u64, 11 i64, 12 f64
size_t scalar_size(uint32_t type) {
    switch (type) {
    case 0:
    case 1:
    case 7:
        return 1;
    case 2:
    case 3:
        return 2;
    case 4:
    case 5:
    case 6:
        return 4;
    case 10:
    case 11:
    case 12:
        return 8;
    default:
        return 0;
    }
}

// Steps over one value and records where its payload lies: a scalar's bytes, a string's characters, an array's
// elements (for an array of strings the first length-prefixed string; nbytes covers all of them).
bool skip_value(Cursor &c, uint32_t type, uint32_t *u32_out, marmot_hip_gguf::Kv *kv) {
    kv->type = type;
    kv->elem_type = 0;
    kv->count = 1;
    if (type == 8) {
        uint64_t len = 0;
        if (!c.read(len) || len > c.size - c.off) {
            return false;
        }
        kv->offset = c.off;
        kv->nbytes = (size_t)len;
        return c.skip(len);
    }
    if (type == 9) {
        uint32_t elem = 0;
        uint64_t count = 0;
        if (!c.read(elem) || !c.read(count)) {
            return false;
        }
        if (elem == 9) {
            return false;  // nested arrays do not occur in GGUF files
        }
        kv->elem_type = elem;
        kv->count = count;
        kv->offset = c.off;
        if (elem == 8) {
            for (uint64_t i = 0; i < count; ++i) {
                if (!c.read_string(nullptr)) {
                    return false;
                }
            }
            kv->nbytes = c.off - kv->offset;
            return true;
        }
        const size_t es = scalar_size(elem);
        if (es == 0 || count > (c.size - c.off) / es) {
            return false;
        }
        kv->nbytes = (size_t)count * es;
        return c.skip(count * es);
    }
    const size_t s = scalar_size(type);
    if (s == 0) {
        return false;
    }
    kv->offset = c.off;
    kv->nbytes = s;
    if (type == 4 && u32_out != nullptr) {
        return c.read(*u32_out);
    }
    return c.skip(s);
}

// ggml tensor type -> (quant kind, dense dtype); loader.cpp:300-490. Dense types this library moves: F32, F16, I32.
bool map_ggml_type(uint32_t t, int *kind, int *dtype) {
    *kind = 0;
    *dtype = MARMOT_HIP_DTYPE_U8;
    switch (t) {
    case 0:
        *dtype = MARMOT_HIP_DTYPE_F32;
        return true;
    case 1:
        *dtype = MARMOT_HIP_DTYPE_F16;
        return true;
    case 26:
        *dtype = MARMOT_HIP_DTYPE_I32;
        return true;
    case 2:
        *kind = MARMOT_HIP_KIND_Q4_0;
        return true;
    case 3:
        *kind = MARMOT_HIP_KIND_Q4_1;
        return true;
    case 6:
        *kind = MARMOT_HIP_KIND_Q5_0;
        return true;
    case 7:
        *kind = MARMOT_HIP_KIND_Q5_1;
        return true;
    case 8:
        *kind = MARMOT_HIP_KIND_Q8_0;
        return true;
    case 9:
        *kind = MARMOT_HIP_KIND_Q8_1;
        return true;
    case 10:
        *kind = MARMOT_HIP_KIND_Q2_K;
        return true;
    case 11:
        *kind = MARMOT_HIP_KIND_Q3_K;
        return true;
    case 12:
        *kind = MARMOT_HIP_KIND_Q4_K;
        return true;
    case 13:
        *kind = MARMOT_HIP_KIND_Q5_K;
        return true;
    case 14:
        *kind = MARMOT_HIP_KIND_Q6_K;
        return true;
    case 15:
        *kind = MARMOT_HIP_KIND_Q8_K;
        return true;
    default:
        return false;
    }
}

// bytes of a tensor: rows of the innermost (GGUF dimension 0) length, in blocks for quantized kinds. The dimensions
// come from the file: 0 when a product does not fit 64 bits (the caller rejects the file).
size_t tensor_bytes(const marmot_hip_gguf::Entry &e, const uint64_t *raw) {
    uint64_t rows = 1;
    for (uint32_t d = 1; d < e.ndim; ++d) {
        if (__builtin_mul_overflow(rows, raw[d], &rows)) {
            return 0;
        }
    }
    uint64_t row_bytes;
    if (e.kind != 0) {
        const uint64_t bv = marmot_hip_block_values(e.kind), bb = marmot_hip_block_bytes(e.kind);
        uint64_t padded;
        if (bv == 0 || __builtin_add_overflow(raw[0], bv - 1, &padded) ||
            __builtin_mul_overflow(padded / bv, bb, &row_bytes)) {
            return 0;
        }
    } else {
        const uint64_t es = e.dtype == MARMOT_HIP_DTYPE_F32 || e.dtype == MARMOT_HIP_DTYPE_I32 ? 4 : 2;
        if (__builtin_mul_overflow(raw[0], es, &row_bytes)) {
            return 0;
        }
    }
    uint64_t total;
    if (__builtin_mul_overflow(rows, row_bytes, &total) || total > (uint64_t)SIZE_MAX) {
        return 0;
    }
    return (size_t)total;
}

void fill_view(const marmot_hip_gguf *g, const marmot_hip_gguf::Entry &e, marmot_hip_gguf_tensor_t *out) {
    out->name = e.name.c_str();
    out->ggml_type = e.ggml_type;
    out->kind = e.kind;
    out->dtype = e.dtype;
    out->ndim = e.ndim;
    for (int d = 0; d < MARMOT_HIP_GGUF_MAX_DIMS; ++d) {
        out->shape[d] = e.shape[d];
    }
    out->data = g->data + e.offset;
    out->nbytes = e.nbytes;
}

}  // namespace

extern "C" {

int marmot_hip_gguf_open(const char *path, marmot_hip_gguf_t **out) {
    if (path == nullptr || out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF path is null");
    }
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Unable to open GGUF file");
    }
    struct stat st {};
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        close(fd);
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Unable to stat GGUF file");
    }
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (map == MAP_FAILED) {
        close(fd);
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Unable to mmap GGUF file");
    }
    marmot_hip_gguf *g = new marmot_hip_gguf();
    g->fd = fd;
    g->data = (uint8_t *)map;
    g->size = (size_t)st.st_size;
    auto fail = [&](int code, const char *msg) {
        marmot_hip_gguf_close(g);
        return set_error(code, "%s", msg);
    };
    Cursor c{g->data, g->size};
    uint32_t magic = 0;
    uint64_t n_tensors = 0, n_kv = 0;
    if (!c.read(magic) || magic != 0x46554747u /* "GGUF" */ || !c.read(g->version) || !c.read(n_tensors) ||
        !c.read(n_kv)) {
        return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Not a GGUF file");
    }
    if (g->version < 2 || g->version > 3) {
        return fail(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "Unsupported GGUF version");
    }
    if (n_tensors > g->size / 24 || n_kv > g->size / 12) {
        return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF table sizes exceed the file");
    }
    g->kv.reserve((size_t)n_kv);
    for (uint64_t i = 0; i < n_kv; ++i) {
        std::string key;
        uint32_t type = 0, u32 = 0;
        if (!c.read_string(&key) || key.empty() || !c.read(type)) {
            return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Invalid GGUF key");
        }
        marmot_hip_gguf::Kv entry;
        if (!skip_value(c, type, &u32, &entry)) {
            return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Unable to parse GGUF value");
        }
        entry.key = key;
        g->kv.push_back(std::move(entry));
        if (key == "general.alignment" && type == 4 && u32 != 0) {
            g->alignment = u32;
        }
    }
    std::vector<std::vector<uint64_t>> raw(n_tensors);
    g->tensors.resize((size_t)n_tensors);
    for (size_t i = 0; i < g->tensors.size(); ++i) {
        marmot_hip_gguf::Entry &e = g->tensors[i];
        if (!c.read_string(&e.name) || e.name.empty() || !c.read(e.ndim) || e.ndim == 0 ||
            e.ndim > MARMOT_HIP_GGUF_MAX_DIMS) {
            return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Invalid GGUF tensor name or rank");
        }
        raw[i].resize(e.ndim);
        for (uint32_t d = 0; d < e.ndim; ++d) {
            if (!c.read(raw[i][d]) || raw[i][d] == 0) {
                return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Invalid GGUF tensor dimension");
            }
        }
        if (!c.read(e.ggml_type) || !c.read(e.offset)) {
            return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Invalid GGUF tensor type or offset");
        }
        if (!map_ggml_type(e.ggml_type, &e.kind, &e.dtype)) {
            return fail(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "Unsupported GGUF tensor type");
        }
        // matrices become [rows, cols] = [ne1, ne0]; other ranks keep the file's order (loader.cpp:737-745)
        if (e.ndim == 2) {
            e.shape[0] = raw[i][1];
            e.shape[1] = raw[i][0];
        } else {
            for (uint32_t d = 0; d < e.ndim; ++d) {
                e.shape[d] = raw[i][d];
            }
        }
    }
    const size_t data_offset = (c.off + g->alignment - 1) / g->alignment * g->alignment;
    if (data_offset > g->size) {
        return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF tensor data offset out of range");
    }
    const size_t data_size = g->size - data_offset;
    // a tensor's span ends where the next one (by offset) starts (loader.cpp:511-528)
    std::vector<size_t> order(g->tensors.size());
    for (size_t i = 0; i < order.size(); ++i) {
        order[i] = i;
    }
    std::sort(order.begin(), order.end(),
              [&](size_t a, size_t b) { return g->tensors[a].offset < g->tensors[b].offset; });
    for (size_t k = 0; k < order.size(); ++k) {
        marmot_hip_gguf::Entry &e = g->tensors[order[k]];
        const uint64_t next = k + 1 < order.size() ? g->tensors[order[k + 1]].offset : (uint64_t)data_size;
        if (e.offset > data_size || next > data_size || next < e.offset) {
            return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF tensor span exceeds file bounds");
        }
        e.nbytes = tensor_bytes(e, raw[order[k]].data());
        if (e.nbytes == 0 || e.nbytes > next - e.offset) {
            return fail(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF tensor storage does not match expected size");
        }
        e.offset += data_offset;  // from here on: offset into the mapping
    }
    *out = g;
    return MARMOT_HIP_SUCCESS;
}

void marmot_hip_gguf_close(marmot_hip_gguf_t *g) {
    if (g == nullptr) {
        return;
    }
    if (g->data != nullptr) {
        munmap(g->data, g->size);
    }
    if (g->fd >= 0) {
        close(g->fd);
    }
    delete g;
}

size_t marmot_hip_gguf_tensor_count(const marmot_hip_gguf_t *g) {
    return g != nullptr ? g->tensors.size() : 0;
}

size_t marmot_hip_gguf_alignment(const marmot_hip_gguf_t *g) {
    return g != nullptr ? g->alignment : 0;
}

int marmot_hip_gguf_tensor(const marmot_hip_gguf_t *g, size_t index, marmot_hip_gguf_tensor_t *out) {
    if (g == nullptr || out == nullptr || index >= g->tensors.size()) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF tensor index out of range");
    }
    fill_view(g, g->tensors[index], out);
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_gguf_find(const marmot_hip_gguf_t *g, const char *name, marmot_hip_gguf_tensor_t *out) {
    if (g == nullptr || name == nullptr || out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF lookup: null argument");
    }
    for (const auto &e : g->tensors) {
        if (e.name == name) {
            fill_view(g, e, out);
            return MARMOT_HIP_SUCCESS;
        }
    }
    return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF tensor '%s' not found", name);
}

// ---- key/value metadata (marmot_gguf_find_kv, include/marmot/graph/gguf_loader.h:165; values of
// marmot_gguf_value_t :108-132 as views into the mapping)
static void fill_kv(const marmot_hip_gguf_t *g, const marmot_hip_gguf::Kv &e, marmot_hip_gguf_kv_t *out) {
    out->key = e.key.c_str();
    out->type = e.type;
    out->elem_type = e.elem_type;
    out->count = e.count;
    out->data = g->data + e.offset;
    out->nbytes = e.nbytes;
}

size_t marmot_hip_gguf_kv_count(const marmot_hip_gguf_t *g) {
    return g != nullptr ? g->kv.size() : 0;
}

int marmot_hip_gguf_kv(const marmot_hip_gguf_t *g, size_t index, marmot_hip_gguf_kv_t *out) {
    if (g == nullptr || out == nullptr || index >= g->kv.size()) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF key/value index out of range");
    }
    fill_kv(g, g->kv[index], out);
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_gguf_find_kv(const marmot_hip_gguf_t *g, const char *key, marmot_hip_gguf_kv_t *out) {
    if (g == nullptr || key == nullptr || out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF lookup: null argument");
    }
    for (const auto &e : g->kv) {
        if (e.key == key) {
            fill_kv(g, e, out);
            return MARMOT_HIP_SUCCESS;
        }
    }
    return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF key '%s' not found", key);
}

// one element of a scalar value (index 0) or of an array of scalars, widened
static bool kv_scalar_at(const marmot_hip_gguf_kv_t *kv, uint64_t index, uint64_t *u, int64_t *i, double *f,
                         int *cls /* 0 unsigned, 1 signed, 2 float */) {
    const uint32_t t = kv->type == 9 ? kv->elem_type : kv->type;
    const size_t es = scalar_size(t);
    if (es == 0 || index >= kv->count || (index + 1) * es > kv->nbytes) {
        return false;
    }
    const uint8_t *p = (const uint8_t *)kv->data + index * es;
    switch (t) {
    case 0: case 7: { uint8_t v; std::memcpy(&v, p, 1); *u = v; *cls = 0; return true; }
    case 1: { int8_t v; std::memcpy(&v, p, 1); *i = v; *cls = 1; return true; }
    case 2: { uint16_t v; std::memcpy(&v, p, 2); *u = v; *cls = 0; return true; }
    case 3: { int16_t v; std::memcpy(&v, p, 2); *i = v; *cls = 1; return true; }
    case 4: { uint32_t v; std::memcpy(&v, p, 4); *u = v; *cls = 0; return true; }
    case 5: { int32_t v; std::memcpy(&v, p, 4); *i = v; *cls = 1; return true; }
    case 6: { float v; std::memcpy(&v, p, 4); *f = v; *cls = 2; return true; }
    case 10: { uint64_t v; std::memcpy(&v, p, 8); *u = v; *cls = 0; return true; }
    case 11: { int64_t v; std::memcpy(&v, p, 8); *i = v; *cls = 1; return true; }
    case 12: { double v; std::memcpy(&v, p, 8); *f = v; *cls = 2; return true; }
    default: return false;
    }
}

int marmot_hip_gguf_kv_int(const marmot_hip_gguf_kv_t *kv, uint64_t index, int64_t *out) {
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0;
    int cls = 0;
    if (kv == nullptr || out == nullptr || !kv_scalar_at(kv, index, &u, &i, &f, &cls) || cls == 2 ||
        (cls == 0 && u > (uint64_t)INT64_MAX)) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF value is not an integer that fits int64");
    }
    *out = cls == 0 ? (int64_t)u : i;
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_gguf_kv_float(const marmot_hip_gguf_kv_t *kv, uint64_t index, double *out) {
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0;
    int cls = 0;
    if (kv == nullptr || out == nullptr || !kv_scalar_at(kv, index, &u, &i, &f, &cls)) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF value is not a number");
    }
    *out = cls == 2 ? f : (cls == 0 ? (double)u : (double)i);
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_gguf_kv_string(const marmot_hip_gguf_kv_t *kv, uint64_t index, const char **chars, size_t *length) {
    if (kv == nullptr || chars == nullptr || length == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF string: null argument");
    }
    if (kv->type == 8 && index == 0) {
        *chars = (const char *)kv->data;
        *length = kv->nbytes;
        return MARMOT_HIP_SUCCESS;
    }
    if (kv->type != 9 || kv->elem_type != 8 || index >= kv->count) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF value is not a string (or the index is out of range)");
    }
    Cursor c{(const uint8_t *)kv->data, kv->nbytes};  // lengths were validated when the file was opened
    for (uint64_t i = 0; i < index; ++i) {
        if (!c.read_string(nullptr)) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF string array is malformed");
        }
    }
    uint64_t len = 0;
    if (!c.read(len) || len > c.size - c.off) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF string array is malformed");
    }
    *chars = (const char *)c.p + c.off;
    *length = (size_t)len;
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_gguf_upload(marmot_hip_device_t *dev, const marmot_hip_gguf_t *g, size_t index, void **d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (g == nullptr || d_out == nullptr || index >= g->tensors.size()) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "GGUF upload: bad argument");
    }
    const auto &e = g->tensors[index];
    void *d = nullptr;
    int st = marmot_hip_alloc(dev, e.nbytes, &d);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    st = marmot_hip_memcpy_to_device(dev, d, g->data + e.offset, e.nbytes);
    if (st != MARMOT_HIP_SUCCESS) {
        marmot_hip_free(dev, d);
        return st;
    }
    *d_out = d;
    return MARMOT_HIP_SUCCESS;
}

}  // extern "C"

// marmot_tensor_t-level HIP backend, written in C23 like the host side of marmot's other backends: device vtable
// with a host-pointer residency table, kernel query, bytecode exec table and the impl functions the generated
// dispatch shims call. Host code only; all device work goes through the raw-pointer C ABI of marmot_hip.h.
#include "marmot_hip.h"
#include "marmot_hip_backend.h"

#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

// ------------------------------------------------------------------ errors
#ifdef MARMOT_HIP_IN_TREE
static marmot_error_t fail(marmot_error_t code, const char *msg) {
    marmot_set_error(code, msg);
    return code;
}
#else
static thread_local marmot_error_t g_last_code = MARMOT_SUCCESS;
static thread_local char g_last_detail[256] = {0};
static marmot_error_t fail(marmot_error_t code, const char *msg) {
    g_last_code = code;
    snprintf(g_last_detail, sizeof(g_last_detail), "%s", msg != nullptr ? msg : "");
    return code;
}
#endif

// a failure of the raw ABI: same numeric codes, text from the library
static marmot_error_t fail_from_lib(int code) {
    return fail((marmot_error_t)code, marmot_hip_last_error());
}

// ------------------------------------------------------------------ residency table
// One device mirror per host address range, kept sorted by the range's first byte. Ranges never overlap: a request
// that is contained in a mirror resolves to an offset inside it; a request that overlaps mirrors without being
// contained in one replaces them with one mirror over the union (their device-newer bytes are brought home first).
typedef struct {
    uintptr_t host;
    size_t bytes;
    void *dev;
    bool host_newer;  // host copy changed since the last upload
    bool dev_newer;   // a kernel wrote the mirror since the last download
} hip_mirror_t;

// Rotary frequencies of one parameter set (the counterpart of marmot_rope_freq_cache_t, src/core/helpers/rope.h):
// computed on the host with the reference's formula, mirrored to the device through the residency table.
typedef struct {
    bool used;
    int scaling_type;
    float theta, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
    uint32_t orig_ctx_len, head_dim_in;
    size_t M;
    uint32_t head_dim;  // resolved
    float attn_scale;
    float *freqs;       // head_dim / 2 values, owned
} hip_rope_entry_t;
#define HIP_ROPE_CACHE 8

// Packed (quantized) copies of fp32 activation tensors, keyed by the tensor's host address: the normalization that
// produces a tensor leaves its rows here already packed, and the first linear that reads an fp32 tensor of nine rows
// or more packs it here for the linears that share the input (gate / up). An entry dies when anything writes the
// tensor, when the host copy changes or when the host memory is released.
typedef struct {
    bool valid;
    uintptr_t host;
    size_t rows, cols;
    int act_kind;       // MARMOT_HIP_KIND_Q8_K or MARMOT_HIP_KIND_Q8_0
    void *packed;       // device buffer, owned
    size_t capacity;
    uint64_t stamp;     // last use: the oldest entry is replaced
} hip_pack_entry_t;
#define HIP_PACK_CACHE 4
#define HIP_PACK_MIN_ROWS 9  // below, the linears quantize fp32 rows inside their own kernels

typedef struct {
    marmot_hip_device_t *dev;
    pthread_mutex_t mu;
    hip_pack_entry_t packs[HIP_PACK_CACHE];
    uint64_t pack_clock, packs_made, pack_hits;
    hip_mirror_t *mirrors;  // sorted by host
    size_t n_mirrors, cap_mirrors;
    hip_rope_entry_t rope[HIP_ROPE_CACHE];
    size_t rope_next;
    bool batching;
    uint64_t uploads, upload_bytes, downloads, download_bytes;
    size_t mirrored_bytes;
} hip_backend_t;

static hip_backend_t *backend_of(const void *device_ctx) {
    return (hip_backend_t *)device_ctx;
}

// index of the first mirror whose start is > p
static size_t upper_bound(const hip_backend_t *b, uintptr_t p) {
    size_t lo = 0, hi = b->n_mirrors;
    while (lo < hi) {
        const size_t mid = lo + (hi - lo) / 2;
        if (b->mirrors[mid].host <= p) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    return lo;
}

static hip_mirror_t *find_containing(hip_backend_t *b, uintptr_t p, size_t n) {
    const size_t i = upper_bound(b, p);
    if (i == 0) {
        return nullptr;
    }
    hip_mirror_t *m = &b->mirrors[i - 1];
    return (p >= m->host && p + n <= m->host + m->bytes) ? m : nullptr;
}

static bool overlaps(const hip_mirror_t *m, uintptr_t p, size_t n) {
    return m->host < p + n && p < m->host + m->bytes;
}

static marmot_error_t upload(hip_backend_t *b, hip_mirror_t *m) {
    const int st = marmot_hip_memcpy_to_device(b->dev, m->dev, (const void *)m->host, m->bytes);
    if (st != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(st);
    }
    b->uploads++;
    b->upload_bytes += m->bytes;
    m->host_newer = false;
    return MARMOT_SUCCESS;
}

static marmot_error_t download(hip_backend_t *b, const hip_mirror_t *m, uintptr_t p, size_t n) {
    const int st = marmot_hip_memcpy_from_device(b->dev, (void *)p, (const uint8_t *)m->dev + (p - m->host), n);
    if (st != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(st);
    }
    b->downloads++;
    b->download_bytes += n;
    return MARMOT_SUCCESS;
}

static void drop_at(hip_backend_t *b, size_t i) {
    marmot_hip_free(b->dev, b->mirrors[i].dev);
    b->mirrored_bytes -= b->mirrors[i].bytes;
    memmove(&b->mirrors[i], &b->mirrors[i + 1], (b->n_mirrors - i - 1) * sizeof(hip_mirror_t));
    b->n_mirrors--;
}

// mirror covering [p, p+n): the existing one, or a new one over the union of [p, p+n) and every mirror it touches
static marmot_error_t cover(hip_backend_t *b, uintptr_t p, size_t n, bool will_read_host, hip_mirror_t **out) {
    hip_mirror_t *hit = find_containing(b, p, n);
    if (hit != nullptr) {
        *out = hit;
        return MARMOT_SUCCESS;
    }
    uintptr_t lo = p, hi = p + n;
    // bring device-newer bytes of overlapping mirrors home, then drop them; restart because the union may grow
    for (size_t i = 0; i < b->n_mirrors;) {
        hip_mirror_t *o = &b->mirrors[i];
        if (!overlaps(o, lo, hi - lo)) {
            ++i;
            continue;
        }
        if (o->dev_newer) {
            const marmot_error_t st = download(b, o, o->host, o->bytes);
            if (st != MARMOT_SUCCESS) {
                return st;
            }
        }
        if (o->host < lo) {
            lo = o->host;
        }
        if (o->host + o->bytes > hi) {
            hi = o->host + o->bytes;
        }
        drop_at(b, i);
        will_read_host = true;  // the union holds bytes that are only on the host now
        i = 0;
    }
    if (b->n_mirrors == b->cap_mirrors) {
        const size_t cap = b->cap_mirrors != 0 ? 2 * b->cap_mirrors : 64;
        hip_mirror_t *grown = realloc(b->mirrors, cap * sizeof(hip_mirror_t));
        if (grown == nullptr) {
            return fail(MARMOT_ERROR_OUT_OF_MEMORY, "HIP residency table: out of host memory");
        }
        b->mirrors = grown;
        b->cap_mirrors = cap;
    }
    hip_mirror_t m = {.host = lo, .bytes = hi - lo, .dev = nullptr, .host_newer = will_read_host, .dev_newer = false};
    const int st = marmot_hip_alloc(b->dev, m.bytes, &m.dev);
    if (st != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(st);
    }
    const size_t at = upper_bound(b, lo);
    memmove(&b->mirrors[at + 1], &b->mirrors[at], (b->n_mirrors - at) * sizeof(hip_mirror_t));
    b->mirrors[at] = m;
    b->n_mirrors++;
    b->mirrored_bytes += m.bytes;
    *out = &b->mirrors[at];
    return MARMOT_SUCCESS;
}

static void packs_invalidate(hip_backend_t *b, uintptr_t p, size_t n) {
    for (int i = 0; i < HIP_PACK_CACHE; ++i) {
        hip_pack_entry_t *e = &b->packs[i];
        if (e->valid && e->host < p + n && p < e->host + e->rows * e->cols * sizeof(float)) {
            e->valid = false;
        }
    }
}

static hip_pack_entry_t *packs_find(hip_backend_t *b, const void *host, size_t rows, size_t cols, int act_kind) {
    for (int i = 0; i < HIP_PACK_CACHE; ++i) {
        hip_pack_entry_t *e = &b->packs[i];
        if (e->valid && e->host == (uintptr_t)host && e->rows == rows && e->cols == cols && e->act_kind == act_kind) {
            e->stamp = ++b->pack_clock;
            return e;
        }
    }
    return nullptr;
}

// an entry (not yet valid) with room for the packed rows: an invalid one, else the least recently used
static marmot_error_t packs_reserve(hip_backend_t *b, int weight_kind, size_t rows, size_t cols,
                                    hip_pack_entry_t **out) {
    hip_pack_entry_t *e = &b->packs[0];
    for (int i = 0; i < HIP_PACK_CACHE; ++i) {
        hip_pack_entry_t *c = &b->packs[i];
        if (!c->valid) {
            e = c;
            break;
        }
        if (c->stamp < e->stamp) {
            e = c;
        }
    }
    e->valid = false;
    const size_t need = marmot_hip_packed_activation_bytes(weight_kind, rows, cols);
    if (need == 0) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "packed activations: unsupported weight kind");
    }
    if (e->capacity < need) {
        if (e->packed != nullptr) {
            marmot_hip_synchronize(b->dev);  // a kernel may still read the old buffer
            marmot_hip_free(b->dev, e->packed);
            e->packed = nullptr;
            e->capacity = 0;
        }
        const int st = marmot_hip_alloc(b->dev, need, &e->packed);
        if (st != MARMOT_HIP_SUCCESS) {
            return fail_from_lib(st);
        }
        e->capacity = need;
    }
    *out = e;
    return MARMOT_SUCCESS;
}

static int act_kind_of_weight(int weight_kind) {
    return marmot_hip_block_values(weight_kind) == 256 ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
}

// device address of a kernel input: uploads the mirror when the host copy is newer
static marmot_error_t acquire_read(hip_backend_t *b, const void *host, size_t n, const void **d_out) {
    hip_mirror_t *m = nullptr;
    marmot_error_t st = cover(b, (uintptr_t)host, n, true, &m);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    if (m->host_newer) {
        st = upload(b, m);
        if (st != MARMOT_SUCCESS) {
            return st;
        }
    }
    *d_out = (const uint8_t *)m->dev + ((uintptr_t)host - m->host);
    return MARMOT_SUCCESS;
}

// device address of a kernel output that is fully overwritten
static marmot_error_t acquire_write(hip_backend_t *b, void *host, size_t n, void **d_out) {
    hip_mirror_t *m = nullptr;
    marmot_error_t st = cover(b, (uintptr_t)host, n, false, &m);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    const bool whole = (uintptr_t)host == m->host && n == m->bytes;
    if (m->host_newer && !whole) {
        st = upload(b, m);  // keep the bytes of the mirror outside the output valid
        if (st != MARMOT_SUCCESS) {
            return st;
        }
    }
    m->host_newer = false;
    m->dev_newer = true;
    packs_invalidate(b, (uintptr_t)host, n);
    *d_out = (uint8_t *)m->dev + ((uintptr_t)host - m->host);
    return MARMOT_SUCCESS;
}

// device address of a kernel output whose rows lie further apart than their length: the bytes between the rows are
// not written by the kernel and must survive the next download of the range, so the host's bytes go up first
// whenever the device does not hold them yet
static marmot_error_t acquire_write_rows(hip_backend_t *b, void *host, size_t span, bool gaps, void **d_out) {
    if (gaps) {
        const void *unused = nullptr;
        const marmot_error_t st = acquire_read(b, host, span, &unused);
        if (st != MARMOT_SUCCESS) {
            return st;
        }
    }
    return acquire_write(b, host, span, d_out);
}

// Several tensors of one call. Covering a host range that overlaps existing mirrors replaces them by one mirror over
// the union (views of one buffer: gate / up halves, q / k / v slices), which frees their device memory: addresses
// taken earlier in the same call would dangle. So every range is covered first, and the addresses are taken in a
// second round, when every range lies inside a mirror and nothing is replaced any more.
typedef enum { HIP_ACQ_READ, HIP_ACQ_WRITE, HIP_ACQ_UPDATE } hip_acq_mode_t;
typedef struct {
    void *host;
    size_t bytes;
    hip_acq_mode_t mode;  // UPDATE: read and written, or written with gaps whose bytes must survive
    void *dev;
} hip_acq_t;

static marmot_error_t acquire_set(hip_backend_t *b, hip_acq_t *v, size_t n) {
    for (int round = 0; round < 2; ++round) {
        for (size_t i = 0; i < n; ++i) {
            marmot_error_t st;
            if (v[i].mode == HIP_ACQ_READ) {
                const void *d = nullptr;
                st = acquire_read(b, v[i].host, v[i].bytes, &d);
                v[i].dev = (void *)d;
            } else {
                st = acquire_write_rows(b, v[i].host, v[i].bytes, v[i].mode == HIP_ACQ_UPDATE, &v[i].dev);
            }
            if (st != MARMOT_SUCCESS) {
                return st;
            }
        }
    }
    return MARMOT_SUCCESS;
}

// ------------------------------------------------------------------ tensor helpers
static size_t dtype_size(marmot_dtype_t t) {
    switch (t) {
    case MARMOT_DTYPE_FLOAT32:
    case MARMOT_DTYPE_INT32:
    case MARMOT_DTYPE_UINT32:
        return 4;
    case MARMOT_DTYPE_FLOAT16:
    case MARMOT_DTYPE_BFLOAT16:
    case MARMOT_DTYPE_INT16:
    case MARMOT_DTYPE_UINT16:
        return 2;
    case MARMOT_DTYPE_INT8:
    case MARMOT_DTYPE_UINT8:
    case MARMOT_DTYPE_FLOAT8_E4M3:
    case MARMOT_DTYPE_FLOAT8_E5M2:
        return 1;
    case MARMOT_DTYPE_FLOAT64:
    case MARMOT_DTYPE_INT64:
    case MARMOT_DTYPE_UINT64:
        return 8;
    default:
        return 0;
    }
}

static bool kind_supported_weight(marmot_quant_kind_t k) {
    return k == MARMOT_QUANT_KIND_Q4_0 || k == MARMOT_QUANT_KIND_Q4_1 || k == MARMOT_QUANT_KIND_Q5_0 ||
        k == MARMOT_QUANT_KIND_Q5_1 || k == MARMOT_QUANT_KIND_Q8_0 || k == MARMOT_QUANT_KIND_Q8_1 ||
        k == MARMOT_QUANT_KIND_Q2_K ||
        k == MARMOT_QUANT_KIND_Q3_K || k == MARMOT_QUANT_KIND_Q4_K || k == MARMOT_QUANT_KIND_Q5_K ||
        k == MARMOT_QUANT_KIND_Q6_K;
}

static bool kind_is_block(marmot_quant_kind_t k) {
    return k > MARMOT_QUANT_KIND_GENERIC && k < MARMOT_QUANT_KIND_COUNT;
}

// block-quantized storage uses byte-sized elements (marmot_quant_storage_dtype_compatible, src/core/helpers/quant.c)
static bool storage_dtype_ok(marmot_dtype_t t) {
    return t == MARMOT_DTYPE_UINT8 || t == MARMOT_DTYPE_INT8;
}

static size_t tensor_numel(const marmot_tensor_t *t) {
    size_t n = 1;
    for (size_t i = 0; i < t->shape.ndim; ++i) {
        n *= t->shape.shape[i];
    }
    return n;
}

static size_t dense_bytes(const marmot_tensor_t *t) {
    return tensor_numel(t) * dtype_size(t->dtype);
}

static bool rows_contiguous(const marmot_tensor_t *t) {
    return t->shape.ndim == 2 && t->shape.strides[1] == 1 && t->shape.strides[0] == t->shape.shape[1];
}

// row-major without gaps, any rank
static bool dense_contiguous(const marmot_tensor_t *t) {
    size_t expect = 1;
    for (size_t i = t->shape.ndim; i-- > 0;) {
        if (t->shape.shape[i] != 1 && t->shape.strides[i] != expect) {
            return false;
        }
        expect *= t->shape.shape[i];
    }
    return true;
}

static void mark_device_output(marmot_tensor_t *t) {
    t->memory_location = MARMOT_MEMORY_DEVICE;
    t->needs_sync = true;
}

// ------------------------------------------------------------------ vtable
static marmot_error_t ops_init(void **device_ctx) {
    if (device_ctx == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP backend init: null device_ctx");
    }
    hip_backend_t *b = calloc(1, sizeof(*b));
    if (b == nullptr) {
        return fail(MARMOT_ERROR_OUT_OF_MEMORY, "HIP backend init: out of host memory");
    }
    const int st = marmot_hip_device_create(0, &b->dev);
    if (st != MARMOT_HIP_SUCCESS) {
        free(b);
        return fail_from_lib(st);
    }
    pthread_mutex_init(&b->mu, nullptr);
    *device_ctx = b;
    return MARMOT_SUCCESS;
}

static void ops_destroy(const void *device_ctx) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr) {
        return;
    }
    marmot_hip_synchronize(b->dev);
    for (size_t i = 0; i < b->n_mirrors; ++i) {
        marmot_hip_free(b->dev, b->mirrors[i].dev);
    }
    free(b->mirrors);
    for (int i = 0; i < HIP_PACK_CACHE; ++i) {
        if (b->packs[i].packed != nullptr) {
            marmot_hip_free(b->dev, b->packs[i].packed);
        }
    }
    for (size_t i = 0; i < HIP_ROPE_CACHE; ++i) {
        free(b->rope[i].freqs);
    }
    marmot_hip_device_destroy(b->dev);
    pthread_mutex_destroy(&b->mu);
    free(b);
}

static marmot_error_t ops_configure(const void *device_ctx, const marmot_context_t *ctx) {
    (void)ctx;
    return device_ctx != nullptr ? MARMOT_SUCCESS
                                 : fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP backend: null device_ctx");
}

static marmot_error_t ops_alloc(const void *device_ctx, size_t size, void **ptr) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || ptr == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP alloc: null argument");
    }
    const int st = marmot_hip_alloc(b->dev, size, ptr);
    return st == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(st);
}

static void ops_free(const void *device_ctx, void *ptr) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b != nullptr && ptr != nullptr) {
        marmot_hip_free(b->dev, ptr);
    }
}

// dst == src == host pointer: the host copy is newer than the mirror (src/core/tensor/transfer.c:22)
static marmot_error_t host_is_newer_locked(hip_backend_t *b, const void *src, size_t size) {
    const uintptr_t p = (uintptr_t)src;
    packs_invalidate(b, p, size);
    hip_mirror_t *m = find_containing(b, p, size);
    if (m != nullptr) {
        if (p == m->host && size == m->bytes) {
            m->host_newer = true;  // uploaded when a kernel next reads it
            m->dev_newer = false;
            return MARMOT_SUCCESS;
        }
        if (m->host_newer) {
            return MARMOT_SUCCESS;  // the whole mirror is refreshed on next use anyway
        }
        const int st = marmot_hip_memcpy_to_device(b->dev, (uint8_t *)m->dev + (p - m->host), src, size);
        if (st != MARMOT_HIP_SUCCESS) {
            return fail_from_lib(st);
        }
        b->uploads++;
        b->upload_bytes += size;
        return MARMOT_SUCCESS;
    }
    // not inside one mirror: partial overlaps are refreshed when a kernel next reads them
    bool any = false;
    for (size_t i = 0; i < b->n_mirrors; ++i) {
        if (overlaps(&b->mirrors[i], p, size)) {
            b->mirrors[i].host_newer = true;
            any = true;
        }
    }
    if (any) {
        return MARMOT_SUCCESS;
    }
    // A range the backend has never seen: marmot_tensor_to_device on a fresh tensor, which is how an execution session
    // puts a model's weights on the device before the first token (src/graph/execution_session.cpp:315-320). Mirror and
    // upload it now, so that the first kernel that reads it finds it resident.
    const void *d = nullptr;
    return acquire_read(b, src, size, &d);
}

static marmot_error_t ops_memcpy_to_device(const void *device_ctx, void *dst, const void *src, size_t size) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || dst == nullptr || src == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP memcpy_to_device: null argument");
    }
    if (size == 0) {
        return MARMOT_SUCCESS;
    }
    if (dst != src) {
        const int st = marmot_hip_memcpy_to_device(b->dev, dst, src, size);
        return st == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(st);
    }
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = host_is_newer_locked(b, src, size);
    pthread_mutex_unlock(&b->mu);
    return st;
}

// dst == src == host pointer: make the host copy current (src/core/tensor/transfer.c:49-55)
static marmot_error_t make_host_current_locked(hip_backend_t *b, void *dst, size_t size) {
    const uintptr_t p = (uintptr_t)dst;
    for (size_t i = 0; i < b->n_mirrors; ++i) {
        hip_mirror_t *m = &b->mirrors[i];
        if (!overlaps(m, p, size) || !m->dev_newer) {
            continue;
        }
        const uintptr_t lo = p > m->host ? p : m->host;
        const uintptr_t hi = (p + size) < (m->host + m->bytes) ? (p + size) : (m->host + m->bytes);
        const marmot_error_t st = download(b, m, lo, hi - lo);
        if (st != MARMOT_SUCCESS) {
            return st;
        }
        if (lo == m->host && hi == m->host + m->bytes) {
            m->dev_newer = false;
        }
    }
    return MARMOT_SUCCESS;
}

static marmot_error_t ops_memcpy_from_device(const void *device_ctx, void *dst, const void *src, size_t size) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || dst == nullptr || src == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP memcpy_from_device: null argument");
    }
    if (size == 0) {
        return MARMOT_SUCCESS;
    }
    if (dst != src) {
        const int st = marmot_hip_memcpy_from_device(b->dev, dst, src, size);
        return st == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(st);
    }
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = make_host_current_locked(b, dst, size);
    pthread_mutex_unlock(&b->mu);
    return st;
}

static marmot_error_t ops_synchronize(const void *device_ctx) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP synchronize: null device_ctx");
    }
    const int st = marmot_hip_synchronize(b->dev);
    return st == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(st);
}

static marmot_error_t ops_allocator_usage(const void *device_ctx, marmot_allocator_usage_t *usage) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || usage == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP allocator_usage: null argument");
    }
    size_t cur = 0, peak = 0, n = 0;
    const int st = marmot_hip_allocator_usage(b->dev, &cur, &peak, &n);
    if (st != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(st);
    }
    memset(usage, 0, sizeof(*usage));
    usage->current_bytes = cur;
    usage->peak_bytes = peak;
    usage->active_allocations = n;
    return MARMOT_SUCCESS;
}

// All kernels of a context are enqueued on one stream in program order, so a batch needs no extra bracket:
// begin/end only record the state that marmot_graph_batch_is_active reports.
static marmot_error_t ops_graph_batch_begin(void *device_ctx) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP graph_batch_begin: null device_ctx");
    }
    b->batching = true;
    return MARMOT_SUCCESS;
}

static marmot_error_t ops_graph_batch_end(void *device_ctx, bool commit) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP graph_batch_end: null device_ctx");
    }
    b->batching = false;
    (void)commit;  // work is already in flight; results are waited for by memcpy_from_device / synchronize
    return MARMOT_SUCCESS;
}

static void ops_on_host_range_freed(void *device_ctx, const void *start, size_t length) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || start == nullptr || length == 0) {
        return;
    }
    pthread_mutex_lock(&b->mu);
    packs_invalidate(b, (uintptr_t)start, length);
    bool synced = false;
    for (size_t i = 0; i < b->n_mirrors;) {
        if (!overlaps(&b->mirrors[i], (uintptr_t)start, length)) {
            ++i;
            continue;
        }
        if (!synced) {
            marmot_hip_synchronize(b->dev);  // kernels still reading the mirror finish first
            synced = true;
        }
        drop_at(b, i);
    }
    pthread_mutex_unlock(&b->mu);
}

static void ops_on_host_ptr_freed(void *device_ctx, const void *ptr) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || ptr == nullptr) {
        return;
    }
    size_t bytes = 1;
    pthread_mutex_lock(&b->mu);
    const size_t i = upper_bound(b, (uintptr_t)ptr);
    if (i > 0 && b->mirrors[i - 1].host == (uintptr_t)ptr) {
        bytes = b->mirrors[i - 1].bytes;
    }
    pthread_mutex_unlock(&b->mu);
    ops_on_host_range_freed(device_ctx, ptr, bytes);
}

static const marmot_device_ops_t k_hip_ops = {
    .init = ops_init,
    .destroy = ops_destroy,
    .configure = ops_configure,
    .alloc = ops_alloc,
    .free = ops_free,
    .memcpy_to_device = ops_memcpy_to_device,
    .memcpy_from_device = ops_memcpy_from_device,
    .synchronize = ops_synchronize,
    .allocator_usage = ops_allocator_usage,
    .graph_batch_begin = ops_graph_batch_begin,
    .graph_batch_end = ops_graph_batch_end,
    .on_host_ptr_freed = ops_on_host_ptr_freed,
    .on_host_range_freed = ops_on_host_range_freed,
};

// ------------------------------------------------------------------ impl functions
typedef struct {
    int kind, in_dtype, out_dtype, bias_dtype;
    size_t N, K, M;
} matmul_plan_t;

static marmot_error_t matmul_locked(hip_backend_t *b, const matmul_plan_t *p, const marmot_tensor_t *input,
                                    const marmot_tensor_t *weight, const marmot_tensor_t *bias, marmot_tensor_t *out) {
    hip_acq_t acq[4] = {
        {weight->data, p->M * marmot_hip_row_bytes(p->kind, p->K), HIP_ACQ_READ, nullptr},
        {input->data, dense_bytes(input), HIP_ACQ_READ, nullptr},
        {out->data, dense_bytes(out), HIP_ACQ_WRITE, nullptr},
        {bias != nullptr ? bias->data : nullptr, bias != nullptr ? dense_bytes(bias) : 0, HIP_ACQ_READ, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, bias != nullptr ? 4 : 3);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    const void *d_w = acq[0].dev, *d_x = acq[1].dev, *d_b = bias != nullptr ? acq[3].dev : nullptr;
    void *d_y = acq[2].dev;
    int rc;
    if (p->in_dtype == MARMOT_HIP_DTYPE_F32 && p->N >= HIP_PACK_MIN_ROWS) {
        // fp32 rows that a normalization already left packed, or that an earlier linear packed: no quantization
        // launch; otherwise pack them here, once, for this linear and the ones that share its input
        const int act_kind = act_kind_of_weight(p->kind);
        hip_pack_entry_t *e = packs_find(b, input->data, p->N, p->K, act_kind);
        if (e != nullptr) {
            b->pack_hits++;
        } else {
            st = packs_reserve(b, p->kind, p->N, p->K, &e);
            if (st != MARMOT_SUCCESS) {
                return st;
            }
            rc = marmot_hip_pack_activations(b->dev, p->kind, d_x, MARMOT_HIP_DTYPE_F32, p->N, p->K, e->packed);
            if (rc != MARMOT_HIP_SUCCESS) {
                return fail_from_lib(rc);
            }
            e->valid = true;
            e->host = (uintptr_t)input->data;
            e->rows = p->N;
            e->cols = p->K;
            e->act_kind = act_kind;
            e->stamp = ++b->pack_clock;
            b->packs_made++;
        }
        rc = marmot_hip_matmul_prepacked(b->dev, p->kind, d_w, e->packed, p->N, p->K, p->M, d_b, p->bias_dtype, d_y,
                                         p->out_dtype);
    } else {
        rc = marmot_hip_matmul_quantized(b->dev, p->kind, d_w, d_x, p->in_dtype, p->N, p->K, p->M, d_b, p->bias_dtype,
                                         d_y, p->out_dtype, 0);
    }
    if (rc != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(rc);
    }
    mark_device_output(out);
    return MARMOT_SUCCESS;
}

static marmot_error_t matmul_quantized(const void *device_ctx, marmot_quant_kind_t expect_kind,
                                       const marmot_tensor_t *input, const marmot_tensor_t *weight,
                                       const marmot_matmul_epilogue_t *epilogue, marmot_tensor_t *out) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || weight == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Quantized matmul: null argument");
    }
    // marmot_matmul_validate_quantized (src/core/helpers/matmul.c:68-136), same order of checks
    if (!kind_is_block(weight->quant_kind)) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Weight tensor is not block-quantized");
    }
    if (weight->quant_layout != MARMOT_QUANT_LAYOUT_GGUF) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Quantized matmul only supports the GGUF layout");
    }
    if (!storage_dtype_ok(weight->dtype)) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Quantized weight uses an unexpected storage dtype");
    }
    if (input == nullptr || out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Quantized matmul: null argument");
    }
    if (input->shape.ndim != 2 || weight->shape.ndim != 2 || out->shape.ndim != 2) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Quantized matmul expects 2D tensors");
    }
    const bool in32 = input->dtype == MARMOT_DTYPE_FLOAT32, in16 = input->dtype == MARMOT_DTYPE_FLOAT16;
    const bool out32 = out->dtype == MARMOT_DTYPE_FLOAT32, out16 = out->dtype == MARMOT_DTYPE_FLOAT16;
    if (!((in32 && out32) || (in16 && (out32 || out16)))) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE,
                    "Quantized matmul requires FLOAT32 input or FLOAT16 activations with FLOAT16/FLOAT32 output");
    }
    matmul_plan_t p = {
        .kind = (int)weight->quant_kind,
        .in_dtype = in32 ? MARMOT_HIP_DTYPE_F32 : MARMOT_HIP_DTYPE_F16,
        .out_dtype = out32 ? MARMOT_HIP_DTYPE_F32 : MARMOT_HIP_DTYPE_F16,
        .bias_dtype = MARMOT_HIP_DTYPE_F32,
        .N = input->shape.shape[0],
        .K = input->shape.shape[1],
        .M = weight->shape.shape[0],
    };
    if (weight->shape.shape[1] != p.K) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Quantized matmul dimension mismatch on K");
    }
    if (out->shape.shape[0] != p.N || out->shape.shape[1] != p.M) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Quantized matmul output shape mismatch");
    }
    if (weight->quant_kind != expect_kind || !kind_supported_weight(weight->quant_kind)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Quantized matmul: weight scheme not handled by this kernel");
    }
    if (!rows_contiguous(input) || !rows_contiguous(out)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Quantized matmul: HIP kernels need contiguous rows");
    }
    if (input->data == nullptr || weight->data == nullptr || out->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Quantized matmul: tensor without data");
    }
    const marmot_tensor_t *bias = epilogue != nullptr ? epilogue->bias : nullptr;
    if (bias != nullptr) {
        if (tensor_numel(bias) != p.M) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Quantized matmul bias length mismatch");
        }
        if (bias->dtype == MARMOT_DTYPE_FLOAT16) {
            p.bias_dtype = MARMOT_HIP_DTYPE_F16;
        } else if (bias->dtype != MARMOT_DTYPE_FLOAT32) {
            return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Quantized matmul bias must be FLOAT32 or FLOAT16");
        }
    }
    if (p.N == 0 || p.M == 0) {
        mark_device_output(out);
        return MARMOT_SUCCESS;
    }
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = matmul_locked(b, &p, input, weight, bias, out);
    pthread_mutex_unlock(&b->mu);
    return st;
}

// marmot_matmul_qkv, separate block-quantized weights. Checks in the order of cpu_matmul_qkv_validate_desc
// (src/backends/cpu/ops/matmul/qkv/matmul_qkv.c:1140-1146, 1230-1300), cpu_matmul_qkv_quant_entry (:1424-1434) and
// cpu_matmul_qkv_run_separate_quantized_impl (:761-789).
// Finds or builds the frequency entry for these parameters (mutex held). An evicted entry's mirror is dropped first.
static marmot_error_t rope_entry_locked(hip_backend_t *b, const marmot_rope_params_t *r, size_t M,
                                        hip_rope_entry_t **out) {
    for (size_t i = 0; i < HIP_ROPE_CACHE; ++i) {
        hip_rope_entry_t *e = &b->rope[i];
        if (e->used && e->scaling_type == (int)r->scaling_type && e->theta == r->theta &&
            e->freq_scale == r->freq_scale && e->ext_factor == r->ext_factor && e->attn_factor == r->attn_factor &&
            e->beta_fast == r->beta_fast && e->beta_slow == r->beta_slow && e->orig_ctx_len == r->orig_ctx_len &&
            e->head_dim_in == r->head_dim && e->M == M) {
            *out = e;
            return MARMOT_SUCCESS;
        }
    }
    float *freqs = malloc((M / 2 + 1) * sizeof(float));
    if (freqs == nullptr) {
        return fail(MARMOT_ERROR_OUT_OF_MEMORY, "Failed to allocate RoPE frequency buffer");
    }
    float attn_scale = 1.0f;
    uint32_t head_dim = 0;
    const int rc = marmot_hip_rope_frequencies((int)r->scaling_type, r->theta, r->freq_scale, r->ext_factor,
                                               r->attn_factor, r->beta_fast, r->beta_slow, r->orig_ctx_len,
                                               r->head_dim, M, freqs, &attn_scale, &head_dim);
    if (rc != MARMOT_HIP_SUCCESS) {
        free(freqs);
        return fail_from_lib(rc);
    }
    hip_rope_entry_t *e = &b->rope[b->rope_next];
    b->rope_next = (b->rope_next + 1) % HIP_ROPE_CACHE;
    if (e->used && e->freqs != nullptr) {
        bool synced = false;
        for (size_t i = 0; i < b->n_mirrors;) {
            if (!overlaps(&b->mirrors[i], (uintptr_t)e->freqs, (size_t)e->head_dim / 2 * sizeof(float))) {
                ++i;
                continue;
            }
            if (!synced) {
                marmot_hip_synchronize(b->dev);
                synced = true;
            }
            drop_at(b, i);
        }
        free(e->freqs);
    }
    *e = (hip_rope_entry_t){.used = true, .scaling_type = (int)r->scaling_type, .theta = r->theta,
                            .freq_scale = r->freq_scale, .ext_factor = r->ext_factor,
                            .attn_factor = r->attn_factor, .beta_fast = r->beta_fast, .beta_slow = r->beta_slow,
                            .orig_ctx_len = r->orig_ctx_len, .head_dim_in = r->head_dim, .M = M,
                            .head_dim = head_dim, .attn_scale = attn_scale, .freqs = freqs};
    *out = e;
    return MARMOT_SUCCESS;
}

static marmot_error_t qkv_locked(hip_backend_t *b, const marmot_matmul_qkv_desc_t *desc, int kind, int dtype, size_t N,
                                 size_t K, size_t M) {
    const marmot_tensor_t *w[3] = {desc->separate.wq, desc->separate.wk, desc->separate.wv};
    const marmot_tensor_t *bias[3] = {desc->separate.bq, desc->separate.bk, desc->separate.bv};
    marmot_tensor_t *out[3] = {desc->out_q, desc->out_k, desc->out_v};
    // every range of the call in one set: input, three weights, three outputs, then the optional ones
    const marmot_rope_params_t *r = desc->rope_params;
    const bool with_rope = r != nullptr && (r->apply_to_q || r->apply_to_k);
    hip_rope_entry_t *e = nullptr;
    marmot_error_t st = MARMOT_SUCCESS;
    if (with_rope) {
        st = rope_entry_locked(b, r, M, &e);
        if (st != MARMOT_SUCCESS) {
            return st;
        }
    }
    hip_acq_t acq[12];
    size_t n_acq = 0;
    acq[n_acq++] = (hip_acq_t){desc->input->data, dense_bytes(desc->input), HIP_ACQ_READ, nullptr};
    for (int i = 0; i < 3; ++i) {
        acq[n_acq++] = (hip_acq_t){w[i]->data, M * marmot_hip_row_bytes(kind, K), HIP_ACQ_READ, nullptr};
    }
    for (int i = 0; i < 3; ++i) {
        acq[n_acq++] = (hip_acq_t){out[i]->data, dense_bytes(out[i]), HIP_ACQ_WRITE, nullptr};
    }
    int bias_at[3] = {-1, -1, -1}, pos_at = -1, freqs_at = -1;
    for (int i = 0; i < 3; ++i) {
        if (bias[i] != nullptr) {
            bias_at[i] = (int)n_acq;
            acq[n_acq++] = (hip_acq_t){bias[i]->data, dense_bytes(bias[i]), HIP_ACQ_READ, nullptr};
        }
    }
    if (with_rope) {
        pos_at = (int)n_acq;
        acq[n_acq++] = (hip_acq_t){r->positions->data, dense_bytes(r->positions), HIP_ACQ_READ, nullptr};
        freqs_at = (int)n_acq;
        acq[n_acq++] = (hip_acq_t){e->freqs, (size_t)e->head_dim / 2 * sizeof(float), HIP_ACQ_READ, nullptr};
    }
    st = acquire_set(b, acq, n_acq);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    const void *d_x = acq[0].dev;
    const void *d_w[3] = {acq[1].dev, acq[2].dev, acq[3].dev}, *d_b[3] = {nullptr, nullptr, nullptr};
    void *d_o[3] = {acq[4].dev, acq[5].dev, acq[6].dev};
    for (int i = 0; i < 3; ++i) {
        if (bias_at[i] >= 0) {
            d_b[i] = acq[bias_at[i]].dev;
        }
    }
    marmot_hip_rope_t rope;
    const marmot_hip_rope_t *rope_ptr = nullptr;
    if (with_rope) {
        const void *d_pos = acq[pos_at].dev, *d_freqs = acq[freqs_at].dev;
        rope = (marmot_hip_rope_t){
            .d_positions = d_pos,
            .positions_dtype = r->positions->dtype == MARMOT_DTYPE_FLOAT32 ? MARMOT_HIP_DTYPE_F32
                : r->positions->dtype == MARMOT_DTYPE_INT32               ? MARMOT_HIP_DTYPE_I32
                                                                          : MARMOT_HIP_DTYPE_I64,
            .d_freqs = d_freqs,
            .attn_scale = e->attn_scale,
            .head_dim = e->head_dim,
            .rope_type = r->rope_type == MARMOT_ROPE_TYPE_NEOX ? 1 : 0,
            .apply_to_q = r->apply_to_q,
            .apply_to_k = r->apply_to_k,
        };
        rope_ptr = &rope;
    }
    const int rc = marmot_hip_matmul_qkv_rope_quantized(b->dev, kind, d_w[0], d_w[1], d_w[2], d_x, dtype, N, K, M,
                                                        d_b[0], d_b[1], d_b[2], dtype, d_o[0], d_o[1], d_o[2], dtype,
                                                        rope_ptr);
    if (rc != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(rc);
    }
    for (int i = 0; i < 3; ++i) {
        mark_device_output(out[i]);
    }
    return MARMOT_SUCCESS;
}

static marmot_error_t matmul_qkv(const void *device_ctx, marmot_quant_kind_t expect_kind,
                                 const marmot_matmul_qkv_desc_t *desc) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "QKV projection: null device context");
    }
    if (desc == nullptr || desc->input == nullptr || desc->out_q == nullptr || desc->out_k == nullptr ||
        desc->out_v == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "QKV projection: null argument");
    }
    if (desc->layout == MARMOT_QKV_LAYOUT_FUSED) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Quantized fused QKV weights are not supported yet");
    }
    if (desc->layout != MARMOT_QKV_LAYOUT_SEPARATE) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Invalid QKV layout for HIP backend");
    }
    const marmot_tensor_t *input = desc->input;
    const marmot_tensor_t *w[3] = {desc->separate.wq, desc->separate.wk, desc->separate.wv};
    const marmot_tensor_t *bias[3] = {desc->separate.bq, desc->separate.bk, desc->separate.bv};
    marmot_tensor_t *out[3] = {desc->out_q, desc->out_k, desc->out_v};
    if (w[0] == nullptr || w[1] == nullptr || w[2] == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Separate QKV requires three weight tensors");
    }
    for (int i = 0; i < 3; ++i) {
        if (input->dtype != out[i]->dtype) {
            return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "QKV tensors must share dtype");
        }
    }
    if (input->shape.ndim != 2) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Separate QKV expects 2D tensors");
    }
    for (int i = 0; i < 3; ++i) {
        if (w[i]->shape.ndim != 2 || out[i]->shape.ndim != 2) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Separate QKV expects 2D tensors");
        }
    }
    const size_t N = input->shape.shape[0], K = input->shape.shape[1], M = w[0]->shape.shape[0];
    for (int i = 0; i < 3; ++i) {
        if (w[i]->shape.shape[1] != K) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Separate QKV weights must share the input dimension");
        }
    }
    if (w[1]->shape.shape[0] != M || w[2]->shape.shape[0] != M) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Separate QKV weights must share the output dimension");
    }
    for (int i = 0; i < 3; ++i) {
        if (out[i]->shape.shape[0] != N || out[i]->shape.shape[1] != M) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Separate QKV output shape mismatch");
        }
    }
    for (int i = 0; i < 3; ++i) {
        if (bias[i] == nullptr) {
            continue;
        }
        if (bias[i]->dtype != input->dtype) {
            return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Separate QKV bias dtype must match activations");
        }
        if (bias[i]->shape.ndim != 1 || bias[i]->shape.shape[0] != M) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Separate QKV bias must be 1D and match rows");
        }
        if (bias[i]->shape.strides[0] != 1) {
            return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Separate QKV bias must be contiguous");
        }
    }
    if (desc->epilogue != nullptr && desc->epilogue->bias != nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT,
                    "Separate QKV epilogue bias must be supplied via the descriptor bias tensors");
    }
    // the kernel entry: block-quantized GGUF weights of the kind this kernel was selected for
    for (int i = 0; i < 3; ++i) {
        if (!kind_is_block(w[i]->quant_kind) || w[i]->quant_layout != MARMOT_QUANT_LAYOUT_GGUF ||
            w[i]->quant_kind != expect_kind || !kind_supported_weight(w[i]->quant_kind)) {
            return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "QKV projection: weight scheme not handled by this kernel");
        }
    }
    if (input->dtype != MARMOT_DTYPE_FLOAT32 && input->dtype != MARMOT_DTYPE_FLOAT16) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "QKV projection takes FLOAT32 or FLOAT16 activations");
    }
    if (!rows_contiguous(input) || !rows_contiguous(out[0]) || !rows_contiguous(out[1]) || !rows_contiguous(out[2])) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "QKV projection: HIP kernels need contiguous rows");
    }
    if (desc->rope_params != nullptr && (desc->rope_params->apply_to_q || desc->rope_params->apply_to_k)) {
        const marmot_tensor_t *pos = desc->rope_params->positions;
        if (pos == nullptr || pos->data == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "QKV projection: RoPE needs a positions tensor");
        }
        if (pos->dtype != MARMOT_DTYPE_FLOAT32 && pos->dtype != MARMOT_DTYPE_INT32 &&
            pos->dtype != MARMOT_DTYPE_INT64) {
            return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "QKV projection: RoPE positions must be FLOAT32, INT32 or INT64");
        }
        if (tensor_numel(pos) < N) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "QKV projection: fewer RoPE positions than activation rows");
        }
        if (desc->rope_params->rope_type != MARMOT_ROPE_TYPE_NORM &&
            desc->rope_params->rope_type != MARMOT_ROPE_TYPE_NEOX) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "QKV projection: unknown RoPE type");
        }
    }
    if (input->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "QKV projection: tensor without data");
    }
    for (int i = 0; i < 3; ++i) {
        if (w[i]->data == nullptr || out[i]->data == nullptr || (bias[i] != nullptr && bias[i]->data == nullptr)) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "QKV projection: tensor without data");
        }
    }
    if (N == 0 || M == 0) {
        for (int i = 0; i < 3; ++i) {
            mark_device_output(out[i]);
        }
        return MARMOT_SUCCESS;
    }
    const int dtype = input->dtype == MARMOT_DTYPE_FLOAT32 ? MARMOT_HIP_DTYPE_F32 : MARMOT_HIP_DTYPE_F16;
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = qkv_locked(b, desc, (int)expect_kind, dtype, N, K, M);
    pthread_mutex_unlock(&b->mu);
    return st;
}

// marmot_embedding_gather, block-quantized table (embedding_scalar.c:460-591)
static marmot_error_t embedding_gather(const void *device_ctx, const marmot_embedding_gather_desc_t *desc) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || desc == nullptr || desc->weights == nullptr || desc->token_ids == nullptr ||
        desc->out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Embedding gather: null argument");
    }
    const marmot_tensor_t *weights = desc->weights, *ids = desc->token_ids;
    marmot_tensor_t *out = desc->out;
    if (weights->shape.ndim != 2) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Embedding weights must be 2D");
    }
    if (!kind_is_block(weights->quant_kind) || weights->quant_layout != MARMOT_QUANT_LAYOUT_GGUF) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Unsupported quantized embedding layout");
    }
    if (!kind_supported_weight(weights->quant_kind)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Quantized embedding kind not supported on HIP");
    }
    const size_t vocab = weights->shape.shape[0], dim = weights->shape.shape[1];
    const size_t tokens = tensor_numel(ids);
    if (ids->dtype != MARMOT_DTYPE_INT32 && ids->dtype != MARMOT_DTYPE_INT64) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Unsupported token dtype for HIP embedding gather");
    }
    if (out->dtype != MARMOT_DTYPE_FLOAT32 && out->dtype != MARMOT_DTYPE_FLOAT16) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "HIP embedding gather writes FLOAT32 or FLOAT16");
    }
    if (tensor_numel(out) != tokens * dim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Embedding output must hold tokens x dim values");
    }
    if (!dense_contiguous(out) || !dense_contiguous(ids)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "Embedding gather: HIP kernels need contiguous tensors");
    }
    if (weights->data == nullptr || ids->data == nullptr || out->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Embedding gather: tensor without data");
    }
    if (tokens == 0 || dim == 0) {
        mark_device_output(out);
        return MARMOT_SUCCESS;
    }
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[3] = {
        {weights->data, vocab * marmot_hip_row_bytes((int)weights->quant_kind, dim), HIP_ACQ_READ, nullptr},
        {ids->data, dense_bytes(ids), HIP_ACQ_READ, nullptr},
        {out->data, dense_bytes(out), HIP_ACQ_WRITE, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, 3);
    const void *d_w = acq[0].dev, *d_ids = acq[1].dev;
    void *d_out = acq[2].dev;
    // the library takes at most 65535 tokens per call
    const size_t id_size = dtype_size(ids->dtype), row_size = dim * dtype_size(out->dtype);
    for (size_t t0 = 0; st == MARMOT_SUCCESS && t0 < tokens; t0 += 65535) {
        const size_t n = tokens - t0 < 65535 ? tokens - t0 : 65535;
        const int rc = marmot_hip_embedding_gather_quantized(
            b->dev, (int)weights->quant_kind, d_w, vocab, dim, (const uint8_t *)d_ids + t0 * id_size,
            ids->dtype == MARMOT_DTYPE_INT32 ? MARMOT_HIP_DTYPE_I32 : MARMOT_HIP_DTYPE_I64, n,
            (uint8_t *)d_out + t0 * row_size,
            out->dtype == MARMOT_DTYPE_FLOAT32 ? MARMOT_HIP_DTYPE_F32 : MARMOT_HIP_DTYPE_F16, desc->scale,
            desc->padding_id, desc->bounds_check ? 1 : 0);
        if (rc == MARMOT_HIP_ERROR_INVALID_ARGUMENT) {
            st = fail(MARMOT_ERROR_INVALID_ARGUMENT, "Embedding id out of range");
        } else if (rc != MARMOT_HIP_SUCCESS) {
            st = fail_from_lib(rc);
        }
    }
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    pthread_mutex_unlock(&b->mu);
    return st;
}

// bytes of E expert slices of [rows, cols] blocks; expert tensors are stored [cols, rows, E] in GGUF order
// (cpu_moe_execute_grouped, src/backends/cpu/ops/moe/moe_ops.c:895-899)
static size_t expert_tensor_bytes(int kind, size_t rows, size_t cols, size_t experts) {
    return experts * rows * marmot_hip_row_bytes(kind, cols);
}

static marmot_error_t moe_locked(hip_backend_t *b, const marmot_moe_experts_desc_t *desc, size_t T, size_t H, size_t F,
                                 size_t E, size_t k) {
    const marmot_tensor_t *h = desc->hidden_states, *g = desc->gate_exps, *u = desc->up_exps, *d = desc->down_exps;
    const int kgu = (int)g->quant_kind, kd = (int)d->quant_kind;
    hip_acq_t acq[7] = {
        {h->data, dense_bytes(h), HIP_ACQ_READ, nullptr},
        {g->data, expert_tensor_bytes(kgu, F, H, E), HIP_ACQ_READ, nullptr},
        {u->data, expert_tensor_bytes(kgu, F, H, E), HIP_ACQ_READ, nullptr},
        {d->data, expert_tensor_bytes(kd, H, F, E), HIP_ACQ_READ, nullptr},
        {desc->topk_ids->data, dense_bytes(desc->topk_ids), HIP_ACQ_READ, nullptr},
        {desc->topk_weights->data, dense_bytes(desc->topk_weights), HIP_ACQ_READ, nullptr},
        {desc->out->data, dense_bytes(desc->out), HIP_ACQ_WRITE, nullptr},
    };
    const marmot_error_t st = acquire_set(b, acq, 7);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    const void *d_h = acq[0].dev, *d_g = acq[1].dev, *d_u = acq[2].dev, *d_d = acq[3].dev, *d_ids = acq[4].dev,
               *d_wts = acq[5].dev;
    void *d_out = acq[6].dev;
    const int rc = marmot_hip_moe_experts(b->dev, (const float *)d_h, T, H, F, E, k, kgu, kd, d_g, d_u, d_d,
                                          (const int32_t *)d_ids, (const float *)d_wts, desc->weights_scale,
                                          (int)desc->router_weight_policy, (int)desc->ffn_type, (float *)d_out);
    if (rc != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(rc);
    }
    mark_device_output(desc->out);
    return MARMOT_SUCCESS;
}

static marmot_error_t moe_experts(const void *device_ctx, const marmot_moe_experts_desc_t *desc) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || desc == nullptr || desc->hidden_states == nullptr || desc->gate_exps == nullptr ||
        desc->up_exps == nullptr || desc->down_exps == nullptr || desc->topk_ids == nullptr ||
        desc->topk_weights == nullptr || desc->out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "MoE descriptor is incomplete");
    }
    const marmot_tensor_t *h = desc->hidden_states, *g = desc->gate_exps, *u = desc->up_exps, *d = desc->down_exps;
    if (g->quant_kind != u->quant_kind || g->quant_layout != u->quant_layout) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "MoE expert quantization must be consistent across weights");
    }
    if (h->dtype != MARMOT_DTYPE_FLOAT32 || desc->topk_weights->dtype != MARMOT_DTYPE_FLOAT32 ||
        desc->out->dtype != MARMOT_DTYPE_FLOAT32 || desc->topk_ids->dtype != MARMOT_DTYPE_INT32) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "HIP MoE experts need FLOAT32 activations and INT32 expert ids");
    }
    if (!kind_supported_weight(g->quant_kind) || !kind_supported_weight(d->quant_kind)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP MoE experts need Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 or Q2_K to Q6_K expert weights");
    }
    if (h->shape.ndim != 2 || g->shape.ndim != 3 || u->shape.ndim != 3 || d->shape.ndim != 3 ||
        desc->topk_ids->shape.ndim != 2 || desc->topk_weights->shape.ndim != 2 || desc->out->shape.ndim != 2) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "MoE experts: unexpected tensor ranks");
    }
    const size_t T = h->shape.shape[0], H = h->shape.shape[1];
    const size_t F = g->shape.shape[1], E = g->shape.shape[2], k = desc->topk_ids->shape.shape[1];
    if (g->shape.shape[0] != H || u->shape.shape[0] != H || u->shape.shape[1] != F || u->shape.shape[2] != E ||
        d->shape.shape[0] != F || d->shape.shape[1] != H || d->shape.shape[2] != E ||
        desc->topk_ids->shape.shape[0] != T || desc->topk_weights->shape.shape[0] != T ||
        desc->topk_weights->shape.shape[1] != k || desc->out->shape.shape[0] != T ||
        desc->out->shape.shape[1] != H) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "MoE experts: tensor shapes do not agree");
    }
    if (!rows_contiguous(h) || !rows_contiguous(desc->out) || !rows_contiguous(desc->topk_ids) ||
        !rows_contiguous(desc->topk_weights)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "MoE experts: HIP kernels need contiguous rows");
    }
    if (T == 0) {
        mark_device_output(desc->out);
        return MARMOT_SUCCESS;
    }
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = moe_locked(b, desc, T, H, F, E, k);
    pthread_mutex_unlock(&b->mu);
    return st;
}

static marmot_error_t topk_locked(hip_backend_t *b, const marmot_topk_desc_t *desc, size_t rows, size_t cols) {
    hip_acq_t acq[3] = {
        {desc->x->data, dense_bytes(desc->x), HIP_ACQ_READ, nullptr},
        {desc->values_out->data, dense_bytes(desc->values_out), HIP_ACQ_WRITE, nullptr},
        {desc->indices_out->data, dense_bytes(desc->indices_out), HIP_ACQ_WRITE, nullptr},
    };
    const marmot_error_t st = acquire_set(b, acq, 3);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    const void *d_x = acq[0].dev;
    void *d_v = acq[1].dev, *d_i = acq[2].dev;
    const int rc = marmot_hip_topk(b->dev, (const float *)d_x, rows, cols, desc->k, (float *)d_v, (int32_t *)d_i);
    if (rc != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(rc);
    }
    mark_device_output(desc->values_out);
    mark_device_output(desc->indices_out);
    return MARMOT_SUCCESS;
}

static marmot_error_t topk(const void *device_ctx, const marmot_topk_desc_t *desc) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || desc == nullptr || desc->x == nullptr || desc->values_out == nullptr ||
        desc->indices_out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "TopK descriptor is incomplete");
    }
    const marmot_tensor_t *x = desc->x;
    if (x->shape.ndim != 2 || desc->values_out->shape.ndim != 2 || desc->indices_out->shape.ndim != 2) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "TopK expects 2D tensors");
    }
    if (desc->axis != 1 && desc->axis != -1) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "TopK is implemented over the last axis");
    }
    if (x->dtype != MARMOT_DTYPE_FLOAT32 || desc->values_out->dtype != MARMOT_DTYPE_FLOAT32 ||
        desc->indices_out->dtype != MARMOT_DTYPE_INT32) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "HIP TopK needs FLOAT32 values and INT32 indices");
    }
    const size_t rows = x->shape.shape[0], cols = x->shape.shape[1], k = desc->k;
    // cpu_topk_impl, src/backends/cpu/ops/moe/moe_ops.c:813-820
    if (k == 0 || k > cols || desc->values_out->shape.shape[0] != rows || desc->indices_out->shape.shape[0] != rows ||
        desc->values_out->shape.shape[1] != k || desc->indices_out->shape.shape[1] != k) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "TopK output shape mismatch");
    }
    if (!rows_contiguous(x) || !rows_contiguous(desc->values_out) || !rows_contiguous(desc->indices_out)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "TopK: HIP kernel needs contiguous rows");
    }
    if (rows == 0) {
        return MARMOT_SUCCESS;
    }
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = topk_locked(b, desc, rows, cols);
    pthread_mutex_unlock(&b->mu);
    return st;
}

static marmot_error_t quantize_locked(hip_backend_t *b, const marmot_tensor_t *input, marmot_tensor_t *output,
                                      size_t rows, size_t k) {
    const int kind = (int)output->quant_kind;
    hip_acq_t acq[2] = {
        {input->data, dense_bytes(input), HIP_ACQ_READ, nullptr},
        {output->data, rows * marmot_hip_row_bytes(kind, k), HIP_ACQ_WRITE, nullptr},
    };
    const marmot_error_t st = acquire_set(b, acq, 2);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    const void *d_x = acq[0].dev;
    void *d_q = acq[1].dev;
    int rc;
    if (kind == MARMOT_QUANT_KIND_Q8_0 || kind == MARMOT_QUANT_KIND_Q8_K) {
        rc = marmot_hip_quantize_activations(
            b->dev, kind, d_x, input->dtype == MARMOT_DTYPE_FLOAT32 ? MARMOT_HIP_DTYPE_F32 : MARMOT_HIP_DTYPE_F16, rows,
            k, d_q);
    } else {
        rc = marmot_hip_quantize_weights(b->dev, kind, (const float *)d_x, rows, k, d_q);
    }
    if (rc != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(rc);
    }
    mark_device_output(output);
    return MARMOT_SUCCESS;
}

static marmot_error_t quantize_block(const void *device_ctx, const marmot_tensor_t *input, marmot_tensor_t *output) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || input == nullptr || output == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Quantize: null argument");
    }
    const bool act_kind = output->quant_kind == MARMOT_QUANT_KIND_Q8_0 || output->quant_kind == MARMOT_QUANT_KIND_Q8_K;
    const bool weight_kind = output->quant_kind == MARMOT_QUANT_KIND_Q4_K ||
        output->quant_kind == MARMOT_QUANT_KIND_Q5_K || output->quant_kind == MARMOT_QUANT_KIND_Q6_K;
    if (!act_kind && !weight_kind) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED,
                    "HIP quantize produces the activation formats Q8_0 and Q8_K and the weight formats Q4_K, Q5_K and Q6_K");
    }
    if (input->dtype != MARMOT_DTYPE_FLOAT32 && !(act_kind && input->dtype == MARMOT_DTYPE_FLOAT16)) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE,
                    "Quantize input must be FLOAT32 (or FLOAT16 for the activation formats)");
    }
    if (!rows_contiguous(input)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Quantize expects a contiguous 2D input");
    }
    const size_t rows = input->shape.shape[0], k = input->shape.shape[1];
    if (rows == 0 || k == 0) {
        return MARMOT_SUCCESS;
    }
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = quantize_locked(b, input, output, rows, k);
    pthread_mutex_unlock(&b->mu);
    return st;
}

static marmot_error_t dequantize_locked(hip_backend_t *b, const marmot_tensor_t *input, marmot_tensor_t *output,
                                        size_t rows, size_t k) {
    const int kind = (int)input->quant_kind;
    hip_acq_t acq[2] = {
        {input->data, rows * marmot_hip_row_bytes(kind, k), HIP_ACQ_READ, nullptr},
        {output->data, dense_bytes(output), HIP_ACQ_WRITE, nullptr},
    };
    const marmot_error_t st = acquire_set(b, acq, 2);
    if (st != MARMOT_SUCCESS) {
        return st;
    }
    const void *d_q = acq[0].dev;
    void *d_y = acq[1].dev;
    const int rc = marmot_hip_dequantize(b->dev, kind, d_q, rows, k, (float *)d_y);
    if (rc != MARMOT_HIP_SUCCESS) {
        return fail_from_lib(rc);
    }
    mark_device_output(output);
    return MARMOT_SUCCESS;
}

static marmot_error_t dequantize_block(const void *device_ctx, const marmot_tensor_t *input, marmot_tensor_t *output) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || input == nullptr || output == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Dequantize: null argument");
    }
    if (!kind_supported_weight(input->quant_kind) && input->quant_kind != MARMOT_QUANT_KIND_Q8_K) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP dequantize handles Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 and Q2_K to Q8_K");
    }
    if (output->dtype != MARMOT_DTYPE_FLOAT32) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Dequantize output must be FLOAT32");
    }
    if (!rows_contiguous(output)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Dequantize expects a contiguous 2D output");
    }
    const size_t rows = output->shape.shape[0], k = output->shape.shape[1];
    if (input->shape.ndim == 2 && (input->shape.shape[0] != rows || input->shape.shape[1] != k)) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Dequantize shape mismatch");
    }
    if (rows == 0 || k == 0) {
        return MARMOT_SUCCESS;
    }
    pthread_mutex_lock(&b->mu);
    const marmot_error_t st = dequantize_locked(b, input, output, rows, k);
    pthread_mutex_unlock(&b->mu);
    return st;
}

// ------------------------------------------------------------------ bytecode exec entries
// ------------------------------------------------------------------ ops between the linears
// marmot_norm_validate (src/core/helpers/norm.c) for RMS normalization: x and out of one shape and dtype, residual
// like x, weight a vector of the last dimension; FLOAT32 only here.
static marmot_error_t rmsnorm(const void *device_ctx, const marmot_rmsnorm_desc_t *desc, float weight_offset) {
    hip_backend_t *b = backend_of(device_ctx);
    if (desc == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RMSNorm descriptor is null");
    }
    const marmot_tensor_t *x = desc->x, *res = desc->residual, *w = desc->weight;
    marmot_tensor_t *out = desc->out;
    if (b == nullptr || x == nullptr || out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RMSNorm requires input and output tensors");
    }
    if (x->shape.ndim == 0 || x->shape.ndim != out->shape.ndim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RMSNorm input/output rank mismatch");
    }
    for (size_t i = 0; i < x->shape.ndim; ++i) {
        if (x->shape.shape[i] != out->shape.shape[i] || (res != nullptr && (res->shape.ndim != x->shape.ndim ||
                                                                           res->shape.shape[i] != x->shape.shape[i]))) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RMSNorm tensor shapes do not match");
        }
    }
    const size_t cols = x->shape.shape[x->shape.ndim - 1];
    if (w != nullptr && tensor_numel(w) != cols) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RMSNorm weight length does not match the normalized dimension");
    }
    if (x->dtype != MARMOT_DTYPE_FLOAT32 || out->dtype != MARMOT_DTYPE_FLOAT32 ||
        (res != nullptr && res->dtype != MARMOT_DTYPE_FLOAT32) || (w != nullptr && w->dtype != MARMOT_DTYPE_FLOAT32)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP RMSNorm handles FLOAT32 tensors");
    }
    if (!dense_contiguous(x) || !dense_contiguous(out) || (res != nullptr && !dense_contiguous(res)) ||
        (w != nullptr && !dense_contiguous(w))) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP RMSNorm needs contiguous tensors");
    }
    const size_t n = tensor_numel(x);
    if (n == 0 || cols == 0) {
        mark_device_output(out);
        return MARMOT_SUCCESS;
    }
    if (x->data == nullptr || out->data == nullptr || (res != nullptr && res->data == nullptr) ||
        (w != nullptr && w->data == nullptr)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RMSNorm: tensor without data");
    }
    const size_t rows = n / cols;
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[4];
    size_t n_acq = 0;
    int res_at = -1, w_at = -1;
    acq[n_acq++] = (hip_acq_t){x->data, n * sizeof(float), HIP_ACQ_READ, nullptr};
    acq[n_acq++] = (hip_acq_t){out->data, n * sizeof(float), HIP_ACQ_WRITE, nullptr};  // also ends any packed copy of the old contents
    if (res != nullptr) {
        res_at = (int)n_acq;
        acq[n_acq++] = (hip_acq_t){res->data, n * sizeof(float), HIP_ACQ_READ, nullptr};
    }
    if (w != nullptr) {
        w_at = (int)n_acq;
        acq[n_acq++] = (hip_acq_t){w->data, cols * sizeof(float), HIP_ACQ_READ, nullptr};
    }
    marmot_error_t st = acquire_set(b, acq, n_acq);
    const void *d_x = acq[0].dev, *d_r = res_at >= 0 ? acq[res_at].dev : nullptr, *d_w = w_at >= 0 ? acq[w_at].dev : nullptr;
    void *d_y = acq[1].dev;
    if (st == MARMOT_SUCCESS) {
        int rc;
        // Rows that the linears behind this normalization would quantize in a launch of their own are packed here,
        // in the same launch: Q8_K when the rows are whole 256-value blocks (K-quant weights), else Q8_0.
        hip_pack_entry_t *e = nullptr;
        const int for_kind = cols % 256 == 0 ? MARMOT_HIP_KIND_Q4_K : MARMOT_HIP_KIND_Q8_0;
        if (rows >= HIP_PACK_MIN_ROWS && cols % 32 == 0 && packs_reserve(b, for_kind, rows, cols, &e) == MARMOT_SUCCESS) {
            rc = marmot_hip_rms_norm_pack(b->dev, (const float *)d_x, (const float *)d_r, (const float *)d_w,
                                          weight_offset, desc->eps, rows, cols, for_kind, (float *)d_y, e->packed);
            if (rc == MARMOT_HIP_SUCCESS) {
                e->valid = true;
                e->host = (uintptr_t)out->data;
                e->rows = rows;
                e->cols = cols;
                e->act_kind = act_kind_of_weight(for_kind);
                e->stamp = ++b->pack_clock;
                b->packs_made++;
            }
        } else {
            rc = marmot_hip_rms_norm(b->dev, (const float *)d_x, (const float *)d_r, (const float *)d_w, weight_offset,
                                     desc->eps, rows, cols, (float *)d_y);
        }
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    return st;
}

// swiglu / geglu / add on FLOAT32 tensors of one shape: contiguous, or 2-D with unit column stride (row-strided, the
// halves of a fused gate/up projection: cpu_row_strided_2d, elementwise_f32_scalar.c:22-45)
typedef enum { HIP_BIN_SWIGLU, HIP_BIN_GEGLU, HIP_BIN_ADD } hip_binary_op_t;

static bool row_strided_2d(const marmot_tensor_t *t) {
    return t->shape.ndim == 2 && t->shape.strides[1] == 1 && t->shape.strides[0] >= t->shape.shape[1];
}

static size_t strided_span_bytes(const marmot_tensor_t *t) {
    if (t->shape.ndim == 2 && !dense_contiguous(t)) {
        return ((t->shape.shape[0] - 1) * t->shape.strides[0] + t->shape.shape[1]) * sizeof(float);
    }
    return dense_bytes(t);
}

static marmot_error_t binary_f32(const void *device_ctx, hip_binary_op_t op, const marmot_tensor_t *a,
                                 const marmot_tensor_t *c, marmot_tensor_t *out) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || a == nullptr || c == nullptr || out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Binary operation: null tensor");
    }
    if (a->shape.ndim != c->shape.ndim || a->shape.ndim != out->shape.ndim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Binary operation: rank mismatch");
    }
    for (size_t i = 0; i < a->shape.ndim; ++i) {
        if (a->shape.shape[i] != c->shape.shape[i] || a->shape.shape[i] != out->shape.shape[i]) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Binary operation: shapes do not match");
        }
    }
    if (a->dtype != MARMOT_DTYPE_FLOAT32 || c->dtype != MARMOT_DTYPE_FLOAT32 || out->dtype != MARMOT_DTYPE_FLOAT32) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP elementwise operations handle FLOAT32 tensors");
    }
    const bool dense = dense_contiguous(a) && dense_contiguous(c) && dense_contiguous(out);
    const bool strided = row_strided_2d(a) && row_strided_2d(c) && row_strided_2d(out);
    if (!dense && !(strided && op != HIP_BIN_ADD)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP elementwise operations need contiguous or row-strided tensors");
    }
    const size_t n = tensor_numel(a);
    if (n == 0) {
        mark_device_output(out);
        return MARMOT_SUCCESS;
    }
    if (a->data == nullptr || c->data == nullptr || out->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Binary operation: tensor without data");
    }
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[3] = {
        {a->data, strided_span_bytes(a), HIP_ACQ_READ, nullptr},
        {c->data, strided_span_bytes(c), HIP_ACQ_READ, nullptr},
        {out->data, strided_span_bytes(out), dense_contiguous(out) ? HIP_ACQ_WRITE : HIP_ACQ_UPDATE, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, 3);
    const void *d_a = acq[0].dev, *d_c = acq[1].dev;
    void *d_y = acq[2].dev;
    if (st == MARMOT_SUCCESS) {
        int rc;
        if (op == HIP_BIN_ADD) {
            rc = marmot_hip_add(b->dev, (const float *)d_a, (const float *)d_c, n, (float *)d_y);
        } else {
            size_t rows = 1, cols = n, sa = n, sc = n, so = n;
            if (!dense) {
                rows = a->shape.shape[0];
                cols = a->shape.shape[1];
                sa = a->shape.strides[0];
                sc = c->shape.strides[0];
                so = out->shape.strides[0];
            }
            rc = marmot_hip_glu(b->dev, op == HIP_BIN_GEGLU ? MARMOT_HIP_FFN_GEGLU : MARMOT_HIP_FFN_SWIGLU,
                                (const float *)d_a, (const float *)d_c, rows, cols, sa, sc, so, (float *)d_y);
        }
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    return st;
}

// marmot_rope (cpu_rope and cpu_rope_validate, src/backends/cpu/ops/rope/rope_dispatch.c:18-88, 145-196): the last
// dimension of x is rotated, one position per row of it; checks in the reference's order. FLOAT32 and FLOAT16 rows.
// The dimensions before the last must lie at one stride from row to row (contiguous tensors, and 2-D views whose
// rows are further apart than their length), which is what the kernel walks.
static bool rows_at_one_stride(const marmot_tensor_t *t, size_t *row_stride_out) {
    const size_t nd = t->shape.ndim;
    const size_t row_stride = t->shape.strides[nd - 2];
    for (size_t i = nd - 2; i > 0; --i) {
        if (t->shape.shape[i - 1] != 1 && t->shape.strides[i - 1] != t->shape.strides[i] * t->shape.shape[i]) {
            return false;
        }
    }
    *row_stride_out = row_stride;
    return true;
}

static marmot_error_t rope(const void *device_ctx, const marmot_tensor_t *x, const marmot_rope_params_t *params,
                           marmot_tensor_t *out) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RoPE: null device context");
    }
    if (params == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RoPE parameters are null");
    }
    const marmot_tensor_t *positions = params->positions;
    if (positions == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RoPE parameters require positions tensor");
    }
    if (x == nullptr || out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null pointer in RoPE");
    }
    const marmot_dtype_t dtype = x->dtype;
    const bool reference_dtype = dtype == MARMOT_DTYPE_FLOAT32 || dtype == MARMOT_DTYPE_FLOAT64 ||
        dtype == MARMOT_DTYPE_FLOAT16 || dtype == MARMOT_DTYPE_BFLOAT16;
    if (!reference_dtype || out->dtype != dtype) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "RoPE dtype not supported");
    }
    if (x->shape.ndim < 2) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RoPE requires at least 2D tensor");
    }
    const size_t ndim = x->shape.ndim;
    const size_t dim = x->shape.shape[ndim - 1];
    if (dim % 2 != 0) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RoPE requires even dimension");
    }
    const size_t total = tensor_numel(x);
    if (x->shape.shape[ndim - 2] == 0 || dim == 0 || total == 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RoPE input tensor must be non-empty");
    }
    const size_t rows = total / dim;
    if (tensor_numel(positions) != rows) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RoPE positions shape mismatch");
    }
    if (out->shape.ndim != ndim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RoPE output shape mismatch");
    }
    for (size_t i = 0; i < ndim; ++i) {
        if (out->shape.shape[i] != x->shape.shape[i]) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RoPE output shape mismatch");
        }
    }
    if (positions->dtype != MARMOT_DTYPE_FLOAT32 && positions->dtype != MARMOT_DTYPE_INT32 &&
        positions->dtype != MARMOT_DTYPE_INT64) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "RoPE positions tensor must be FLOAT32, INT32, or INT64");
    }
    if (x->shape.strides[ndim - 1] != 1 || out->shape.strides[ndim - 1] != 1) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "RoPE requires contiguous inner dimension");
    }
    if (x->shape.strides[ndim - 2] < dim || out->shape.strides[ndim - 2] < dim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "RoPE requires row strides >= feature dimension");
    }
    if (dtype != MARMOT_DTYPE_FLOAT32 && dtype != MARMOT_DTYPE_FLOAT16) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP RoPE handles FLOAT32 and FLOAT16 tensors");
    }
    if (params->rope_type != MARMOT_ROPE_TYPE_NORM && params->rope_type != MARMOT_ROPE_TYPE_NEOX) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RoPE: unknown rope type");
    }
    size_t x_stride = 0, out_stride = 0;
    if (!rows_at_one_stride(x, &x_stride) || !rows_at_one_stride(out, &out_stride) || !dense_contiguous(positions)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP RoPE needs rows at one stride and contiguous positions");
    }
    if (x->data == nullptr || out->data == nullptr || positions->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "RoPE: tensor without data");
    }
    const size_t elt = dtype_size(dtype);
    const size_t x_span = ((rows - 1) * x_stride + dim) * elt, out_span = ((rows - 1) * out_stride + dim) * elt;
    marmot_rope_params_t keyed = *params;  // the frequencies are those of the rotated dimension (rope.c:143-200)
    keyed.head_dim = (uint32_t)dim;
    pthread_mutex_lock(&b->mu);
    hip_rope_entry_t *e = nullptr;
    marmot_error_t st = rope_entry_locked(b, &keyed, dim, &e);
    const void *d_x = nullptr, *d_pos = nullptr, *d_freqs = nullptr;
    void *d_y = nullptr;
    if (st == MARMOT_SUCCESS) {
        hip_acq_t acq[4] = {
            {x->data, x_span, HIP_ACQ_READ, nullptr},
            {positions->data, dense_bytes(positions), HIP_ACQ_READ, nullptr},
            {e->freqs, dim / 2 * sizeof(float), HIP_ACQ_READ, nullptr},
            {out->data, out_span, out_stride != dim ? HIP_ACQ_UPDATE : HIP_ACQ_WRITE, nullptr},
        };
        st = acquire_set(b, acq, 4);
        d_x = acq[0].dev, d_pos = acq[1].dev, d_freqs = acq[2].dev, d_y = acq[3].dev;
    }
    if (st == MARMOT_SUCCESS) {
        const marmot_hip_rope_t r = {
            .d_positions = d_pos,
            .positions_dtype = positions->dtype == MARMOT_DTYPE_FLOAT32 ? MARMOT_HIP_DTYPE_F32
                : positions->dtype == MARMOT_DTYPE_INT32               ? MARMOT_HIP_DTYPE_I32
                                                                       : MARMOT_HIP_DTYPE_I64,
            .d_freqs = d_freqs,
            .attn_scale = e->attn_scale,
            .head_dim = e->head_dim,
            .rope_type = params->rope_type == MARMOT_ROPE_TYPE_NEOX ? 1 : 0,
        };
        const int rc = marmot_hip_rope(b->dev, d_x, dtype == MARMOT_DTYPE_FLOAT16 ? MARMOT_HIP_DTYPE_F16
                                                                                   : MARMOT_HIP_DTYPE_F32,
                                       rows, dim, x_stride, out_stride, &r, d_y);
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    return st;
}

// ------------------------------------------------------------------ paged attention
static bool pa_float_dtype(marmot_dtype_t t) {
    return t == MARMOT_DTYPE_FLOAT32 || t == MARMOT_DTYPE_FLOAT16 || t == MARMOT_DTYPE_BFLOAT16;
}

static int pa_lib_dtype(marmot_dtype_t t) {
    return t == MARMOT_DTYPE_FLOAT16     ? MARMOT_HIP_DTYPE_F16
        : t == MARMOT_DTYPE_BFLOAT16     ? MARMOT_HIP_DTYPE_BF16
        : t == MARMOT_DTYPE_FLOAT8_E4M3 ? MARMOT_HIP_DTYPE_F8_E4M3
                                         : MARMOT_HIP_DTYPE_F32;
}

// bytes from the first to one past the last element of a tensor of any rank and strides
static size_t strided_extent_bytes(const marmot_tensor_t *t) {
    size_t last = 0;
    for (size_t i = 0; i < t->shape.ndim; ++i) {
        if (t->shape.shape[i] == 0) {
            return 0;
        }
        last += (t->shape.shape[i] - 1) * t->shape.strides[i];
    }
    return (last + 1) * dtype_size(t->dtype);
}

// marmot_paged_attention: the checks of cpu_paged_attention_impl (paged_attention_ref.c:573-823) in its order, then
// the library call on the mirrors. The token metadata is a host tensor here, so its ranges are checked on the host.
static marmot_error_t paged_attention(const void *device_ctx, const marmot_paged_attention_desc_t *desc) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention: null device context");
    }
    if (desc == nullptr || desc->struct_version != MARMOT_PAGED_ATTENTION_DESC_VERSION ||
        desc->struct_size < sizeof(marmot_paged_attention_desc_t) || desc->token_meta == nullptr || desc->q == nullptr ||
        desc->k_new == nullptr || desc->v_new == nullptr || desc->kv_k == nullptr || desc->kv_v == nullptr ||
        desc->block_table == nullptr || desc->out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention descriptor invalid");
    }
    if (desc->token_count == 0) {
        return MARMOT_SUCCESS;
    }
    if (desc->num_q_heads == 0 || desc->num_kv_heads == 0 || desc->head_dim == 0 || desc->block_size == 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention requires non-zero dimensions");
    }
    if ((desc->block_size & (desc->block_size - 1u)) != 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention block_size must be power of two");
    }
    if (desc->num_q_heads % desc->num_kv_heads != 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention requires num_q_heads divisible by num_kv_heads");
    }
    const marmot_tensor_t *meta = desc->token_meta, *q = desc->q, *k_new = desc->k_new, *v_new = desc->v_new;
    const marmot_tensor_t *kv_k = desc->kv_k, *kv_v = desc->kv_v, *table = desc->block_table;
    marmot_tensor_t *out = desc->out;
    const marmot_paged_attention_kv_scale_ext_t *ext = (const marmot_paged_attention_kv_scale_ext_t *)desc->pnext;
    const bool has_scales = ext != nullptr && ext->struct_version == MARMOT_PAGED_ATTENTION_KV_SCALE_EXT_VERSION &&
        ext->struct_size >= sizeof(*ext) && (ext->kv_k_scale != nullptr || ext->kv_v_scale != nullptr);
    if (meta->dtype != MARMOT_DTYPE_UINT32 || table->dtype != MARMOT_DTYPE_UINT32) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "paged_attention requires uint32 metadata");
    }
    const bool kv_fp8 = kv_k->dtype == MARMOT_DTYPE_FLOAT8_E4M3 && kv_v->dtype == MARMOT_DTYPE_FLOAT8_E4M3;
    if (!pa_float_dtype(q->dtype) || !pa_float_dtype(k_new->dtype) || !pa_float_dtype(v_new->dtype) ||
        !pa_float_dtype(out->dtype) || (!kv_fp8 && (!pa_float_dtype(kv_k->dtype) || !pa_float_dtype(kv_v->dtype)))) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "paged_attention dtype not supported");
    }
    if (q->dtype != k_new->dtype || q->dtype != v_new->dtype || q->dtype != out->dtype) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "paged_attention requires matching q/k_new/v_new/out dtypes");
    }
    if (meta->shape.ndim != 2 || meta->shape.shape[1] != 4 || meta->shape.shape[0] != desc->token_count) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention token_meta shape invalid");
    }
    if (table->shape.ndim != 2) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention block_table must be 2D");
    }
    if (q->shape.ndim != 3 || k_new->shape.ndim != 3 || v_new->shape.ndim != 3 || out->shape.ndim != 3) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention expects 3D q/k_new/v_new/out tensors");
    }
    if (q->shape.shape[0] < desc->token_count || k_new->shape.shape[0] < desc->token_count ||
        v_new->shape.shape[0] < desc->token_count || out->shape.shape[0] < desc->token_count) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention token_count exceeds tensor rows");
    }
    if (q->shape.shape[1] != desc->num_q_heads || out->shape.shape[1] != desc->num_q_heads) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention num_q_heads mismatch");
    }
    if (k_new->shape.shape[1] != desc->num_kv_heads || v_new->shape.shape[1] != desc->num_kv_heads) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention num_kv_heads mismatch");
    }
    if (q->shape.shape[2] != desc->head_dim || k_new->shape.shape[2] != desc->head_dim ||
        v_new->shape.shape[2] != desc->head_dim || out->shape.shape[2] != desc->head_dim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention head_dim mismatch");
    }
    if (kv_k->shape.ndim != 5 || kv_v->shape.ndim != 5) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention kv cache must be 5D");
    }
    if (kv_k->shape.shape[1] <= desc->layer_idx) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention layer_idx out of range");
    }
    if (kv_k->shape.shape[2] != desc->num_kv_heads || kv_v->shape.shape[2] != desc->num_kv_heads) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention kv head mismatch");
    }
    if (kv_k->shape.shape[3] != desc->block_size || kv_v->shape.shape[3] != desc->block_size) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention block_size mismatch");
    }
    if (kv_k->shape.shape[4] != desc->head_dim || kv_v->shape.shape[4] != desc->head_dim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention kv head_dim mismatch");
    }
    if (kv_k->dtype != kv_v->dtype) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention kv dtype mismatch");
    }
    const marmot_tensor_t *k_scale = has_scales ? ext->kv_k_scale : nullptr, *v_scale = has_scales ? ext->kv_v_scale : nullptr;
    if (kv_fp8) {  // paged_attention_ref.c:694-722
        if (k_scale == nullptr || v_scale == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention FP8 KV requires scale tensors");
        }
        if (k_scale->dtype != MARMOT_DTYPE_FLOAT32 || v_scale->dtype != MARMOT_DTYPE_FLOAT32) {
            return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "paged_attention FP8 scale dtype must be float32");
        }
        if (k_scale->shape.ndim != 3 || v_scale->shape.ndim != 3) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention FP8 scale tensors must be 3D");
        }
        for (size_t i = 0; i < 3; ++i) {
            if (k_scale->shape.shape[i] != kv_k->shape.shape[i] || v_scale->shape.shape[i] != kv_v->shape.shape[i]) {
                return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention FP8 scale tensor shape mismatch");
            }
        }
        if (k_scale->data == nullptr || v_scale->data == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention FP8 scale tensors missing data");
        }
    } else if (has_scales) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention scale tensors require FP8 KV");
    }
    if (meta->data == nullptr || table->data == nullptr || q->data == nullptr || k_new->data == nullptr ||
        v_new->data == nullptr || kv_k->data == nullptr || kv_v->data == nullptr || out->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "paged_attention requires non-null tensor data");
    }
    uint32_t shift = 0;
    while ((1u << shift) < desc->block_size) {
        ++shift;
    }
    const uint32_t *meta_host = (const uint32_t *)meta->data;
    for (size_t t = 0; t < desc->token_count; ++t) {
        const uint32_t seq_slot = meta_host[t * meta->shape.strides[0]];
        const uint32_t kv_slot = meta_host[t * meta->shape.strides[0] + 2 * meta->shape.strides[1]];
        if (seq_slot >= table->shape.shape[0]) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention seq_slot out of range");
        }
        if ((kv_slot >> shift) >= kv_k->shape.shape[0]) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "paged_attention kv_slot block out of range");
        }
    }
    if (desc->head_dim > 256) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP paged_attention handles head dimensions up to 256");
    }
    for (size_t i = 0; i < 5; ++i) {
        if (kv_k->shape.strides[i] != kv_v->shape.strides[i]) {
            return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP paged_attention needs key and value caches of one layout");
        }
    }
    for (size_t i = 0; kv_fp8 && i < 3; ++i) {
        if (k_scale->shape.strides[i] != v_scale->shape.strides[i]) {
            return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP paged_attention needs key and value scales of one layout");
        }
    }
    marmot_hip_paged_attention_t a = {
        .token_count = desc->token_count, .layer_idx = desc->layer_idx, .num_q_heads = desc->num_q_heads,
        .num_kv_heads = desc->num_kv_heads, .head_dim = desc->head_dim, .block_size = desc->block_size,
        .scale = desc->scale, .act_dtype = pa_lib_dtype(q->dtype), .kv_dtype = pa_lib_dtype(kv_k->dtype),
        .kv_blocks = kv_k->shape.shape[0], .kv_layers = kv_k->shape.shape[1],
        .max_seqs = table->shape.shape[0], .max_blocks_per_seq = table->shape.shape[1],
    };
    for (size_t i = 0; i < 2; ++i) {
        a.meta_stride[i] = meta->shape.strides[i];
        a.table_stride[i] = table->shape.strides[i];
    }
    for (size_t i = 0; i < 3; ++i) {
        a.q_stride[i] = q->shape.strides[i];
        a.k_stride[i] = k_new->shape.strides[i];
        a.v_stride[i] = v_new->shape.strides[i];
        a.out_stride[i] = out->shape.strides[i];
    }
    for (size_t i = 0; i < 5; ++i) {
        a.kv_stride[i] = kv_k->shape.strides[i];
    }
    for (size_t i = 0; kv_fp8 && i < 3; ++i) {
        a.scale_stride[i] = k_scale->shape.strides[i];
    }
    pthread_mutex_lock(&b->mu);
    // the caches are read and written; an output that is a view with gaps, or has more rows than tokens, keeps its
    // other bytes: the host's bytes go up first
    hip_acq_t acq[10] = {
        {meta->data, strided_extent_bytes(meta), HIP_ACQ_READ, nullptr},
        {table->data, strided_extent_bytes(table), HIP_ACQ_READ, nullptr},
        {q->data, strided_extent_bytes(q), HIP_ACQ_READ, nullptr},
        {k_new->data, strided_extent_bytes(k_new), HIP_ACQ_READ, nullptr},
        {v_new->data, strided_extent_bytes(v_new), HIP_ACQ_READ, nullptr},
        {kv_k->data, strided_extent_bytes(kv_k), HIP_ACQ_UPDATE, nullptr},
        {kv_v->data, strided_extent_bytes(kv_v), HIP_ACQ_UPDATE, nullptr},
        {out->data, strided_extent_bytes(out),
         dense_contiguous(out) && out->shape.shape[0] == desc->token_count ? HIP_ACQ_WRITE : HIP_ACQ_UPDATE, nullptr},
    };
    if (kv_fp8) {
        acq[8] = (hip_acq_t){k_scale->data, strided_extent_bytes(k_scale), HIP_ACQ_UPDATE, nullptr};
        acq[9] = (hip_acq_t){v_scale->data, strided_extent_bytes(v_scale), HIP_ACQ_UPDATE, nullptr};
    }
    marmot_error_t st = acquire_set(b, acq, kv_fp8 ? 10 : 8);
    const void *d_meta = acq[0].dev, *d_table = acq[1].dev, *d_q = acq[2].dev, *d_k = acq[3].dev, *d_v = acq[4].dev;
    void *d_kv_k = acq[5].dev, *d_kv_v = acq[6].dev, *d_out = acq[7].dev;
    if (st == MARMOT_SUCCESS) {
        a.d_token_meta = (const uint32_t *)d_meta, a.d_block_table = (const uint32_t *)d_table;
        a.d_q = d_q, a.d_k_new = d_k, a.d_v_new = d_v, a.d_kv_k = d_kv_k, a.d_kv_v = d_kv_v, a.d_out = d_out;
        if (kv_fp8) {
            a.d_kv_k_scale = (float *)acq[8].dev, a.d_kv_v_scale = (float *)acq[9].dev;
        }
        const int rc = marmot_hip_paged_attention(b->dev, &a, 0);
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
        mark_device_output((marmot_tensor_t *)kv_k);
        mark_device_output((marmot_tensor_t *)kv_v);
        if (kv_fp8) {
            mark_device_output((marmot_tensor_t *)k_scale);
            mark_device_output((marmot_tensor_t *)v_scale);
        }
    }
    return st;
}

// ------------------------------------------------------------------ the remaining nodes of a model graph
// bytes a tensor occupies (marmot_tensor_size_bytes, src/core/tensor/metadata.c:74-146): block-quantized tensors of
// two or more dimensions by rows of blocks (for ranks other than two the first dimension is the row length)
static size_t tensor_storage_bytes(const marmot_tensor_t *t) {
    const size_t n = tensor_numel(t);
    if (n == 0) {
        return 0;
    }
    if (kind_is_block(t->quant_kind) && t->quant_layout == MARMOT_QUANT_LAYOUT_GGUF && t->shape.ndim >= 2) {
        size_t rows, inner;
        if (t->shape.ndim == 2) {
            rows = t->shape.shape[0];
            inner = t->shape.shape[1];
        } else {
            inner = t->shape.shape[0];
            rows = n / inner;
        }
        return rows * marmot_hip_row_bytes((int)t->quant_kind, inner);
    }
    if (t->dtype == MARMOT_DTYPE_INT4 || t->dtype == MARMOT_DTYPE_UINT4) {
        return (n + 1) / 2;
    }
    return n * dtype_size(t->dtype);
}

static bool same_shape(const marmot_tensor_t *a, const marmot_tensor_t *c) {
    if (a->shape.ndim != c->shape.ndim) {
        return false;
    }
    for (size_t i = 0; i < a->shape.ndim; ++i) {
        if (a->shape.shape[i] != c->shape.shape[i]) {
            return false;
        }
    }
    return true;
}

static void ops_on_host_ptr_freed(void *device_ctx, const void *ptr);

// the output takes over the input's storage: what the alias-making operations share (tensor_ops.c:74-89, 138-155)
static void alias_storage(const marmot_tensor_t *x, marmot_tensor_t *out, size_t byte_offset) {
    out->data = (uint8_t *)x->data + byte_offset;
    out->capacity_bytes = x->capacity_bytes > byte_offset ? x->capacity_bytes - byte_offset : 0;
    out->owns_data = false;
    out->quant_params = x->quant_params;
    out->quant_kind = x->quant_kind;
    out->quant_layout = x->quant_layout;
    out->backend = x->backend;
    out->memory_location = x->memory_location;
    out->needs_sync = x->needs_sync;
    out->packed_data = nullptr;
    out->packed_src_data = nullptr;
    out->packed_bytes = 0;
    out->packed_row_bytes = 0;
    out->packed_rows = 0;
}

// marmot_reshape (cpu_reshape, src/backends/cpu/ops/tensor_ops/tensor_ops.c:29-91): metadata only. The output aliases
// the input's host bytes; the residency table resolves both to one mirror, so nothing moves on the device either.
static marmot_error_t reshape(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out,
                              const size_t *new_shape, size_t new_ndim) {
    if (x == nullptr || out == nullptr || new_shape == nullptr || new_ndim == 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null pointer in reshape");
    }
    if (new_ndim > MARMOT_MAX_DIMS) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Reshape rank exceeds the tensor rank limit");
    }
    size_t new_elements = 1;
    for (size_t i = 0; i < new_ndim; ++i) {
        new_elements *= new_shape[i];
    }
    if (tensor_numel(x) != new_elements) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Reshape element count mismatch");
    }
    if (out->owns_data && out->data != nullptr && out->data != x->data) {
        ops_on_host_ptr_freed((void *)device_ctx, out->data);
        free(out->data);
    }
    out->shape.ndim = new_ndim;
    for (size_t i = 0; i < new_ndim; ++i) {
        out->shape.shape[i] = new_shape[i];
    }
    bool has_stride = false;
    for (size_t i = 0; i < new_ndim; ++i) {
        if (out->shape.strides[i] != 0) {
            has_stride = true;
            break;
        }
    }
    if (!has_stride) {
        out->shape.strides[new_ndim - 1] = 1;
        for (size_t i = new_ndim - 1; i-- > 0;) {
            out->shape.strides[i] = out->shape.strides[i + 1] * out->shape.shape[i + 1];
        }
    }
    out->dtype = x->dtype;
    alias_storage(x, out, 0);
    out->capacity_bytes = x->capacity_bytes;
    return MARMOT_SUCCESS;
}

// marmot_view (cpu_view, tensor_ops.c:93-158): metadata only, checks in the reference's order
static marmot_error_t view(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out, size_t byte_offset) {
    if (x == nullptr || out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null pointer in view");
    }
    if (x->dtype != out->dtype) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "View requires matching dtypes");
    }
    if (x->backend != out->backend) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "View requires matching backends");
    }
    const size_t elem_size = dtype_size(x->dtype);
    if (elem_size != 0 && (byte_offset % elem_size) != 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "View byte offset must align to dtype size");
    }
    marmot_tensor_t probe = *out;
    probe.quant_kind = x->quant_kind;
    probe.quant_layout = x->quant_layout;
    const size_t out_bytes = tensor_storage_bytes(&probe);
    if (x->capacity_bytes < byte_offset) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "View byte offset exceeds input capacity");
    }
    if (out_bytes > x->capacity_bytes - byte_offset) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "View exceeds input capacity");
    }
    if (out_bytes != 0 && x->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "View requires non-null input data");
    }
    if (out->owns_data && out->data != nullptr) {
        ops_on_host_ptr_freed((void *)device_ctx, out->data);
        free(out->data);
    }
    if (out->packed_data != nullptr) {
        free(out->packed_data);
    }
    if (out->quant_params != nullptr && out->quant_params != x->quant_params) {
        free(out->quant_params);
    }
    alias_storage(x, out, byte_offset);
    return MARMOT_SUCCESS;
}

// marmot_slice (cpu_slice, tensor_ops.c:401-462): the box [starts, starts + sizes) of a contiguous tensor. The
// reference walks the shapes, not the strides, and does not check the box; here a box outside the input and an output
// whose shape is not `sizes` are errors.
static marmot_error_t slice(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out,
                            const size_t *starts, const size_t *sizes) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || x == nullptr || out == nullptr || starts == nullptr || sizes == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null pointer in slice");
    }
    const size_t ndim = x->shape.ndim;
    if (ndim == 0) {
        return MARMOT_SUCCESS;
    }
    if (ndim > 8 || out->shape.ndim != ndim) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Slice input and output ranks must match (at most 8)");
    }
    if (x->dtype != out->dtype) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Slice requires matching input/output dtypes");
    }
    const size_t elem_size = dtype_size(x->dtype);
    if (elem_size == 0 || kind_is_block(x->quant_kind)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP slice handles dense element types");
    }
    for (size_t d = 0; d < ndim; ++d) {
        if (out->shape.shape[d] != sizes[d]) {
            return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Slice output shape must equal the slice sizes");
        }
        if (starts[d] > x->shape.shape[d] || sizes[d] > x->shape.shape[d] - starts[d]) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Slice box lies outside the input");
        }
    }
    if (!dense_contiguous(x) || !dense_contiguous(out)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP slice needs contiguous tensors");
    }
    if (tensor_numel(out) == 0) {
        mark_device_output(out);
        return MARMOT_SUCCESS;
    }
    if (x->data == nullptr || out->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Slice: tensor without data");
    }
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[2] = {
        {x->data, dense_bytes(x), HIP_ACQ_READ, nullptr},
        {out->data, dense_bytes(out), HIP_ACQ_WRITE, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, 2);
    if (st == MARMOT_SUCCESS) {
        const int rc = marmot_hip_slice(b->dev, acq[0].dev, elem_size, (int)ndim, x->shape.shape, starts, sizes, acq[1].dev);
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    return st;
}

// marmot_gather_rows (cpu_gather_rows, tensor_ops.c:464-547): checks in the reference's order; rows with unit column
// stride (the reference also walks column strides)
static marmot_error_t gather_rows(const void *device_ctx, const marmot_tensor_t *input, const marmot_tensor_t *indices,
                                  marmot_tensor_t *out) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || input == nullptr || indices == nullptr || out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null pointer in gather_rows");
    }
    if (input->shape.ndim != 2 || out->shape.ndim != 2) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "gather_rows expects 2D input/output tensors");
    }
    if (indices->shape.ndim != 1) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "gather_rows indices must be 1D");
    }
    if (input->dtype != out->dtype) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "gather_rows requires matching input/output dtypes");
    }
    const size_t rows_in = input->shape.shape[0], cols = input->shape.shape[1], rows_out = out->shape.shape[0];
    if (rows_out != indices->shape.shape[0] || cols != out->shape.shape[1]) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "gather_rows output shape mismatch");
    }
    if (rows_out == 0 || cols == 0) {
        return MARMOT_SUCCESS;
    }
    const size_t elem_size = dtype_size(input->dtype);
    if (elem_size == 0) {
        return MARMOT_SUCCESS;
    }
    if (input->data == nullptr || out->data == nullptr || indices->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "gather_rows requires non-null tensor data");
    }
    if (indices->dtype != MARMOT_DTYPE_INT32 && indices->dtype != MARMOT_DTYPE_UINT32) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "gather_rows indices dtype unsupported");
    }
    if (kind_is_block(input->quant_kind)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP gather_rows handles dense element types");
    }
    const size_t in_s0 = input->shape.strides[0], out_s0 = out->shape.strides[0], idx_s0 = indices->shape.strides[0];
    if ((cols != 1 && (input->shape.strides[1] != 1 || out->shape.strides[1] != 1)) || (rows_in > 1 && in_s0 < cols) ||
        (rows_out > 1 && out_s0 < cols)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP gather_rows needs rows with unit column stride");
    }
    if (rows_in == 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "gather_rows index out of range");
    }
    const size_t row_bytes = cols * elem_size;
    const size_t in_span = ((rows_in - 1) * in_s0 + cols) * elem_size;
    const size_t out_span = ((rows_out - 1) * out_s0 + cols) * elem_size;
    const size_t idx_span = ((rows_out - 1) * idx_s0 + 1) * 4;
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[3] = {
        {input->data, in_span, HIP_ACQ_READ, nullptr},
        {indices->data, idx_span, HIP_ACQ_READ, nullptr},
        {out->data, out_span, out_s0 == cols || rows_out == 1 ? HIP_ACQ_WRITE : HIP_ACQ_UPDATE, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, 3);
    // the library takes at most 65535 rows per call
    for (size_t r0 = 0; st == MARMOT_SUCCESS && r0 < rows_out; r0 += 65535) {
        const size_t n = rows_out - r0 < 65535 ? rows_out - r0 : 65535;
        const int rc = marmot_hip_gather_rows(
            b->dev, acq[0].dev, rows_in, row_bytes, in_s0 * elem_size, (const uint8_t *)acq[1].dev + r0 * idx_s0 * 4,
            indices->dtype == MARMOT_DTYPE_INT32 ? MARMOT_HIP_DTYPE_I32 : MARMOT_HIP_DTYPE_U32, idx_s0, n,
            (uint8_t *)acq[2].dev + r0 * out_s0 * elem_size, out_s0 * elem_size);
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    return st;
}

// marmot_softmax (cpu_softmax_impl, src/backends/cpu/ops/softmax/softmax_dispatch.c:67-103; marmot_softmax_prepare,
// src/core/helpers/norm.c:123-179, checks in its order): FLOAT32, FLOAT16 or BFLOAT16, contiguous, any axis
static marmot_error_t softmax(const void *device_ctx, const marmot_softmax_desc_t *desc) {
    hip_backend_t *b = backend_of(device_ctx);
    if (desc == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Softmax descriptor is null");
    }
    if (desc->x == nullptr || desc->out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Softmax input or output is null");
    }
    if (b == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "HIP context is null for softmax");
    }
    const marmot_tensor_t *x = desc->x;
    marmot_tensor_t *out = desc->out;
    if (x->dtype != out->dtype) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Softmax input and output dtype mismatch");
    }
    if (!same_shape(x, out)) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Softmax input/output shape mismatch");
    }
    if (x->shape.ndim == 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Softmax requires at least 1D tensor");
    }
    int axis = desc->axis;
    if (axis < 0) {
        axis += (int)x->shape.ndim;
    }
    if (axis < 0 || axis >= (int)x->shape.ndim) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Softmax axis out of range");
    }
    const size_t axis_size = x->shape.shape[axis];
    if (axis_size == 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Softmax axis dimension must be non-zero");
    }
    size_t inner = 1;
    for (size_t i = (size_t)axis + 1; i < x->shape.ndim; ++i) {
        inner *= x->shape.shape[i];
    }
    if (axis_size * inner == 0) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Softmax row extent is zero");
    }
    const size_t total = tensor_numel(x);
    const size_t outer = total / (axis_size * inner);
    if (x->dtype != MARMOT_DTYPE_FLOAT32 && x->dtype != MARMOT_DTYPE_FLOAT16 && x->dtype != MARMOT_DTYPE_BFLOAT16) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP softmax handles FLOAT32, FLOAT16 and BFLOAT16 tensors");
    }
    if (!dense_contiguous(x) || !dense_contiguous(out)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP softmax needs contiguous tensors");
    }
    if (total == 0) {
        mark_device_output(out);
        return MARMOT_SUCCESS;
    }
    if (x->data == nullptr || out->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Softmax: tensor without data");
    }
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[2] = {
        {x->data, dense_bytes(x), HIP_ACQ_READ, nullptr},
        {out->data, dense_bytes(out), HIP_ACQ_WRITE, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, 2);
    if (st == MARMOT_SUCCESS) {
        const int rc = marmot_hip_softmax_typed(b->dev, pa_lib_dtype(x->dtype), acq[0].dev, outer, axis_size, inner,
                                                acq[1].dev);
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    return st;
}

// GELU (erf form), GELU (tanh form), SiLU of contiguous FLOAT32 / FLOAT16 tensors (cpu_unary_{gelu,gelu_tanh,silu}_*,
// src/backends/cpu/ops/unary/scalar/unary_scalar.c:201-218, 387-396)
static marmot_error_t unary(const void *device_ctx, int op, const marmot_tensor_t *x,
                            const marmot_activation_params_t *params, marmot_tensor_t *out) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || x == nullptr || out == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Unary operation: null tensor");
    }
    if (params != nullptr && (params->bias != nullptr || params->parameter_tensor != nullptr)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP unary operations take no bias or parameter tensor");
    }
    if (x->dtype != out->dtype) {
        return fail(MARMOT_ERROR_UNSUPPORTED_DTYPE, "Unary operation: input and output dtype mismatch");
    }
    if (!same_shape(x, out)) {
        return fail(MARMOT_ERROR_DIMENSION_MISMATCH, "Unary operation: shapes do not match");
    }
    if (x->dtype != MARMOT_DTYPE_FLOAT32 && x->dtype != MARMOT_DTYPE_FLOAT16) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP unary operations handle FLOAT32 and FLOAT16 tensors");
    }
    if (!dense_contiguous(x) || !dense_contiguous(out)) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP unary operations need contiguous tensors");
    }
    const size_t n = tensor_numel(x);
    if (n == 0) {
        mark_device_output(out);
        return MARMOT_SUCCESS;
    }
    if (x->data == nullptr || out->data == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Unary operation: tensor without data");
    }
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[2] = {
        {x->data, dense_bytes(x), HIP_ACQ_READ, nullptr},
        {out->data, dense_bytes(out), HIP_ACQ_WRITE, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, 2);
    if (st == MARMOT_SUCCESS) {
        const int rc = marmot_hip_unary(b->dev, op, acq[0].dev,
                                        x->dtype == MARMOT_DTYPE_FLOAT32 ? MARMOT_HIP_DTYPE_F32 : MARMOT_HIP_DTYPE_F16, n,
                                        acq[1].dev);
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    pthread_mutex_unlock(&b->mu);
    if (st == MARMOT_SUCCESS) {
        mark_device_output(out);
    }
    return st;
}

// marmot_convert between FLOAT32, FLOAT16 and BFLOAT16 (src/backends/cpu/ops/convert/dtype_convert.c). The operation
// names host addresses, not tensors, so no tensor can be marked "device copy is newer": outside a graph batch the
// destination's host bytes are brought up to date before the call returns; inside a batch (whose values are consumed by
// later nodes on the device) the device copy stays the current one, like any node's output.
static marmot_error_t convert(const void *device_ctx, marmot_dtype_t dst_dtype, void *dst, marmot_dtype_t src_dtype,
                              const void *src, size_t n) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || dst == nullptr || src == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Convert: null argument");
    }
    const bool src_ok = src_dtype == MARMOT_DTYPE_FLOAT32 || src_dtype == MARMOT_DTYPE_FLOAT16 ||
        src_dtype == MARMOT_DTYPE_BFLOAT16;
    const bool dst_ok = dst_dtype == MARMOT_DTYPE_FLOAT32 || dst_dtype == MARMOT_DTYPE_FLOAT16 ||
        dst_dtype == MARMOT_DTYPE_BFLOAT16;
    if (!src_ok || !dst_ok) {
        return fail(MARMOT_ERROR_NOT_IMPLEMENTED, "HIP convert handles FLOAT32, FLOAT16 and BFLOAT16");
    }
    if (n == 0) {
        return MARMOT_SUCCESS;
    }
    const size_t src_bytes = n * dtype_size(src_dtype), dst_bytes = n * dtype_size(dst_dtype);
    pthread_mutex_lock(&b->mu);
    hip_acq_t acq[2] = {
        {(void *)src, src_bytes, HIP_ACQ_READ, nullptr},
        {dst, dst_bytes, HIP_ACQ_WRITE, nullptr},
    };
    marmot_error_t st = acquire_set(b, acq, 2);
    if (st == MARMOT_SUCCESS) {
        // marmot_dtype_t and the library's dtype codes agree for these three types
        const int rc = marmot_hip_convert(b->dev, acq[1].dev, (int)dst_dtype, acq[0].dev, (int)src_dtype, n);
        st = rc == MARMOT_HIP_SUCCESS ? MARMOT_SUCCESS : fail_from_lib(rc);
    }
    if (st == MARMOT_SUCCESS && !b->batching) {
        st = make_host_current_locked(b, dst, dst_bytes);
    }
    pthread_mutex_unlock(&b->mu);
    return st;
}

static uint16_t rd_u16(const uint8_t **pc) {
    const uint16_t v = (uint16_t)((*pc)[0] | ((*pc)[1] << 8));
    *pc += 2;
    return v;
}
static uint32_t rd_u32(const uint8_t **pc) {
    const uint32_t v = (uint32_t)(*pc)[0] | ((uint32_t)(*pc)[1] << 8) | ((uint32_t)(*pc)[2] << 16) |
        ((uint32_t)(*pc)[3] << 24);
    *pc += 4;
    return v;
}
static float rd_f32(const uint8_t **pc) {
    const uint32_t bits = rd_u32(pc);
    float f;
    memcpy(&f, &bits, sizeof(f));
    return f;
}

static marmot_tensor_t *reg(marmot_tensor_t **regs, uint16_t idx) {
    return idx == MARMOT_BC_REG_INVALID ? nullptr : regs[idx];
}

static bool exec_args_ok(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm) {
    const marmot_bc_exec_ctx_t *c = exec_ctx;
    return c != nullptr && c->device_ctx != nullptr && regs != nullptr && imm != nullptr;
}

static marmot_error_t bc_exec_matmul(marmot_quant_kind_t kind, const void *exec_ctx, marmot_tensor_t **regs,
                                     const uint8_t *imm, const uint8_t *const_pool) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const void *device_ctx = ((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx;
    const uint8_t *pc = imm;
    const uint16_t input_idx = rd_u16(&pc);
    const uint16_t weight_idx = rd_u16(&pc);
    const uint16_t bias_idx = rd_u16(&pc);
    const uint32_t epilogue_off = rd_u32(&pc);
    const uint16_t output_idx = rd_u16(&pc);
    marmot_matmul_epilogue_t epilogue;
    const marmot_matmul_epilogue_t *epilogue_ptr = nullptr;
    if (epilogue_off != MARMOT_BC_INVALID_OFFSET) {
        if (const_pool == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null const pool for matmul epilogue");
        }
        memcpy(&epilogue, const_pool + epilogue_off, sizeof(epilogue));
        epilogue_ptr = &epilogue;
    }
    if (bias_idx != MARMOT_BC_REG_INVALID) {
        if (epilogue_ptr == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Missing matmul epilogue");
        }
        epilogue.bias = reg(regs, bias_idx);  // the register wins over the pointer frozen into the pool
    }
    return matmul_quantized(device_ctx, kind, reg(regs, input_idx), reg(regs, weight_idx), epilogue_ptr,
                            reg(regs, output_idx));
}

#define HIP_BC_MATMUL_ENTRY(name, kind)                                                                                \
    static marmot_error_t name(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,                       \
                               const uint8_t *const_pool) {                                                            \
        return bc_exec_matmul(kind, exec_ctx, regs, imm, const_pool);                                                  \
    }
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q4_0, MARMOT_QUANT_KIND_Q4_0)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q8_0, MARMOT_QUANT_KIND_Q8_0)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q4_k, MARMOT_QUANT_KIND_Q4_K)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q6_k, MARMOT_QUANT_KIND_Q6_K)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q5_k, MARMOT_QUANT_KIND_Q5_K)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q4_1, MARMOT_QUANT_KIND_Q4_1)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q5_0, MARMOT_QUANT_KIND_Q5_0)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q5_1, MARMOT_QUANT_KIND_Q5_1)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q2_k, MARMOT_QUANT_KIND_Q2_K)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q3_k, MARMOT_QUANT_KIND_Q3_K)
HIP_BC_MATMUL_ENTRY(bc_exec_matmul_q8_1, MARMOT_QUANT_KIND_Q8_1)

// QKV immediates (bytecode_compile.c:670-715): the tensors come from the registers, the epilogue and the rotary
// parameters from the constant pool.
static marmot_error_t bc_exec_qkv(marmot_quant_kind_t kind, const void *exec_ctx, marmot_tensor_t **regs,
                                  const uint8_t *imm, const uint8_t *const_pool) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const void *device_ctx = ((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx;
    const uint8_t *pc = imm;
    uint16_t idx[7];
    for (int i = 0; i < 7; ++i) {
        idx[i] = rd_u16(&pc);
    }
    const uint32_t epilogue_off = rd_u32(&pc);
    const uint32_t rope_off = rd_u32(&pc);
    const uint16_t out_q = rd_u16(&pc), out_k = rd_u16(&pc), out_v = rd_u16(&pc);
    marmot_matmul_epilogue_t epilogue;
    marmot_rope_params_t rope;
    marmot_matmul_qkv_desc_t desc;
    memset(&desc, 0, sizeof(desc));
    if (epilogue_off != MARMOT_BC_INVALID_OFFSET || rope_off != MARMOT_BC_INVALID_OFFSET) {
        if (const_pool == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null const pool for qkv parameters");
        }
    }
    if (epilogue_off != MARMOT_BC_INVALID_OFFSET) {
        memcpy(&epilogue, const_pool + epilogue_off, sizeof(epilogue));
        desc.epilogue = &epilogue;
    }
    if (rope_off != MARMOT_BC_INVALID_OFFSET) {
        memcpy(&rope, const_pool + rope_off, sizeof(rope));
        desc.rope_params = &rope;
    }
    desc.input = reg(regs, idx[0]);
    desc.layout = MARMOT_QKV_LAYOUT_SEPARATE;
    desc.separate.wq = reg(regs, idx[1]);
    desc.separate.wk = reg(regs, idx[2]);
    desc.separate.wv = reg(regs, idx[3]);
    desc.separate.bq = reg(regs, idx[4]);
    desc.separate.bk = reg(regs, idx[5]);
    desc.separate.bv = reg(regs, idx[6]);
    desc.out_q = reg(regs, out_q);
    desc.out_k = reg(regs, out_k);
    desc.out_v = reg(regs, out_v);
    return matmul_qkv(device_ctx, kind, &desc);
}

#define HIP_BC_QKV_ENTRY(name, kind)                                                                                   \
    static marmot_error_t name(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,                       \
                               const uint8_t *const_pool) {                                                            \
        return bc_exec_qkv(kind, exec_ctx, regs, imm, const_pool);                                                     \
    }
HIP_BC_QKV_ENTRY(bc_exec_qkv_q4_0, MARMOT_QUANT_KIND_Q4_0)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q8_0, MARMOT_QUANT_KIND_Q8_0)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q4_k, MARMOT_QUANT_KIND_Q4_K)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q6_k, MARMOT_QUANT_KIND_Q6_K)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q5_k, MARMOT_QUANT_KIND_Q5_K)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q4_1, MARMOT_QUANT_KIND_Q4_1)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q5_0, MARMOT_QUANT_KIND_Q5_0)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q5_1, MARMOT_QUANT_KIND_Q5_1)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q2_k, MARMOT_QUANT_KIND_Q2_K)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q3_k, MARMOT_QUANT_KIND_Q3_K)
HIP_BC_QKV_ENTRY(bc_exec_qkv_q8_1, MARMOT_QUANT_KIND_Q8_1)

// EMBEDDING immediates (bytecode_compile.c:989-1018) -> the descriptor the generated shim builds
// (src/backends/cpu/dispatch/misc_dispatch_cpu.gen.c:115-133)
static marmot_error_t bc_exec_embedding(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                        const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const uint16_t weights = rd_u16(&pc), token_ids = rd_u16(&pc), out = rd_u16(&pc);
    const uint32_t dtype_out = rd_u32(&pc);
    const float scale = rd_f32(&pc);
    const uint32_t padding_id = rd_u32(&pc);
    const uint8_t bounds_check = pc[0], prefer_gpu = pc[1], allow_decode = pc[2];
    const marmot_embedding_gather_desc_t desc = {
        .weights = reg(regs, weights),
        .token_ids = reg(regs, token_ids),
        .out = reg(regs, out),
        .dtype_out = (marmot_dtype_t)dtype_out,
        .scale = scale,
        .padding_id = (int32_t)padding_id,
        .bounds_check = bounds_check != 0,
        .prefer_gpu_private = prefer_gpu ? MARMOT_PREFERENCE_ENABLE : MARMOT_PREFERENCE_DISABLE,
        .allow_quant_decode_on_the_fly = allow_decode ? MARMOT_PREFERENCE_ENABLE : MARMOT_PREFERENCE_DISABLE,
    };
    return embedding_gather(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, &desc);
}

static marmot_error_t bc_exec_moe(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                  const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    marmot_moe_experts_desc_t desc = {0};
    desc.hidden_states = reg(regs, rd_u16(&pc));
    desc.gate_exps = reg(regs, rd_u16(&pc));
    desc.up_exps = reg(regs, rd_u16(&pc));
    desc.down_exps = reg(regs, rd_u16(&pc));
    desc.topk_ids = reg(regs, rd_u16(&pc));
    desc.topk_weights = reg(regs, rd_u16(&pc));
    desc.out = reg(regs, rd_u16(&pc));
    desc.ffn_type = (marmot_ffn_type_t)rd_u32(&pc);
    desc.weights_scale = rd_f32(&pc);
    desc.router_weight_policy = (marmot_router_weight_policy_t)rd_u32(&pc);
    return moe_experts(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, &desc);
}

static marmot_error_t bc_exec_topk(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                   const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    marmot_topk_desc_t desc = {0};
    desc.x = reg(regs, rd_u16(&pc));
    desc.values_out = reg(regs, rd_u16(&pc));
    desc.indices_out = reg(regs, rd_u16(&pc));
    desc.axis = (int32_t)rd_u32(&pc);
    desc.k = rd_u32(&pc);
    return topk(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, &desc);
}

static marmot_error_t bc_exec_quantize(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                       const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *input = reg(regs, rd_u16(&pc));
    (void)rd_u32(&pc);  // quant params: unused by the block formats
    marmot_tensor_t *output = reg(regs, rd_u16(&pc));
    const uint32_t kind = rd_u32(&pc);
    const uint32_t layout = rd_u32(&pc);
    if (output != nullptr && ((uint32_t)output->quant_kind != kind || layout != MARMOT_QUANT_LAYOUT_GGUF)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Quantize: kind/layout immediates disagree with the output tensor");
    }
    return quantize_block(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, input, output);
}

static marmot_error_t bc_exec_dequantize(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                         const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *input = reg(regs, rd_u16(&pc));
    marmot_tensor_t *output = reg(regs, rd_u16(&pc));
    const uint32_t kind = rd_u32(&pc);
    const uint32_t layout = rd_u32(&pc);
    if (input != nullptr && ((uint32_t)input->quant_kind != kind || layout != MARMOT_QUANT_LAYOUT_GGUF)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Dequantize: kind/layout immediates disagree with the input tensor");
    }
    return dequantize_block(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, input, output);
}

// RMS_NORM: u16 input, weight, residual (0xFFFF none), output; f32 eps (bytecode_compile.c:530-552)
static marmot_error_t bc_exec_rms_norm_offset(float weight_offset, const void *exec_ctx, marmot_tensor_t **regs,
                                              const uint8_t *imm) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    marmot_rmsnorm_desc_t desc = {0};
    desc.x = reg(regs, rd_u16(&pc));
    desc.weight = reg(regs, rd_u16(&pc));
    desc.residual = reg(regs, rd_u16(&pc));
    desc.out = reg(regs, rd_u16(&pc));
    desc.eps = rd_f32(&pc);
    return rmsnorm(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, &desc, weight_offset);
}

static marmot_error_t bc_exec_rms_norm(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                       const uint8_t *const_pool) {
    (void)const_pool;
    return bc_exec_rms_norm_offset(0.0f, exec_ctx, regs, imm);
}

static marmot_error_t bc_exec_rms_norm_gemma(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                             const uint8_t *const_pool) {
    (void)const_pool;
    return bc_exec_rms_norm_offset(1.0f, exec_ctx, regs, imm);
}

// BINARY: u16 input_a, input_b, output (bytecode_compile.c:357-375)
static marmot_error_t bc_exec_binary(hip_binary_op_t op, const void *exec_ctx, marmot_tensor_t **regs,
                                     const uint8_t *imm) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *a = reg(regs, rd_u16(&pc));
    const marmot_tensor_t *c = reg(regs, rd_u16(&pc));
    marmot_tensor_t *out = reg(regs, rd_u16(&pc));
    return binary_f32(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, op, a, c, out);
}

static marmot_error_t bc_exec_swiglu(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                     const uint8_t *const_pool) {
    (void)const_pool;
    return bc_exec_binary(HIP_BIN_SWIGLU, exec_ctx, regs, imm);
}

static marmot_error_t bc_exec_geglu(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                    const uint8_t *const_pool) {
    (void)const_pool;
    return bc_exec_binary(HIP_BIN_GEGLU, exec_ctx, regs, imm);
}

static marmot_error_t bc_exec_add(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                  const uint8_t *const_pool) {
    (void)const_pool;
    return bc_exec_binary(HIP_BIN_ADD, exec_ctx, regs, imm);
}

// ROPE: u16 input, output, positions (0xFFFF: the positions of the parameters); u32 rope-params const offset;
// u32 n_past; u32 n_rot (bytecode_compile.c:598-623; bytecode_exec_cpu.gen.c:41088-41119). n_past and n_rot are
// carried but not read by the operation (rope_dispatch.c:145-372).
static marmot_error_t bc_exec_rope(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                   const uint8_t *const_pool) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *x = reg(regs, rd_u16(&pc));
    marmot_tensor_t *out = reg(regs, rd_u16(&pc));
    const uint16_t positions_idx = rd_u16(&pc);
    const uint32_t params_off = rd_u32(&pc);
    marmot_rope_params_t params;
    const marmot_rope_params_t *params_ptr = nullptr;
    if (params_off != MARMOT_BC_INVALID_OFFSET) {
        if (const_pool == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null const pool for rope params");
        }
        memcpy(&params, const_pool + params_off, sizeof(params));
        params_ptr = &params;
    }
    if (positions_idx != MARMOT_BC_REG_INVALID) {
        if (params_ptr == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Missing rope params");
        }
        params.positions = regs[positions_idx];
    }
    return rope(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, x, params_ptr, out);
}

// PAGED_ATTENTION immediates (bytecode_compile.c:553-597) -> the descriptor the generated shim builds
static marmot_error_t bc_exec_paged_attention(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                              const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    marmot_paged_attention_desc_t desc = {.struct_size = sizeof(desc), .struct_version = MARMOT_PAGED_ATTENTION_DESC_VERSION};
    desc.token_meta = reg(regs, rd_u16(&pc));
    desc.q = reg(regs, rd_u16(&pc));
    desc.k_new = reg(regs, rd_u16(&pc));
    desc.v_new = reg(regs, rd_u16(&pc));
    desc.kv_k = reg(regs, rd_u16(&pc));
    desc.kv_v = reg(regs, rd_u16(&pc));
    desc.block_table = reg(regs, rd_u16(&pc));
    marmot_paged_attention_kv_scale_ext_t ext = {.struct_size = sizeof(ext),
                                                 .struct_version = MARMOT_PAGED_ATTENTION_KV_SCALE_EXT_VERSION};
    ext.kv_k_scale = reg(regs, rd_u16(&pc));
    ext.kv_v_scale = reg(regs, rd_u16(&pc));
    desc.out = reg(regs, rd_u16(&pc));
    desc.token_count = rd_u32(&pc);
    desc.layer_idx = rd_u32(&pc);
    desc.num_q_heads = rd_u32(&pc);
    desc.num_kv_heads = rd_u32(&pc);
    desc.head_dim = rd_u32(&pc);
    desc.block_size = rd_u32(&pc);
    desc.scale = rd_f32(&pc);
    if (ext.kv_k_scale != nullptr || ext.kv_v_scale != nullptr) {
        desc.pnext = &ext;
    }
    return paged_attention(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, &desc);
}

static uint64_t rd_u64(const uint8_t **pc) {
    const uint64_t lo = rd_u32(pc);
    const uint64_t hi = rd_u32(pc);
    return lo | (hi << 32);
}

// data of the const pool at an offset (marmot_bc_const_data, src/core/bytecode/bytecode.h): nullptr for "none"
static const void *const_data(const uint8_t *const_pool, uint32_t off) {
    return off == MARMOT_BC_INVALID_OFFSET || const_pool == nullptr ? nullptr : const_pool + off;
}

// UNARY: u16 input, output; u32 activation-params const offset (bytecode_compile.c:331-356)
static marmot_error_t bc_exec_unary(int op, const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                    const uint8_t *const_pool) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *x = reg(regs, rd_u16(&pc));
    marmot_tensor_t *out = reg(regs, rd_u16(&pc));
    const uint32_t params_off = rd_u32(&pc);
    marmot_activation_params_t params;
    const marmot_activation_params_t *params_ptr = nullptr;
    if (params_off != MARMOT_BC_INVALID_OFFSET) {
        if (const_pool == nullptr) {
            return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null const pool for unary params");
        }
        memcpy(&params, const_pool + params_off, sizeof(params));
        params_ptr = &params;
    }
    return unary(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, op, x, params_ptr, out);
}

static marmot_error_t bc_exec_gelu(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                   const uint8_t *const_pool) {
    return bc_exec_unary(MARMOT_HIP_UNARY_GELU, exec_ctx, regs, imm, const_pool);
}

static marmot_error_t bc_exec_gelu_tanh(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                        const uint8_t *const_pool) {
    return bc_exec_unary(MARMOT_HIP_UNARY_GELU_TANH, exec_ctx, regs, imm, const_pool);
}

static marmot_error_t bc_exec_silu(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                   const uint8_t *const_pool) {
    return bc_exec_unary(MARMOT_HIP_UNARY_SILU, exec_ctx, regs, imm, const_pool);
}

// SOFTMAX: u16 input, output; u32 axis (bytecode_compile.c:440-458)
static marmot_error_t bc_exec_softmax(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                      const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    marmot_softmax_desc_t desc = {0};
    desc.x = reg(regs, rd_u16(&pc));
    desc.out = reg(regs, rd_u16(&pc));
    desc.axis = (int32_t)rd_u32(&pc);
    return softmax(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, &desc);
}

// RESHAPE: u16 input, output; u32 const offset of the new shape; u64 new_ndim (bytecode_compile.c:718-745)
static marmot_error_t bc_exec_reshape(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                      const uint8_t *const_pool) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *x = reg(regs, rd_u16(&pc));
    marmot_tensor_t *out = reg(regs, rd_u16(&pc));
    const uint32_t shape_off = rd_u32(&pc);
    const uint64_t ndim = rd_u64(&pc);
    if (shape_off != MARMOT_BC_INVALID_OFFSET && const_pool == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null const pool for reshape shape");
    }
    if (ndim > MARMOT_MAX_DIMS) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Reshape rank exceeds the tensor rank limit");
    }
    size_t shape[MARMOT_MAX_DIMS] = {0};
    const void *src = const_data(const_pool, shape_off);
    if (src != nullptr) {
        memcpy(shape, src, (size_t)ndim * sizeof(size_t));
    }
    return reshape(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, x, out, src != nullptr ? shape : nullptr,
                   (size_t)ndim);
}

// VIEW: u16 input, output; u64 byte offset (bytecode_compile.c:746-763)
static marmot_error_t bc_exec_view(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                   const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *x = reg(regs, rd_u16(&pc));
    marmot_tensor_t *out = reg(regs, rd_u16(&pc));
    const uint64_t byte_offset = rd_u64(&pc);
    return view(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, x, out, (size_t)byte_offset);
}

// SLICE: u16 input, output; u32 const offsets of starts and sizes, one size_t per output dimension
// (bytecode_compile.c:863-892)
static marmot_error_t bc_exec_slice(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                    const uint8_t *const_pool) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *x = reg(regs, rd_u16(&pc));
    marmot_tensor_t *out = reg(regs, rd_u16(&pc));
    const uint32_t starts_off = rd_u32(&pc);
    const uint32_t sizes_off = rd_u32(&pc);
    if ((starts_off != MARMOT_BC_INVALID_OFFSET || sizes_off != MARMOT_BC_INVALID_OFFSET) && const_pool == nullptr) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null const pool for slice starts");
    }
    size_t starts[MARMOT_MAX_DIMS] = {0}, sizes[MARMOT_MAX_DIMS] = {0};
    const void *s0 = const_data(const_pool, starts_off), *s1 = const_data(const_pool, sizes_off);
    const size_t ndim = out != nullptr && out->shape.ndim <= MARMOT_MAX_DIMS ? out->shape.ndim : 0;
    if (s0 != nullptr) {
        memcpy(starts, s0, ndim * sizeof(size_t));
    }
    if (s1 != nullptr) {
        memcpy(sizes, s1, ndim * sizeof(size_t));
    }
    return slice(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, x, out, s0 != nullptr ? starts : nullptr,
                 s1 != nullptr ? sizes : nullptr);
}

// GATHER_ROWS: u16 input, indices, output (bytecode_compile.c:893-911)
static marmot_error_t bc_exec_gather_rows(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                          const uint8_t *const_pool) {
    (void)const_pool;
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const marmot_tensor_t *x = reg(regs, rd_u16(&pc));
    const marmot_tensor_t *idx = reg(regs, rd_u16(&pc));
    marmot_tensor_t *out = reg(regs, rd_u16(&pc));
    return gather_rows(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, x, idx, out);
}

// CONVERT: u32 const offsets of the destination and source host addresses; u64 n; u32 dst dtype; u32 src dtype
// (bytecode_compile.c:1020-1043; the addresses are stored by value, marmot_bc_add_const_ptr_value :88)
static marmot_error_t bc_exec_convert(const void *exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                      const uint8_t *const_pool) {
    if (!exec_args_ok(exec_ctx, regs, imm)) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null bytecode exec arguments");
    }
    const uint8_t *pc = imm;
    const uint32_t dst_off = rd_u32(&pc);
    const uint32_t src_off = rd_u32(&pc);
    const uint64_t n = rd_u64(&pc);
    const marmot_dtype_t dst_dtype = (marmot_dtype_t)rd_u32(&pc);
    const marmot_dtype_t src_dtype = (marmot_dtype_t)rd_u32(&pc);
    if (const_pool == nullptr || dst_off == MARMOT_BC_INVALID_OFFSET || src_off == MARMOT_BC_INVALID_OFFSET) {
        return fail(MARMOT_ERROR_INVALID_ARGUMENT, "Null const pool for convert dst");
    }
    void *dst = nullptr;
    const void *src = nullptr;
    memcpy(&dst, const_pool + dst_off, sizeof(dst));
    memcpy(&src, const_pool + src_off, sizeof(src));
    return convert(((const marmot_bc_exec_ctx_t *)exec_ctx)->device_ctx, dst_dtype, dst, src_dtype, src, (size_t)n);
}

static const uint16_t k_imm_size[MARMOT_HIP_BC_OP_COUNT] = {
    0,               // END
    12, 12, 12, 12,  // MATMUL: 3 x u16 + u32 + u16
    26, 26, 26, 26,  // MOE_EXPERTS: 7 x u16 + u32 + f32 + u32
    14,              // TOPK: 3 x u16 + 2 x u32
    16,              // QUANTIZE: u16 + u32 + u16 + 2 x u32
    12,              // DEQUANTIZE: 2 x u16 + 2 x u32
    28, 28, 28, 28,  // QKV: 7 x u16 + 2 x u32 + 3 x u16
    21, 21, 21, 21,  // EMBEDDING: 3 x u16 + u32 + f32 + u32 + 3 x u8
    12, 26, 28, 21,  // Q5_K: MATMUL, MOE_EXPERTS, QKV, EMBEDDING
    12, 26, 28, 21,  // Q4_1
    12, 26, 28, 21,  // Q5_0
    12, 26, 28, 21,  // Q5_1
    12, 26, 28, 21,  // Q2_K
    12, 26, 28, 21,  // Q3_K
    12, 26, 28, 21,  // Q8_1
    12, 12,          // RMS_NORM, RMS_NORM_GEMMA: 4 x u16 + f32
    6, 6, 6,         // SWIGLU, GEGLU, ADD (BINARY): 3 x u16
    18,              // ROPE: 3 x u16 + 3 x u32
    48,              // PAGED_ATTENTION: 10 x u16 + 6 x u32 + f32
    8, 8, 8,         // GELU, GELU_TANH, SILU (UNARY): 2 x u16 + u32
    8,               // SOFTMAX: 2 x u16 + u32
    16,              // RESHAPE: 2 x u16 + u32 + u64
    12,              // VIEW: 2 x u16 + u64
    12,              // SLICE: 2 x u16 + 2 x u32
    6,               // GATHER_ROWS: 3 x u16
    24,              // CONVERT: 2 x u32 + u64 + 2 x u32
};

static const marmot_bc_schema_id_t k_schema_id[MARMOT_HIP_BC_OP_COUNT] = {
    MARMOT_BC_SCHEMA_INVALID,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MATMUL,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_MOE_EXPERTS,
    MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_TOPK,
    MARMOT_BC_SCHEMA_QUANTIZE,    MARMOT_BC_SCHEMA_DEQUANTIZE,  MARMOT_BC_SCHEMA_QKV,
    MARMOT_BC_SCHEMA_QKV,         MARMOT_BC_SCHEMA_QKV,         MARMOT_BC_SCHEMA_QKV,
    MARMOT_BC_SCHEMA_EMBEDDING,   MARMOT_BC_SCHEMA_EMBEDDING,   MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_EMBEDDING,   MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS,
    MARMOT_BC_SCHEMA_QKV,         MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_QKV, MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_QKV, MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_QKV, MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_QKV, MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_QKV, MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_MATMUL,      MARMOT_BC_SCHEMA_MOE_EXPERTS, MARMOT_BC_SCHEMA_QKV, MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_RMS_NORM,    MARMOT_BC_SCHEMA_RMS_NORM,
    MARMOT_BC_SCHEMA_BINARY,      MARMOT_BC_SCHEMA_BINARY,      MARMOT_BC_SCHEMA_BINARY,
    MARMOT_BC_SCHEMA_ROPE,
    MARMOT_BC_SCHEMA_PAGED_ATTENTION,
    MARMOT_BC_SCHEMA_UNARY,       MARMOT_BC_SCHEMA_UNARY,       MARMOT_BC_SCHEMA_UNARY,
    MARMOT_BC_SCHEMA_SOFTMAX,
    MARMOT_BC_SCHEMA_RESHAPE,     MARMOT_BC_SCHEMA_VIEW,        MARMOT_BC_SCHEMA_SLICE,
    MARMOT_BC_SCHEMA_GATHER_ROWS, MARMOT_BC_SCHEMA_CONVERT,
};

static const marmot_bc_exec_fn k_exec_table[MARMOT_HIP_BC_OP_COUNT] = {
    nullptr,
    bc_exec_matmul_q4_0, bc_exec_matmul_q8_0, bc_exec_matmul_q4_k, bc_exec_matmul_q6_k,
    bc_exec_moe,         bc_exec_moe,         bc_exec_moe,         bc_exec_moe,
    bc_exec_topk,        bc_exec_quantize,    bc_exec_dequantize,
    bc_exec_qkv_q4_0,    bc_exec_qkv_q8_0,    bc_exec_qkv_q4_k,    bc_exec_qkv_q6_k,
    bc_exec_embedding,   bc_exec_embedding,   bc_exec_embedding,   bc_exec_embedding,
    bc_exec_matmul_q5_k, bc_exec_moe,         bc_exec_qkv_q5_k,    bc_exec_embedding,
    bc_exec_matmul_q4_1, bc_exec_moe,         bc_exec_qkv_q4_1,    bc_exec_embedding,
    bc_exec_matmul_q5_0, bc_exec_moe,         bc_exec_qkv_q5_0,    bc_exec_embedding,
    bc_exec_matmul_q5_1, bc_exec_moe,         bc_exec_qkv_q5_1,    bc_exec_embedding,
    bc_exec_matmul_q2_k, bc_exec_moe,         bc_exec_qkv_q2_k,    bc_exec_embedding,
    bc_exec_matmul_q3_k, bc_exec_moe,         bc_exec_qkv_q3_k,    bc_exec_embedding,
    bc_exec_matmul_q8_1, bc_exec_moe,         bc_exec_qkv_q8_1,    bc_exec_embedding,
    bc_exec_rms_norm,    bc_exec_rms_norm_gemma,
    bc_exec_swiglu,      bc_exec_geglu,       bc_exec_add,
    bc_exec_rope,
    bc_exec_paged_attention,
    bc_exec_gelu,        bc_exec_gelu_tanh,   bc_exec_silu,
    bc_exec_softmax,
    bc_exec_reshape,     bc_exec_view,        bc_exec_slice,
    bc_exec_gather_rows, bc_exec_convert,
};

// ------------------------------------------------------------------ kernel query
static marmot_kernel_selection_t unsupported(const char *reason) {
    marmot_kernel_selection_t s = {0};
    s.supported = false;
    s.kernel_id = MARMOT_KERNEL_INVALID;
    s.op_index = MARMOT_KERNEL_OP_INDEX_INVALID;
    s.fallback_reason = reason;
    return s;
}

static marmot_kernel_selection_t selected(uint16_t op_index, double est_us, double workspace_mb) {
    marmot_kernel_selection_t s = {0};
    s.supported = true;
#ifdef MARMOT_HIP_IN_TREE
    s.kernel_id = marmot_hip_kernel_id_of_op(op_index);  // table emitted by the code generator
#else
    s.kernel_id = (marmot_kernel_id_t)(MARMOT_KERNEL_HIP_BASE + op_index);
#endif
    s.op_index = op_index;
    s.estimated_us = est_us;
    s.est_workspace_mb = workspace_mb;
    s.confidence = 0.8f;
    return s;
}

static int kind_of_scheme(marmot_qscheme_id_t q) {
    switch (q) {
    case MARMOT_QSCHEME_Q4_0:
        return MARMOT_HIP_KIND_Q4_0;
    case MARMOT_QSCHEME_Q4_1:
        return MARMOT_HIP_KIND_Q4_1;
    case MARMOT_QSCHEME_Q5_0:
        return MARMOT_HIP_KIND_Q5_0;
    case MARMOT_QSCHEME_Q5_1:
        return MARMOT_HIP_KIND_Q5_1;
    case MARMOT_QSCHEME_Q8_0:
        return MARMOT_HIP_KIND_Q8_0;
    case MARMOT_QSCHEME_Q8_1:
        return MARMOT_HIP_KIND_Q8_1;
    case MARMOT_QSCHEME_Q2_K:
        return MARMOT_HIP_KIND_Q2_K;
    case MARMOT_QSCHEME_Q3_K:
        return MARMOT_HIP_KIND_Q3_K;
    case MARMOT_QSCHEME_Q4_K:
        return MARMOT_HIP_KIND_Q4_K;
    case MARMOT_QSCHEME_Q5_K:
        return MARMOT_HIP_KIND_Q5_K;
    case MARMOT_QSCHEME_Q6_K:
        return MARMOT_HIP_KIND_Q6_K;
    case MARMOT_QSCHEME_Q8_K:
        return MARMOT_HIP_KIND_Q8_K;
    default:
        return 0;
    }
}

static uint16_t matmul_op_of_kind(int kind) {
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_0:
        return MARMOT_HIP_BC_OP_MATMUL_Q4_0;
    case MARMOT_HIP_KIND_Q8_0:
        return MARMOT_HIP_BC_OP_MATMUL_Q8_0;
    case MARMOT_HIP_KIND_Q4_K:
        return MARMOT_HIP_BC_OP_MATMUL_Q4_K;
    case MARMOT_HIP_KIND_Q6_K:
        return MARMOT_HIP_BC_OP_MATMUL_Q6_K;
    case MARMOT_HIP_KIND_Q5_K:
        return MARMOT_HIP_BC_OP_MATMUL_Q5_K;
    case MARMOT_HIP_KIND_Q4_1:
        return MARMOT_HIP_BC_OP_MATMUL_Q4_1;
    case MARMOT_HIP_KIND_Q5_0:
        return MARMOT_HIP_BC_OP_MATMUL_Q5_0;
    case MARMOT_HIP_KIND_Q5_1:
        return MARMOT_HIP_BC_OP_MATMUL_Q5_1;
    case MARMOT_HIP_KIND_Q8_1:
        return MARMOT_HIP_BC_OP_MATMUL_Q8_1;
    case MARMOT_HIP_KIND_Q2_K:
        return MARMOT_HIP_BC_OP_MATMUL_Q2_K;
    case MARMOT_HIP_KIND_Q3_K:
        return MARMOT_HIP_BC_OP_MATMUL_Q3_K;
    default:
        return MARMOT_KERNEL_OP_INDEX_INVALID;
    }
}

// The operation of a family (its Q4_0 op and its Q5_K op given) for the kind whose matmul op is mm: the first four
// kinds are numbered alike in every family; the kinds added behind them take four consecutive ops each, in the
// order MATMUL, MOE_EXPERTS, QKV, EMBEDDING.
static uint16_t family_op(uint16_t mm, uint16_t family_q4_0, uint16_t family_q5_k) {
    if (mm >= MARMOT_HIP_BC_OP_MATMUL_Q5_K) {
        return (uint16_t)(mm + (family_q5_k - MARMOT_HIP_BC_OP_MATMUL_Q5_K));
    }
    return (uint16_t)(family_q4_0 + (mm - MARMOT_HIP_BC_OP_MATMUL_Q4_0));
}

// ------------------------------------------------------------------ exports
const marmot_device_ops_t *marmot_get_hip_ops(void) {
    return &k_hip_ops;
}

marmot_kernel_selection_t marmot_hip_query_kernel(const marmot_op_signature_t *sig, const marmot_device_caps_t *caps) {
    if (sig == nullptr || caps == nullptr) {
        return unsupported("Invalid kernel query arguments");
    }
    const float bw_gbps = caps->mem_bw_gbps > 0.0f ? caps->mem_bw_gbps : 8000.0f;
    const float tflops = caps->peak_flops_tflops_fp16 > 0.0f ? caps->peak_flops_tflops_fp16 : 2500.0f;
    const double launch_us = caps->launch_overhead_us > 0.0f ? caps->launch_overhead_us : 2.0;
    const bool in32 = sig->input_dtype == MARMOT_DTYPE_FLOAT32, in16 = sig->input_dtype == MARMOT_DTYPE_FLOAT16;
    const bool out32 = sig->output_dtype == MARMOT_DTYPE_FLOAT32, out16 = sig->output_dtype == MARMOT_DTYPE_FLOAT16;
    switch (sig->op_id) {
    case MARMOT_OP_MATMUL:
    case MARMOT_OP_LINEAR: {
        const int kind = kind_of_scheme(sig->qscheme_id);
        const uint16_t op = matmul_op_of_kind(kind);
        if (op == MARMOT_KERNEL_OP_INDEX_INVALID) {
            return unsupported("HIP matmul handles Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 and Q2_K to Q6_K weights");
        }
        if (sig->matmul_layout != MARMOT_MATMUL_LAYOUT_NT) {
            return unsupported("HIP quantized matmul needs layout NT");
        }
        if (!((in32 && out32) || (in16 && (out32 || out16)))) {
            return unsupported("HIP quantized matmul: unsupported activation/output dtypes");
        }
        if (sig->accum_dtype != MARMOT_DTYPE_FLOAT32) {
            return unsupported("HIP quantized matmul accumulates in FLOAT32");
        }
        if (sig->weight_layout != MARMOT_WEIGHT_LAYOUT_SEPARATE) {
            return unsupported("HIP quantized matmul needs separate weights");
        }
        if (sig->stride_mode != MARMOT_STRIDE_MODE_CONTIGUOUS && sig->stride_mode != MARMOT_STRIDE_MODE_ANY) {
            return unsupported("HIP quantized matmul needs contiguous rows");
        }
        if ((sig->epilogue_flags & ~(uint32_t)MARMOT_EPILOGUE_BIAS) != 0 || sig->variant_flags != 0) {
            return unsupported("HIP quantized matmul fuses only the bias epilogue");
        }
        const size_t N = sig->dims.matmul.N, K = sig->dims.matmul.K, M = sig->dims.matmul.M;
        const double bytes =
            (double)M * (double)marmot_hip_row_bytes(kind, K) + (double)N * K * (in32 ? 4 : 2) + (double)N * M * 4;
        const double t_mem = bytes / (bw_gbps * 1e3);          // us
        const double t_mma = 2.0 * N * M * K / (tflops * 1e6);  // us
        const double ws_mb = in32 ? (double)marmot_hip_packed_activation_bytes(kind, N, K) / 1048576.0 : 0.0;
        return selected(op, launch_us + (t_mem > t_mma ? t_mem : t_mma), ws_mb);
    }
    case MARMOT_OP_QKV_PROJECTION:
    case MARMOT_OP_QKV_SHARED_INPUT:
    case MARMOT_OP_QKV_ROPE: {
        // cpu/kernels/matmul_qkv.def:19-36, 54-71: quantized weights of one scheme, layout NT, separate weights,
        // contiguous, FLOAT32 accumulation; outputs have the input dtype (matmul_qkv.c:1240-1243)
        const int kind = kind_of_scheme(sig->qscheme_id);
        const uint16_t mm = matmul_op_of_kind(kind);
        if (mm == MARMOT_KERNEL_OP_INDEX_INVALID) {
            return unsupported("HIP QKV projection handles Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 and Q2_K to Q6_K weights");
        }
        if (sig->matmul_layout != MARMOT_MATMUL_LAYOUT_NT) {
            return unsupported("HIP QKV projection needs layout NT");
        }
        if (!((in32 && out32) || (in16 && out16))) {
            return unsupported("HIP QKV projection: outputs must have the activation dtype (FLOAT32 or FLOAT16)");
        }
        if (sig->accum_dtype != MARMOT_DTYPE_FLOAT32) {
            return unsupported("HIP QKV projection accumulates in FLOAT32");
        }
        if (sig->weight_layout != MARMOT_WEIGHT_LAYOUT_SEPARATE) {
            return unsupported("HIP QKV projection needs separate weights");
        }
        if (sig->stride_mode != MARMOT_STRIDE_MODE_CONTIGUOUS && sig->stride_mode != MARMOT_STRIDE_MODE_ANY) {
            return unsupported("HIP QKV projection needs contiguous rows");
        }
        if ((sig->epilogue_flags & ~(uint32_t)(MARMOT_EPILOGUE_BIAS | MARMOT_EPILOGUE_ROPE)) != 0 ||
            sig->variant_flags != 0) {
            return unsupported("HIP QKV projection fuses the bias and rotary epilogues only");
        }
        const size_t N = sig->dims.matmul.N, K = sig->dims.matmul.K, M = sig->dims.matmul.M;
        const double bytes = 3.0 * (double)M * (double)marmot_hip_row_bytes(kind, K) +
                             (double)N * K * (in32 ? 4 : 2) + 3.0 * (double)N * M * (out32 ? 4 : 2);
        const double t_mem = bytes / (bw_gbps * 1e3);
        const double t_mma = 6.0 * N * M * K / (tflops * 1e6);
        const double ws_mb = (double)marmot_hip_packed_activation_bytes(kind, N, K) / 1048576.0;
        const uint16_t op = family_op(mm, MARMOT_HIP_BC_OP_QKV_Q4_0, MARMOT_HIP_BC_OP_QKV_Q5_K);
        return selected(op, launch_us + (t_mem > t_mma ? t_mem : t_mma), ws_mb);
    }
    case MARMOT_OP_EMBEDDING: {
        // cpu/kernels/embedding.def:19-30: the input dtype of this op is the index type
        const int kind = kind_of_scheme(sig->qscheme_id);
        const uint16_t mm = matmul_op_of_kind(kind);
        if (mm == MARMOT_KERNEL_OP_INDEX_INVALID) {
            return unsupported("HIP embedding gather handles Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 and Q2_K to Q6_K tables");
        }
        if (sig->input_dtype != MARMOT_DTYPE_INT32 && sig->input_dtype != MARMOT_DTYPE_INT64) {
            return unsupported("HIP embedding gather takes INT32 or INT64 token ids");
        }
        if (!out32 && !out16) {
            return unsupported("HIP embedding gather writes FLOAT32 or FLOAT16");
        }
        return selected(family_op(mm, MARMOT_HIP_BC_OP_EMBEDDING_Q4_0, MARMOT_HIP_BC_OP_EMBEDDING_Q5_K), launch_us, 0.0);
    }
    case MARMOT_OP_MOE_EXPERTS: {
        const int kind = kind_of_scheme(sig->qscheme_id);
        if (matmul_op_of_kind(kind) == MARMOT_KERNEL_OP_INDEX_INVALID) {
            return unsupported("HIP MoE experts handle Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 and Q2_K to Q6_K expert weights");
        }
        if (!in32 || !out32) {
            return unsupported("HIP MoE experts take FLOAT32 activations");
        }
        const uint16_t op = family_op(matmul_op_of_kind(kind), MARMOT_HIP_BC_OP_MOE_EXPERTS_Q4_0,
                                      MARMOT_HIP_BC_OP_MOE_EXPERTS_Q5_K);
        return selected(op, 0.0, 0.0);
    }
    case MARMOT_OP_RMS_NORM:
    case MARMOT_OP_RMS_NORM_GEMMA:
        // rms_norm_scalar / rms_norm_gemma_scalar (cpu/kernels/normalization.def): FLOAT32 rows, contiguous
        if (!in32 || !out32) {
            return unsupported("HIP RMSNorm handles FLOAT32 tensors");
        }
        return selected(sig->op_id == MARMOT_OP_RMS_NORM ? MARMOT_HIP_BC_OP_RMS_NORM_F32
                                                         : MARMOT_HIP_BC_OP_RMS_NORM_GEMMA_F32, launch_us, 0.0);
    case MARMOT_OP_SWIGLU:
    case MARMOT_OP_GEGLU:
    case MARMOT_OP_ADD:
        // glu_scalar / elementwise add (cpu/kernels/elementwise.def): FLOAT32
        if (!in32 || !out32) {
            return unsupported("HIP elementwise operations handle FLOAT32 tensors");
        }
        return selected(sig->op_id == MARMOT_OP_SWIGLU  ? MARMOT_HIP_BC_OP_SWIGLU_F32
                        : sig->op_id == MARMOT_OP_GEGLU ? MARMOT_HIP_BC_OP_GEGLU_F32
                                                        : MARMOT_HIP_BC_OP_ADD_F32, launch_us, 0.0);
    case MARMOT_OP_ROPE:
        // rope_scalar (cpu/kernels/rope.def): rows and result of one type, FLOAT32 or FLOAT16
        if (!((in32 && out32) || (in16 && out16))) {
            return unsupported("HIP RoPE handles FLOAT32 and FLOAT16 tensors");
        }
        return selected(MARMOT_HIP_BC_OP_ROPE, launch_us, 0.0);
    case MARMOT_OP_PAGED_ATTENTION: {
        // paged_attention_scalar (cpu/kernels/paged_attention.def): activations and result of one float type, the
        // cache type as the weight type, FLOAT8_E4M3 included
        const bool act_ok = pa_float_dtype(sig->input_dtype) && sig->output_dtype == sig->input_dtype;
        if (!act_ok || !(pa_float_dtype(sig->weight_dtype) || sig->weight_dtype == MARMOT_DTYPE_FLOAT8_E4M3)) {
            return unsupported("HIP paged attention handles FLOAT32, FLOAT16 and BFLOAT16 activations and those or "
                               "FLOAT8_E4M3 caches");
        }
        return selected(MARMOT_HIP_BC_OP_PAGED_ATTENTION, 2.0 * launch_us, 0.0);
    }
    case MARMOT_OP_TOPK:
        if (!in32 || !out32) {
            return unsupported("HIP TopK takes FLOAT32 values");
        }
        return selected(MARMOT_HIP_BC_OP_TOPK_F32, launch_us, 0.0);
    case MARMOT_OP_QUANTIZE: {
        const bool act = sig->qscheme_id == MARMOT_QSCHEME_Q8_0 || sig->qscheme_id == MARMOT_QSCHEME_Q8_K;
        const bool wgt = sig->qscheme_id == MARMOT_QSCHEME_Q4_K || sig->qscheme_id == MARMOT_QSCHEME_Q5_K ||
            sig->qscheme_id == MARMOT_QSCHEME_Q6_K;
        if (!((act && (in32 || in16)) || (wgt && in32))) {
            return unsupported("HIP quantize produces Q8_0 and Q8_K from FLOAT32/FLOAT16, Q4_K, Q5_K and Q6_K from FLOAT32");
        }
        return selected(MARMOT_HIP_BC_OP_QUANTIZE_BLOCK, launch_us, 0.0);
    }
    case MARMOT_OP_DEQUANTIZE:
        if (kind_of_scheme(sig->qscheme_id) == 0 || !out32) {
            return unsupported("HIP dequantize handles Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 and Q2_K to Q8_K to FLOAT32");
        }
        return selected(MARMOT_HIP_BC_OP_DEQUANTIZE_BLOCK, launch_us, 0.0);
    case MARMOT_OP_GELU:
    case MARMOT_OP_GELU_TANH:
    case MARMOT_OP_SILU:
        // gelu / gelu_tanh / silu (cpu/kernels/unary.def): values and result of one type, FLOAT32 or FLOAT16
        if (!((in32 && out32) || (in16 && out16))) {
            return unsupported("HIP unary operations handle FLOAT32 and FLOAT16 tensors");
        }
        return selected(sig->op_id == MARMOT_OP_GELU        ? MARMOT_HIP_BC_OP_GELU
                        : sig->op_id == MARMOT_OP_GELU_TANH ? MARMOT_HIP_BC_OP_GELU_TANH
                                                            : MARMOT_HIP_BC_OP_SILU, launch_us, 0.0);
    case MARMOT_OP_SOFTMAX: {
        // one executor for the three types: it reads the type from the tensors
        const bool bf = sig->input_dtype == MARMOT_DTYPE_BFLOAT16 && sig->output_dtype == MARMOT_DTYPE_BFLOAT16;
        if (!((in32 && out32) || (in16 && out16) || bf)) {
            return unsupported("HIP softmax handles FLOAT32, FLOAT16 and BFLOAT16 tensors");
        }
        return selected(MARMOT_HIP_BC_OP_SOFTMAX_F32, launch_us, 0.0);
    }
    case MARMOT_OP_RESHAPE:
        return selected(MARMOT_HIP_BC_OP_RESHAPE, 0.0, 0.0);  // metadata only
    case MARMOT_OP_VIEW:
        return selected(MARMOT_HIP_BC_OP_VIEW, 0.0, 0.0);  // metadata only
    case MARMOT_OP_SLICE:
        return selected(MARMOT_HIP_BC_OP_SLICE, launch_us, 0.0);
    case MARMOT_OP_GATHER_ROWS:
        return selected(MARMOT_HIP_BC_OP_GATHER_ROWS, launch_us, 0.0);
    case MARMOT_OP_CONVERT: {
        const bool src_ok = in32 || in16 || sig->input_dtype == MARMOT_DTYPE_BFLOAT16;
        const bool dst_ok = out32 || out16 || sig->output_dtype == MARMOT_DTYPE_BFLOAT16;
        if (!src_ok || !dst_ok) {
            return unsupported("HIP convert handles FLOAT32, FLOAT16 and BFLOAT16");
        }
        return selected(MARMOT_HIP_BC_OP_CONVERT, launch_us, 0.0);
    }
    default:
        return unsupported("Operation not provided by the HIP backend");
    }
}

marmot_device_caps_t marmot_hip_detect_default_caps(void) {
    marmot_device_caps_t c = {0};
    // published MI355X figures; a live device refines the counts
    c.peak_flops_tflops_fp32 = 157.3f;
    c.peak_flops_tflops_fp16 = 2500.0f;
    c.mem_bw_gbps = 8000.0f;
    c.launch_overhead_us = 2.0f;
    c.edge_penalty_alpha = 0.0f;
    c.l1_cache_kb = 32;
    c.l2_cache_kb = 4096;
    c.l3_cache_mb = 256;
    c.num_compute_units = 256;
    c.simd_width = 64;
    c.has_fma = true;
    c.has_fp16_compute = true;
    c.has_bf16_compute = true;
    c.has_tensor_cores = true;
    c.has_simdgroup_mm = false;
    c.h2d_bw_gbps = 64.0f;
    c.d2h_bw_gbps = 64.0f;
    c.d2d_bw_gbps = 4000.0f;
    c.d2d_lat_us = 2.0f;
    c.copy_engines = 2;
    c.max_streams = 4;
    marmot_hip_device_t *dev = nullptr;
    if (marmot_hip_device_create(0, &dev) == MARMOT_HIP_SUCCESS) {
        marmot_hip_caps_t hc;
        if (marmot_hip_get_caps(dev, &hc) == MARMOT_HIP_SUCCESS) {
            c.num_compute_units = hc.num_compute_units;
            c.simd_width = hc.wavefront_size;
            c.l2_cache_kb = hc.l2_cache_kb;
            c.mem_bw_gbps = hc.mem_bw_gbps;
            c.peak_flops_tflops_fp16 = hc.peak_tflops_fp16;
        }
        marmot_hip_device_destroy(dev);
    }
    return c;
}

bool marmot_hip_default_preferences(const marmot_device_caps_t *caps, marmot_backend_preferences_t *prefs_out) {
    if (caps == nullptr || prefs_out == nullptr) {
        return false;
    }
    memset(prefs_out, 0, sizeof(*prefs_out));
    prefs_out->policy.embedding_quant_output_dtype = MARMOT_DTYPE_FLOAT32;
    prefs_out->policy.quant_activation_mode = MARMOT_QUANT_ACTIVATION_AUTO;
    prefs_out->policy.variant_flags_mask = 0;  // no fused variants yet
    prefs_out->policy.embedding_prefer_gpu_private = false;
    prefs_out->policy.embedding_allow_quant_decode_on_the_fly = false;
    // views into a mirrored range resolve to offsets in the mirror, so offset views need no temporaries
    prefs_out->policy.matmul_requires_temp_tensors = false;
    prefs_out->policy.matmul_prefer_packed_weights = false;  // kernels read native GGUF blocks
    prefs_out->routing_policy = MARMOT_ROUTING_ALWAYS_GPU;
    return true;
}

bool marmot_hip_bc_get_tables(marmot_bc_tables_t *out) {
    if (out == nullptr) {
        return false;
    }
    out->imm_size = k_imm_size;
    out->exec_table = k_exec_table;
    out->schema_id = k_schema_id;
    out->op_count = MARMOT_HIP_BC_OP_COUNT;
    return true;
}

marmot_error_t hip_matmul_quantized_q4_0(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q4_0, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q8_0(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q8_0, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q4_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q4_K, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q4_1(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q4_1, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q5_0(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q5_0, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q5_1(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q5_1, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q2_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q2_K, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q3_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q3_K, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q8_1(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q8_1, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q5_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q5_K, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_quantized_q6_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out) {
    return matmul_quantized(device_ctx, MARMOT_QUANT_KIND_Q6_K, input, weight, epilogue, out);
}
marmot_error_t hip_matmul_qkv_q4_0(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q4_0, desc);
}
marmot_error_t hip_matmul_qkv_q8_0(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q8_0, desc);
}
marmot_error_t hip_matmul_qkv_q4_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q4_K, desc);
}
marmot_error_t hip_matmul_qkv_q4_1(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q4_1, desc);
}
marmot_error_t hip_matmul_qkv_q5_0(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q5_0, desc);
}
marmot_error_t hip_matmul_qkv_q5_1(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q5_1, desc);
}
marmot_error_t hip_matmul_qkv_q2_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q2_K, desc);
}
marmot_error_t hip_matmul_qkv_q3_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q3_K, desc);
}
marmot_error_t hip_matmul_qkv_q8_1(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q8_1, desc);
}
marmot_error_t hip_matmul_qkv_q5_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q5_K, desc);
}
marmot_error_t hip_matmul_qkv_q6_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc) {
    return matmul_qkv(device_ctx, MARMOT_QUANT_KIND_Q6_K, desc);
}
marmot_error_t hip_embedding_gather(const void *device_ctx, const marmot_embedding_gather_desc_t *desc) {
    return embedding_gather(device_ctx, desc);
}
marmot_error_t hip_moe_experts_impl(const void *device_ctx, const marmot_moe_experts_desc_t *desc) {
    return moe_experts(device_ctx, desc);
}
marmot_error_t hip_topk_impl(const void *device_ctx, const marmot_topk_desc_t *desc) {
    return topk(device_ctx, desc);
}
marmot_error_t hip_rmsnorm_impl(const void *device_ctx, const marmot_rmsnorm_desc_t *desc) {
    return rmsnorm(device_ctx, desc, 0.0f);
}
marmot_error_t hip_rmsnorm_gemma_impl(const void *device_ctx, const marmot_rmsnorm_desc_t *desc) {
    return rmsnorm(device_ctx, desc, 1.0f);
}
marmot_error_t hip_swiglu_f32(const void *device_ctx, const marmot_tensor_t *a, const marmot_tensor_t *b,
                              marmot_tensor_t *out) {
    return binary_f32(device_ctx, HIP_BIN_SWIGLU, a, b, out);
}
marmot_error_t hip_geglu_f32(const void *device_ctx, const marmot_tensor_t *a, const marmot_tensor_t *b,
                             marmot_tensor_t *out) {
    return binary_f32(device_ctx, HIP_BIN_GEGLU, a, b, out);
}
marmot_error_t hip_add_f32(const void *device_ctx, const marmot_tensor_t *a, const marmot_tensor_t *b,
                           marmot_tensor_t *out) {
    return binary_f32(device_ctx, HIP_BIN_ADD, a, b, out);
}
marmot_error_t hip_paged_attention_impl(const void *device_ctx, const marmot_paged_attention_desc_t *desc) {
    return paged_attention(device_ctx, desc);
}
marmot_error_t hip_rope(const void *device_ctx, const marmot_tensor_t *x, const marmot_rope_params_t *params,
                        marmot_tensor_t *out) {
    return rope(device_ctx, x, params, out);
}
marmot_error_t hip_gelu(const void *device_ctx, const marmot_tensor_t *x, const marmot_activation_params_t *params,
                        marmot_tensor_t *out) {
    return unary(device_ctx, MARMOT_HIP_UNARY_GELU, x, params, out);
}
marmot_error_t hip_gelu_tanh(const void *device_ctx, const marmot_tensor_t *x, const marmot_activation_params_t *params,
                             marmot_tensor_t *out) {
    return unary(device_ctx, MARMOT_HIP_UNARY_GELU_TANH, x, params, out);
}
marmot_error_t hip_silu(const void *device_ctx, const marmot_tensor_t *x, const marmot_activation_params_t *params,
                        marmot_tensor_t *out) {
    return unary(device_ctx, MARMOT_HIP_UNARY_SILU, x, params, out);
}
marmot_error_t hip_softmax_impl(const void *device_ctx, const marmot_softmax_desc_t *desc) {
    return softmax(device_ctx, desc);
}
marmot_error_t hip_reshape(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out,
                           const size_t *new_shape, size_t new_ndim) {
    return reshape(device_ctx, x, out, new_shape, new_ndim);
}
marmot_error_t hip_view(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out, size_t byte_offset) {
    return view(device_ctx, x, out, byte_offset);
}
marmot_error_t hip_slice(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out, const size_t *starts,
                         const size_t *sizes) {
    return slice(device_ctx, x, out, starts, sizes);
}
marmot_error_t hip_gather_rows(const void *device_ctx, const marmot_tensor_t *input, const marmot_tensor_t *indices,
                               marmot_tensor_t *out) {
    return gather_rows(device_ctx, input, indices, out);
}
marmot_error_t hip_convert(const void *device_ctx, marmot_dtype_t dst_dtype, void *dst, marmot_dtype_t src_dtype,
                           const void *src, size_t n) {
    return convert(device_ctx, dst_dtype, dst, src_dtype, src, n);
}
marmot_error_t hip_quantize_block(const void *device_ctx, const marmot_tensor_t *input, marmot_tensor_t *output) {
    return quantize_block(device_ctx, input, output);
}
marmot_error_t hip_dequantize_block(const void *device_ctx, const marmot_tensor_t *input, marmot_tensor_t *output) {
    return dequantize_block(device_ctx, input, output);
}

marmot_error_t marmot_hip_backend_last_error(const char **detail_out) {
#ifdef MARMOT_HIP_IN_TREE
    if (detail_out != nullptr) {
        *detail_out = marmot_get_last_error_detail();
    }
    return marmot_get_last_error();
#else
    if (detail_out != nullptr) {
        *detail_out = g_last_detail;
    }
    return g_last_code;
#endif
}

void marmot_hip_backend_residency_stats(const void *device_ctx, marmot_hip_residency_stats_t *out) {
    hip_backend_t *b = backend_of(device_ctx);
    if (b == nullptr || out == nullptr) {
        return;
    }
    pthread_mutex_lock(&b->mu);
    out->mirrors = b->n_mirrors;
    out->mirrored_bytes = b->mirrored_bytes;
    out->uploads = b->uploads;
    out->upload_bytes = b->upload_bytes;
    out->downloads = b->downloads;
    out->download_bytes = b->download_bytes;
    out->activation_packs = b->packs_made;
    out->activation_pack_hits = b->pack_hits;
    pthread_mutex_unlock(&b->mu);
}

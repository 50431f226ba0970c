// Device object, memory, events, error text: the plumbing half of the C ABI (include/marmot_hip.h).
#include "mh_common.h"

#include <stdlib.h>

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

namespace mh {

static thread_local char g_error[512] = "";
static thread_local char g_route[96] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

void set_route(const char *name) {
    snprintf(g_route, sizeof(g_route), "%s", name);
}

int check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) {
        return MARMOT_HIP_SUCCESS;
    }
    const int code = (e == hipErrorOutOfMemory) ? MARMOT_HIP_ERROR_OUT_OF_MEMORY
        : (e == hipErrorNoDevice || e == hipErrorInvalidDevice) ? MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE
                                                                : MARMOT_HIP_ERROR_INVALID_OPERATION;
    return set_error(code, "HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
}

int workspace_reserve(marmot_hip_device *dev, size_t bytes, void **out) {
    if (dev->use_static_scratch) {
        if (bytes > dev->static_scratch_bytes) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT,
                             "this call needs %zu bytes of scratch; the entry point that does not allocate has %zu "
                             "(use the allocating entry point for this shape)", bytes, dev->static_scratch_bytes);
        }
        *out = dev->static_scratch;
        return MARMOT_HIP_SUCCESS;
    }
    if (bytes > dev->workspace_bytes) {
        if (dev->capturing) {
            return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION,
                             "workspace of %zu bytes is needed but the stream is being captured; run the call once "
                             "eagerly before capturing", bytes);
        }
        // round up so that a sequence of growing requests does not reallocate every time
        size_t want = dev->workspace_bytes ? dev->workspace_bytes : (size_t)1 << 20;
        while (want < bytes) {
            want *= 2;
        }
        MH_HIP(hipStreamSynchronize(dev->stream));
        void *fresh = nullptr;
        MH_HIP(hipMalloc(&fresh, want));
        if (dev->workspace != nullptr) {
            // Executable graphs captured earlier replay kernels whose arguments point into the old workspace: it
            // stays allocated until the last of them is destroyed.
            if (dev->live_graphs > 0) {
                dev->retired_workspaces.push_back(dev->workspace);
            } else {
                MH_HIP(hipFree(dev->workspace));
            }
        }
        dev->workspace = fresh;
        dev->workspace_bytes = want;
    }
    *out = dev->workspace;
    return MARMOT_HIP_SUCCESS;
}

int allow_large_lds(marmot_hip_device *dev, const void *kernel) {
    std::lock_guard<std::mutex> lock(dev->mu);
    if (dev->large_lds_kernels.count(kernel) == 0) {
        MH_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        dev->large_lds_kernels.insert(kernel);
    }
    return MARMOT_HIP_SUCCESS;
}

static inline size_t round256(size_t v) {
    return (v + 255) & ~(size_t)255;
}

size_t act_scratch_layout(int act_kind, size_t rows, size_t k, void *base, ActScratch *out) {
    const size_t bv = block_values(act_kind);
    const size_t nb = (k + bv - 1) / bv;
    const size_t kp = nb * bv;
    const size_t qs_bytes = round256(rows * kp);
    const size_t d_bytes = round256(rows * nb * sizeof(float));
    const size_t sums_per_block = (act_kind == MARMOT_HIP_KIND_Q8_K) ? 16 : 1;
    const size_t sums_bytes = round256(rows * nb * sums_per_block * sizeof(int16_t));
    if (out != nullptr) {
        uint8_t *p = (uint8_t *)base;
        out->qs = (int8_t *)p;
        out->d = (float *)(p + qs_bytes);
        out->sums = (int16_t *)(p + qs_bytes + d_bytes);
        out->kp = kp;
        out->nb = nb;
    }
    return qs_bytes + d_bytes + sums_bytes;
}

} // namespace mh

using namespace mh;

extern "C" {

int marmot_hip_fill_bytes_internal(marmot_hip_device_t *dev, void *d_dst, int value, size_t size);
int marmot_hip_copy16_internal(marmot_hip_device_t *dev, void *d_dst, const void *d_src, size_t size);

const char *marmot_hip_last_error(void) {
    return g_error;
}

const char *marmot_hip_last_route(void) {
    return g_route;
}

const char *marmot_hip_version(void) {
    return "marmot_hip 0.1 (gfx950)";
}

size_t marmot_hip_block_values(int kind) {
    return block_values(kind);
}
size_t marmot_hip_block_bytes(int kind) {
    return block_bytes(kind);
}
size_t marmot_hip_row_bytes(int kind, size_t k) {
    const size_t bv = block_values(kind);
    return bv == 0 ? 0 : ((k + bv - 1) / bv) * block_bytes(kind);
}

// Streams and events of the branch sections (marmot_hip_branch_*), made by the first section of a device object and
// never inside a stream capture. Not at creation: the runtime spreads a process's streams over a few hardware queues
// (four by default) in the order they are made, so three idle side streams per device object would put the main
// streams of several device objects onto ONE hardware queue and serialize work that ran side by side before
// (measured: three linears on three device objects 19 us together, 31 us with the side streams made up front).
// Default priority, like the main stream.
static int branches_init(marmot_hip_device *dev) {
    if (dev->fork_event != nullptr) {
        return 0;
    }
    for (int i = 0; i < marmot_hip_device::MAX_BRANCHES - 1; ++i) {
        if (check_hip(hipStreamCreateWithFlags(&dev->side_streams[i], hipStreamNonBlocking), "hipStreamCreateWithFlags") != 0 ||
            check_hip(hipEventCreateWithFlags(&dev->side_done[i], hipEventDisableTiming), "hipEventCreateWithFlags") != 0) {
            return -1;
        }
    }
    return check_hip(hipEventCreateWithFlags(&dev->fork_event, hipEventDisableTiming), "hipEventCreateWithFlags");
}

static void branches_destroy(marmot_hip_device *dev) {
    for (int i = 0; i < marmot_hip_device::MAX_BRANCHES - 1; ++i) {
        if (dev->side_streams[i] != nullptr) {
            (void)hipStreamDestroy(dev->side_streams[i]);
        }
        if (dev->side_done[i] != nullptr) {
            (void)hipEventDestroy(dev->side_done[i]);
        }
    }
    if (dev->fork_event != nullptr) {
        (void)hipEventDestroy(dev->fork_event);
    }
}

// Waits for everything this device object has enqueued: the open stream and, inside a branch section, the main stream
// and the side streams of the branches opened so far.
static hipError_t streams_synchronize(marmot_hip_device *dev) {
    hipError_t e = hipStreamSynchronize(dev->stream);
    if (dev->branch >= 0) {
        if (e == hipSuccess && dev->stream != dev->main_stream) {
            e = hipStreamSynchronize(dev->main_stream);
        }
        for (int i = 1; i < dev->branches_used && e == hipSuccess; ++i) {
            if (dev->side_streams[i - 1] != dev->stream) {
                e = hipStreamSynchronize(dev->side_streams[i - 1]);
            }
        }
    }
    return e;
}

int marmot_hip_device_create(int device_index, marmot_hip_device_t **out_dev) {
    if (out_dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "out_dev is null");
    }
    *out_dev = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "no HIP device available (%s)",
                         e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    }
    if (device_index < 0 || device_index >= count) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "device index %d out of range (%d devices)",
                         device_index, count);
    }
    MH_HIP(hipSetDevice(device_index));
    marmot_hip_device *dev = new marmot_hip_device();
    dev->device_index = device_index;
    if (check_hip(hipGetDeviceProperties(&dev->props, device_index), "hipGetDeviceProperties") != 0) {
        delete dev;
        return MARMOT_HIP_ERROR_BACKEND_INIT_FAILED;
    }
    if (strncmp(dev->props.gcnArchName, "gfx950", 6) != 0) {
        const int st = set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE,
                                 "libmarmot_hip is built for gfx950 only; device %d is %s", device_index,
                                 dev->props.gcnArchName);
        delete dev;
        return st;
    }
    // route switches: read here, never on a launch path
    dev->knobs.no_mmq = getenv("MARMOT_HIP_NO_MMQ") != nullptr;
    dev->knobs.no_row_kernels = getenv("MARMOT_HIP_NO_ROW_KERNELS") != nullptr;
    dev->knobs.no_resident_rows = getenv("MARMOT_HIP_NO_RESIDENT_ROWS") != nullptr;
    dev->knobs.no_attention_mfma = getenv("MARMOT_HIP_NO_ATTENTION_MFMA") != nullptr;
    dev->knobs.no_fp8_update_fused = getenv("MARMOT_HIP_NO_FP8_UPDATE_FUSED") != nullptr;
    dev->knobs.no_lds_ring = getenv("MARMOT_HIP_NO_LDS_RING") != nullptr;
    dev->knobs.no_fused_quant = getenv("MARMOT_HIP_NO_FUSED_QUANT") != nullptr;
    dev->knobs.no_gemm = getenv("MARMOT_HIP_NO_GEMM") != nullptr;
    dev->knobs.no_gemm_loaders = getenv("MARMOT_HIP_NO_GEMM_LOADERS") != nullptr;
    dev->knobs.gemm_wide = getenv("MARMOT_HIP_GEMM_WIDE") != nullptr;
    dev->knobs.no_gemm_wide = getenv("MARMOT_HIP_NO_GEMM_WIDE") != nullptr;
    dev->knobs.no_gemm_i8 = getenv("MARMOT_HIP_NO_GEMM_I8") != nullptr;
    dev->knobs.moe_no_validate = getenv("MARMOT_HIP_MOE_NO_VALIDATE") != nullptr;
    // default priority, non-blocking with respect to the legacy default stream
    if (check_hip(hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking), "hipStreamCreateWithFlags") != 0) {
        delete dev;
        return MARMOT_HIP_ERROR_BACKEND_INIT_FAILED;
    }
    dev->main_stream = dev->stream;
    if (static_scratch_init(dev) != 0) {
        branches_destroy(dev);
        (void)hipStreamDestroy(dev->stream);
        delete dev;
        return MARMOT_HIP_ERROR_BACKEND_INIT_FAILED;
    }
    if (const char *limit = getenv("MARMOT_HIP_SPIN_LIMIT")) {
        const long long v = atoll(limit);
        dev->spin_limit = v < 0 ? 0u : (v > 0xffffffffll ? 0xffffffffu : (uint32_t)v);
    }
    if (check_hip(hipMalloc((void **)&dev->fault_word, 256), "hipMalloc(fault word)") != 0 ||
        check_hip(hipMemset(dev->fault_word, 0, 256), "hipMemset(fault word)") != 0) {
        branches_destroy(dev);
        (void)hipStreamDestroy(dev->stream);
        delete dev;
        return MARMOT_HIP_ERROR_BACKEND_INIT_FAILED;
    }
    *out_dev = dev;
    return MARMOT_HIP_SUCCESS;
}

void marmot_hip_device_destroy(marmot_hip_device_t *dev) {
    if (dev == nullptr) {
        return;
    }
    (void)hipSetDevice(dev->device_index);
    (void)streams_synchronize(dev);
    if (dev->workspace != nullptr) {
        (void)hipFree(dev->workspace);
    }
    for (auto &parked : dev->branch_workspace) {
        if (parked.ptr != nullptr) {
            (void)hipFree(parked.ptr);
        }
    }
    for (void *w : dev->retired_workspaces) {
        (void)hipFree(w);
    }
    for (auto &kv : dev->allocs) {
        (void)hipFree(kv.first);
    }
    if (dev->fault_word != nullptr) {
        (void)hipFree(dev->fault_word);
    }
    branches_destroy(dev);
    (void)hipStreamDestroy(dev->main_stream);
    delete dev;
}

int marmot_hip_alloc(marmot_hip_device_t *dev, size_t size, void **out_dptr) {
    if (dev == nullptr || out_dptr == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "alloc: null argument");
    }
    *out_dptr = nullptr;
    if (size == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "alloc: size is 0");
    }
    void *p = nullptr;
    MH_HIP(hipMalloc(&p, size));
    {
        std::lock_guard<std::mutex> lock(dev->mu);
        dev->allocs[p] = size;
        dev->current_bytes += size;
        if (dev->current_bytes > dev->peak_bytes) {
            dev->peak_bytes = dev->current_bytes;
        }
    }
    *out_dptr = p;
    return MARMOT_HIP_SUCCESS;
}

void marmot_hip_free(marmot_hip_device_t *dev, void *dptr) {
    if (dev == nullptr || dptr == nullptr) {
        return;
    }
    {
        std::lock_guard<std::mutex> lock(dev->mu);
        auto it = dev->allocs.find(dptr);
        if (it == dev->allocs.end()) {
            return; // not ours
        }
        dev->current_bytes -= it->second;
        dev->allocs.erase(it);
    }
    (void)streams_synchronize(dev);
    (void)hipFree(dptr);
}

int marmot_hip_memcpy_to_device(marmot_hip_device_t *dev, void *d_dst, const void *host_src, size_t size) {
    if (dev == nullptr || d_dst == nullptr || host_src == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "memcpy_to_device: null argument");
    }
    if (size == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipMemcpyAsync(d_dst, host_src, size, hipMemcpyHostToDevice, dev->stream));
    MH_HIP(hipStreamSynchronize(dev->stream));
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_memcpy_from_device(marmot_hip_device_t *dev, void *host_dst, const void *d_src, size_t size) {
    if (dev == nullptr || host_dst == nullptr || d_src == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "memcpy_from_device: null argument");
    }
    if (size == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipMemcpyAsync(host_dst, d_src, size, hipMemcpyDeviceToHost, dev->stream));
    MH_HIP(hipStreamSynchronize(dev->stream));
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_memcpy_device(marmot_hip_device_t *dev, void *d_dst, const void *d_src, size_t size) {
    if (dev == nullptr || d_dst == nullptr || d_src == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "memcpy_device: null argument");
    }
    if (size == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (size % 16 == 0 && ((((uintptr_t)d_dst) | ((uintptr_t)d_src)) & 15) == 0) {
        return marmot_hip_copy16_internal(dev, d_dst, d_src, size);  // a kernel: capturable, on this stream
    }
    MH_HIP(hipMemcpyAsync(d_dst, d_src, size, hipMemcpyDeviceToDevice, dev->stream));
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_memset(marmot_hip_device_t *dev, void *d_dst, int value, size_t size) {
    if (dev == nullptr || d_dst == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "memset: null argument");
    }
    if (size == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    // a fill kernel rather than hipMemsetAsync, so that callers may capture this call into a HIP graph
    return marmot_hip_fill_bytes_internal(dev, d_dst, value, size);
}

int marmot_hip_synchronize(marmot_hip_device_t *dev) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "synchronize: null device");
    }
    MH_HIP(streams_synchronize(dev));
    // a row-owning kernel whose wavefronts gave up waiting for one another (SpinGuard, mh_rows.h) has left its mark
    uint32_t fault = 0;
    MH_HIP(hipMemcpy(&fault, dev->fault_word, sizeof(fault), hipMemcpyDeviceToHost));
    if (fault != 0) {
        MH_HIP(hipMemset(dev->fault_word, 0, sizeof(fault)));
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION,
                         "a row-owning kernel gave up waiting inside a workgroup (spin limit %u): its outputs are not valid",
                         dev->spin_limit);
    }
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_allocator_usage(marmot_hip_device_t *dev, size_t *current_bytes, size_t *peak_bytes, size_t *n_allocs) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "allocator_usage: null device");
    }
    std::lock_guard<std::mutex> lock(dev->mu);
    if (current_bytes != nullptr) {
        *current_bytes = dev->current_bytes;
    }
    if (peak_bytes != nullptr) {
        *peak_bytes = dev->peak_bytes;
    }
    if (n_allocs != nullptr) {
        *n_allocs = dev->allocs.size();
    }
    return MARMOT_HIP_SUCCESS;
}

void *marmot_hip_stream(marmot_hip_device_t *dev) {
    return dev != nullptr ? (void *)dev->stream : nullptr;
}

int marmot_hip_get_caps(marmot_hip_device_t *dev, marmot_hip_caps_t *caps) {
    if (dev == nullptr || caps == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "get_caps: null argument");
    }
    memset(caps, 0, sizeof(*caps));
    snprintf(caps->name, sizeof(caps->name), "%s", dev->props.name);
    snprintf(caps->arch, sizeof(caps->arch), "%s", dev->props.gcnArchName);
    caps->num_compute_units = (uint32_t)dev->props.multiProcessorCount;
    caps->wavefront_size = (uint32_t)dev->props.warpSize;
    caps->clock_mhz = (uint32_t)(dev->props.clockRate / 1000);
    caps->mem_clock_mhz = (uint32_t)(dev->props.memoryClockRate / 1000);
    caps->mem_bus_bits = (uint32_t)dev->props.memoryBusWidth;
    caps->l2_cache_kb = (uint32_t)(dev->props.l2CacheSize / 1024);
    caps->lds_kb_per_cu = (uint32_t)(dev->props.maxSharedMemoryPerMultiProcessor / 1024);
    caps->total_mem_bytes = (uint64_t)dev->props.totalGlobalMem;
    // published MI355X peaks (dense): HBM3E 8 TB/s, fp16 MFMA 2.5 PFLOP/s, int8 MFMA 5.0 POP/s
    caps->mem_bw_gbps = 8000.0f;
    caps->peak_tflops_fp16 = 2500.0f;
    caps->peak_tops_int8 = 5000.0f;
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_graph_begin_capture(marmot_hip_device_t *dev) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "graph_begin_capture: null device");
    }
    if (dev->capturing) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "graph_begin_capture: a capture is already active");
    }
    if (dev->branch >= 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION,
                         "graph_begin_capture: a branch section is open; join it first");
    }
    MH_HIP(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeThreadLocal));
    dev->capturing = true;
    return MARMOT_HIP_SUCCESS;
}

// Parks the open branch's workspace and makes branch `to` the open one (its stream, its workspace).
static void branch_switch(marmot_hip_device *dev, int to) {
    dev->branch_workspace[dev->branch].ptr = dev->workspace;
    dev->branch_workspace[dev->branch].bytes = dev->workspace_bytes;
    dev->workspace = dev->branch_workspace[to].ptr;
    dev->workspace_bytes = dev->branch_workspace[to].bytes;
    dev->branch_workspace[to].ptr = nullptr;
    dev->branch_workspace[to].bytes = 0;
    dev->branch = to;
    dev->stream = to == 0 ? dev->main_stream : dev->side_streams[to - 1];
}

int marmot_hip_branch_begin(marmot_hip_device_t *dev) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "branch_begin: null device");
    }
    if (dev->branch >= 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "branch_begin: a branch section is already open");
    }
    if (dev->fork_event == nullptr) {
        if (dev->capturing) {
            return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION,
                             "branch_begin: the first section of a device object makes its side streams and cannot be "
                             "recorded; run one section eagerly before capturing");
        }
        MH_HIP(hipSetDevice(dev->device_index));
        if (branches_init(dev) != 0) {
            return MARMOT_HIP_ERROR_BACKEND_INIT_FAILED;
        }
    }
    MH_HIP(hipEventRecord(dev->fork_event, dev->main_stream));
    dev->branch = 0;
    dev->branches_used = 1;
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_branch_next(marmot_hip_device_t *dev) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "branch_next: null device");
    }
    if (dev->branch < 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "branch_next: no branch section is open");
    }
    if (dev->branch + 1 >= marmot_hip_device::MAX_BRANCHES) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "branch_next: a section holds at most %d branches",
                         marmot_hip_device::MAX_BRANCHES);
    }
    const int to = dev->branch + 1;
    // the new branch starts behind everything that was enqueued before the section
    MH_HIP(hipStreamWaitEvent(dev->side_streams[to - 1], dev->fork_event, 0));
    branch_switch(dev, to);
    dev->branches_used = to + 1;
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_branch_join(marmot_hip_device_t *dev) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "branch_join: null device");
    }
    if (dev->branch < 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "branch_join: no branch section is open");
    }
    const int used = dev->branches_used;
    branch_switch(dev, 0);
    dev->branch = -1;
    dev->branches_used = 0;
    for (int i = 1; i < used; ++i) {
        MH_HIP(hipEventRecord(dev->side_done[i - 1], dev->side_streams[i - 1]));
        MH_HIP(hipStreamWaitEvent(dev->main_stream, dev->side_done[i - 1], 0));
    }
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_rows_plan_probe(int kernel, uint32_t compute_units, size_t N, size_t K, size_t M, int weights, int packed,
                               uint32_t *out, size_t n_out) {
    if (out == nullptr || compute_units == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "rows_plan_probe: null output or no compute units");
    }
    const bool ok = kernel == 0   ? mh::rows_plan_probe(compute_units, N, K, M, weights, out, n_out)
                    : kernel == 1 ? mh::mmq_rows_plan_probe(compute_units, N, K, M, weights, packed != 0, out, n_out)
                                  : false;
    return ok ? MARMOT_HIP_SUCCESS : MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
}

int marmot_hip_timeline_attach(marmot_hip_device_t *dev, void *d_marks, size_t bytes) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "timeline_attach: null device");
    }
#if defined(MH_TIMELINE)
    if (d_marks != nullptr && ((((uintptr_t)d_marks) & 7) != 0 || bytes / 8 > 0xffffffffull)) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "timeline_attach: the buffer must be 8-byte aligned");
    }
    dev->timeline = (unsigned long long *)d_marks;
    dev->timeline_words = d_marks != nullptr ? (uint32_t)(bytes / 8) : 0;
    return MARMOT_HIP_SUCCESS;
#else
    (void)d_marks;
    (void)bytes;
    return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "timeline_attach: this library was built without -DMH_TIMELINE");
#endif
}

size_t marmot_hip_graph_max_nodes(void) {
    return MARMOT_HIP_GRAPH_MAX_NODES;
}

int marmot_hip_graph_end_capture(marmot_hip_device_t *dev, void **out_graph_exec) {
    if (dev == nullptr || out_graph_exec == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "graph_end_capture: null argument");
    }
    *out_graph_exec = nullptr;
    if (!dev->capturing) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "graph_end_capture: no capture is active");
    }
    if (dev->branch >= 0) {
        // the side streams have not joined the main stream yet: ending the capture now would fail inside the runtime
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION,
                         "graph_end_capture: a branch section is open; call marmot_hip_branch_join first");
    }
    dev->capturing = false;
    hipGraph_t graph = nullptr;
    MH_HIP(hipStreamEndCapture(dev->stream, &graph));
    size_t nodes = 0;
    hipError_t e = hipGraphGetNodes(graph, nullptr, &nodes);
    dev->last_capture_nodes = e == hipSuccess ? nodes : 0;
    if (e == hipSuccess && nodes > MARMOT_HIP_GRAPH_MAX_NODES) {
        (void)hipGraphDestroy(graph);
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION,
                         "graph_end_capture: %zu nodes were recorded, the limit is %d per graph: capture the batch in "
                         "several graphs", nodes, MARMOT_HIP_GRAPH_MAX_NODES);
    }
    hipGraphExec_t exec = nullptr;
    if (e == hipSuccess) {
        e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    }
    (void)hipGraphDestroy(graph);
    MH_HIP(e);
    ++dev->live_graphs;
    *out_graph_exec = (void *)exec;
    return MARMOT_HIP_SUCCESS;
}

size_t marmot_hip_graph_last_capture_nodes(marmot_hip_device_t *dev) {
    return dev != nullptr ? dev->last_capture_nodes : 0;
}

int marmot_hip_graph_launch(marmot_hip_device_t *dev, void *graph_exec) {
    if (dev == nullptr || graph_exec == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "graph_launch: null argument");
    }
    MH_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, dev->stream));
    return MARMOT_HIP_SUCCESS;
}

void marmot_hip_graph_destroy(marmot_hip_device_t *dev, void *graph_exec) {
    if (graph_exec == nullptr) {
        return;
    }
    if (dev != nullptr) {
        (void)hipStreamSynchronize(dev->stream);  // a replay may still be running
    }
    (void)hipGraphExecDestroy((hipGraphExec_t)graph_exec);
    if (dev != nullptr && dev->live_graphs > 0 && --dev->live_graphs == 0) {
        for (void *w : dev->retired_workspaces) {
            (void)hipFree(w);
        }
        dev->retired_workspaces.clear();
    }
}

int marmot_hip_event_create(marmot_hip_device_t *dev, void **out_event) {
    if (dev == nullptr || out_event == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "event_create: null argument");
    }
    hipEvent_t ev;
    MH_HIP(hipEventCreate(&ev));
    *out_event = (void *)ev;
    return MARMOT_HIP_SUCCESS;
}

void marmot_hip_event_destroy(marmot_hip_device_t *dev, void *event) {
    (void)dev;
    if (event != nullptr) {
        (void)hipEventDestroy((hipEvent_t)event);
    }
}

int marmot_hip_event_record(marmot_hip_device_t *dev, void *event) {
    if (dev == nullptr || event == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "event_record: null argument");
    }
    MH_HIP(hipEventRecord((hipEvent_t)event, dev->stream));
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_event_elapsed_ms(marmot_hip_device_t *dev, void *start, void *stop, float *out_ms) {
    if (dev == nullptr || start == nullptr || stop == nullptr || out_ms == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "event_elapsed: null argument");
    }
    MH_HIP(hipEventSynchronize((hipEvent_t)stop));
    MH_HIP(hipEventElapsedTime(out_ms, (hipEvent_t)start, (hipEvent_t)stop));
    return MARMOT_HIP_SUCCESS;
}

} // extern "C"

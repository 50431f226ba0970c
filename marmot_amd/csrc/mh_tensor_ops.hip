// The small tensor operations a GGUF model graph places around the quantized linears, so that a whole graph can stay
// on the device between its first and last node:
//   * unary activations GELU (erf form), GELU (tanh form), SiLU on FLOAT32 or FLOAT16 values (gelu_scalar,
//     gelu_tanh_scalar, silu_scalar_fn: src/backends/cpu/ops/unary/scalar/unary_scalar.c:201-218; FLOAT16 values are
//     widened, computed in fp32 and rounded back);
//   * softmax of FLOAT32 values along one axis (softmax_f32_scalar, src/backends/cpu/ops/softmax/scalar/
//     softmax_f32_scalar.c:30-83: maximum, exp(x - max) flushed to zero at or below -88, sum, one multiplication by
//     1 / sum);
//   * conversions between FLOAT32, FLOAT16 and BFLOAT16 (src/backends/cpu/ops/convert/dtype_convert.c:17-130): to
//     FLOAT16 and BFLOAT16 round to nearest even, between the two 16-bit types through FLOAT32
//     (src/utils/dtype_ref.c:86-114). The reference's FLOAT32 -> FLOAT16 loop rounds to nearest even in its vector
//     body and truncates the last n % 8 (n % 4) elements in its scalar tail (dtype_ref.c:14-50); every element is
//     rounded to nearest even here;
//   * gather_rows (cpu_gather_rows, src/backends/cpu/ops/tensor_ops/tensor_ops.c:464-547): rows of a 2-D tensor picked
//     by INT32 or UINT32 indices, any row strides;
//   * slice (cpu_slice, tensor_ops.c:401-462): a box [starts, starts + sizes) of a contiguous tensor of up to 8
//     dimensions copied into a contiguous output.
// The copies are bit-exact; the activations and the softmax differ from the CPU code only through the device's expf /
// erff / tanhf and, for softmax rows of more than 128 values or with an inner stride, the order in which a row's
// exponentials are added (256 threads, fixed tree; shorter contiguous rows are summed in index order by one thread).
#include "mh_common.h"

#include <math.h>

namespace mh {

// ------------------------------------------------------------------ 16-bit types
// marmot_f32_to_bf16_ref / marmot_bf16_to_f32_ref (src/utils/dtype_ref.c:86-104): round to nearest even on the bits
__device__ __forceinline__ uint16_t to_bf16(float v) {
    const uint32_t bits = __float_as_uint(v);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float from_bf16(uint16_t h) {
    return __uint_as_float((uint32_t)h << 16);
}

template <int DTYPE>
__device__ __forceinline__ float load_as_f32(const void *p, size_t i) {
    if constexpr (DTYPE == MARMOT_HIP_DTYPE_F32) {
        return ((const float *)p)[i];
    } else if constexpr (DTYPE == MARMOT_HIP_DTYPE_F16) {
        return h2f(((const uint16_t *)p)[i]);
    } else {
        return from_bf16(((const uint16_t *)p)[i]);
    }
}
template <int DTYPE>
__device__ __forceinline__ void store_from_f32(void *p, size_t i, float v) {
    if constexpr (DTYPE == MARMOT_HIP_DTYPE_F32) {
        ((float *)p)[i] = v;
    } else if constexpr (DTYPE == MARMOT_HIP_DTYPE_F16) {
        ((uint16_t *)p)[i] = f2h(v);
    } else {
        ((uint16_t *)p)[i] = to_bf16(v);
    }
}

// ------------------------------------------------------------------ unary activations
template <int OP>
__device__ __forceinline__ float unary_value(float x) {
    if constexpr (OP == MARMOT_HIP_UNARY_GELU) {
        return x * 0.5f * (1.0f + erff(x * 0.7071067811865475f));
    } else if constexpr (OP == MARMOT_HIP_UNARY_GELU_TANH) {
        const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
        return 0.5f * x * (1.0f + tanhf(inner));
    } else {
        return x / (1.0f + expf(-x));
    }
}

template <int OP, int DTYPE>
__global__ __launch_bounds__(256) void k_unary(const void *x, void *out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        store_from_f32<DTYPE>(out, i, unary_value<OP>(load_as_f32<DTYPE>(x, i)));
    }
}

// ------------------------------------------------------------------ softmax
// One workgroup of 256 threads per softmax row (outer index o, inner index j): elements x[(o * axis + a) * inner + j].
// Every thread folds its elements a = t, t + 256, ... in index order; wavefront butterflies and a fixed (0 + 1) +
// (2 + 3) tree combine the 256 partial results. The exponentials are kept in the output between the passes like the
// reference does.
__device__ __forceinline__ float block_reduce(float v, float *red, bool is_max) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off);
        v = is_max ? fmaxf(v, o) : v + o;
    }
    __syncthreads();  // red may still be read from the previous reduction
    if (lane == 0) {
        red[wave] = v;
    }
    __syncthreads();
    return is_max ? fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) : (red[0] + red[1]) + (red[2] + red[3]);
}

// FLOAT16 / BFLOAT16 rows follow softmax_f16_scalar / softmax_bf16_scalar (scalar/softmax_misc_scalar.c:4-122): maximum
// and sum in FLOAT32, every exponential rounded to the tensor's type when it is stored (the sum takes the unrounded
// one), and the stored value, widened again, times 1 / sum rounded a second time.
template <int DTYPE>
__global__ __launch_bounds__(256) void k_softmax(const void *x, void *out, size_t axis, size_t inner) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const size_t o = row / inner, j = row - o * inner;
    const size_t base = o * axis * inner + j;
    float m = -INFINITY;
    for (size_t a = threadIdx.x; a < axis; a += 256) {
        m = fmaxf(m, load_as_f32<DTYPE>(x, base + a * inner));
    }
    m = block_reduce(m, red, true);
    float sum = 0.0f;
    for (size_t a = threadIdx.x; a < axis; a += 256) {
        const float diff = load_as_f32<DTYPE>(x, base + a * inner) - m;
        const float e = diff <= -88.0f ? 0.0f : expf(diff);  // softmax_safe_expf, softmax_internal.h:14-26
        store_from_f32<DTYPE>(out, base + a * inner, e);
        sum += e;
    }
    sum = block_reduce(sum, red, false);
    const float inv = 1.0f / sum;
    for (size_t a = threadIdx.x; a < axis; a += 256) {
        // written by this thread above
        store_from_f32<DTYPE>(out, base + a * inner, load_as_f32<DTYPE>(out, base + a * inner) * inv);
    }
}

// Short rows that lie contiguously (inner == 1, at most SOFTMAX_SMALL values, e.g. router logits over the experts): one
// thread per row, everything in index order like the scalar CPU loop.
constexpr size_t SOFTMAX_SMALL = 128;
template <int DTYPE>
__global__ __launch_bounds__(64) void k_softmax_small(const void *x, void *out, size_t rows, size_t axis) {
    const size_t row = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (row >= rows) {
        return;
    }
    const size_t base = row * axis;
    // FLOAT32 rows start from their first value, the 16-bit rows from -FLT_MAX (softmax_find_max_f16,
    // softmax_internal.h:119-150): the same maximum unless a row holds nothing above -FLT_MAX
    float m = DTYPE == MARMOT_HIP_DTYPE_F32 ? load_as_f32<DTYPE>(x, base) : -3.402823466e+38f;
    for (size_t i = DTYPE == MARMOT_HIP_DTYPE_F32 ? 1 : 0; i < axis; ++i) {
        const float v = load_as_f32<DTYPE>(x, base + i);
        m = v > m ? v : m;
    }
    float sum = 0.0f;
    for (size_t i = 0; i < axis; ++i) {
        const float diff = load_as_f32<DTYPE>(x, base + i) - m;
        const float e = diff <= -88.0f ? 0.0f : expf(diff);
        store_from_f32<DTYPE>(out, base + i, e);
        sum += e;
    }
    const float inv = 1.0f / sum;
    for (size_t i = 0; i < axis; ++i) {
        store_from_f32<DTYPE>(out, base + i, load_as_f32<DTYPE>(out, base + i) * inv);
    }
}

template <int DTYPE>
static int launch_softmax(marmot_hip_device *dev, const void *d_x, size_t rows, size_t axis, size_t inner, void *d_out) {
    if (inner == 1 && axis <= SOFTMAX_SMALL) {
        hipLaunchKernelGGL(k_softmax_small<DTYPE>, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, dev->stream, d_x,
                           d_out, rows, axis);
    } else {
        hipLaunchKernelGGL(k_softmax<DTYPE>, dim3((unsigned)rows), dim3(256), 0, dev->stream, d_x, d_out, axis, inner);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

// ------------------------------------------------------------------ conversion
template <int DST, int SRC>
__global__ __launch_bounds__(256) void k_convert(void *__restrict__ dst, const void *__restrict__ src, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        if constexpr (DST == SRC && DST != MARMOT_HIP_DTYPE_F32) {
            ((uint16_t *)dst)[i] = ((const uint16_t *)src)[i];  // equal types: a copy, NaN payloads included
        } else {
            store_from_f32<DST>(dst, i, load_as_f32<SRC>(src, i));
        }
    }
}

// ------------------------------------------------------------------ gather_rows
// One workgroup row per output row (blockIdx.y), UNIT-byte pieces along the row. An index outside [0, rows_in) raises
// the flag (when there is one) and leaves the row zeroed.
template <typename UNIT>
__global__ __launch_bounds__(256) void k_gather_rows(const uint8_t *__restrict__ x, size_t rows_in, size_t row_units,
                                                     size_t in_stride, const void *__restrict__ idx, int idx_signed,
                                                     size_t idx_stride, uint8_t *__restrict__ out, size_t out_stride,
                                                     int *flag) {
    const size_t r = blockIdx.y;
    long long row;
    if (idx_signed) {
        row = ((const int32_t *)idx)[r * idx_stride];
    } else {
        row = ((const uint32_t *)idx)[r * idx_stride];
    }
    const bool ok = row >= 0 && (size_t)row < rows_in;
    if (!ok && flag != nullptr && threadIdx.x == 0 && blockIdx.x == 0) {
        *flag = 1;
    }
    const UNIT *src = (const UNIT *)(x + (ok ? (size_t)row : 0) * in_stride);
    UNIT *dst = (UNIT *)(out + r * out_stride);
    for (size_t c = (size_t)blockIdx.x * 256 + threadIdx.x; c < row_units; c += (size_t)gridDim.x * 256) {
        UNIT v = src[c];
        if (!ok) {
            v = UNIT{};
        }
        dst[c] = v;
    }
}

// ------------------------------------------------------------------ slice
struct SliceParams {
    int ndim;
    size_t n;             // elements of the output
    size_t sizes[8];      // output shape
    size_t in_stride[8];  // contiguous strides of the input, in elements
    size_t in_first;      // element offset of starts[] in the input
};

template <typename UNIT>
__global__ __launch_bounds__(256) void k_slice(const UNIT *__restrict__ x, UNIT *__restrict__ out, const SliceParams p) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < p.n; i += (size_t)gridDim.x * blockDim.x) {
        size_t rest = i, src = p.in_first;
        for (int d = p.ndim - 1; d >= 0; --d) {
            const size_t q = rest / p.sizes[d], c = rest - q * p.sizes[d];
            src += c * p.in_stride[d];
            rest = q;
        }
        out[i] = x[src];
    }
}

static unsigned grid_for(size_t n) {
    const size_t g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

template <int OP>
static bool launch_unary(marmot_hip_device *dev, int dtype, const void *x, void *out, size_t n) {
    const dim3 grid(grid_for(n)), block(256);
    if (dtype == MARMOT_HIP_DTYPE_F32) {
        hipLaunchKernelGGL((k_unary<OP, MARMOT_HIP_DTYPE_F32>), grid, block, 0, dev->stream, x, out, n);
    } else if (dtype == MARMOT_HIP_DTYPE_F16) {
        hipLaunchKernelGGL((k_unary<OP, MARMOT_HIP_DTYPE_F16>), grid, block, 0, dev->stream, x, out, n);
    } else {
        return false;
    }
    return true;
}

template <int DST>
static bool launch_convert_to(marmot_hip_device *dev, void *dst, const void *src, int src_dtype, size_t n) {
    const dim3 grid(grid_for(n)), block(256);
    switch (src_dtype) {
    case MARMOT_HIP_DTYPE_F32:
        hipLaunchKernelGGL((k_convert<DST, MARMOT_HIP_DTYPE_F32>), grid, block, 0, dev->stream, dst, src, n);
        return true;
    case MARMOT_HIP_DTYPE_F16:
        hipLaunchKernelGGL((k_convert<DST, MARMOT_HIP_DTYPE_F16>), grid, block, 0, dev->stream, dst, src, n);
        return true;
    case MARMOT_HIP_DTYPE_BF16:
        hipLaunchKernelGGL((k_convert<DST, MARMOT_HIP_DTYPE_BF16>), grid, block, 0, dev->stream, dst, src, n);
        return true;
    default:
        return false;
    }
}

} // namespace mh

using namespace mh;

extern "C" {

int marmot_hip_unary(marmot_hip_device_t *dev, int op, const void *d_x, int dtype, size_t n, void *d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (dtype != MARMOT_HIP_DTYPE_F32 && dtype != MARMOT_HIP_DTYPE_F16) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "unary: values must be FLOAT32 or FLOAT16");
    }
    if (n == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    bool ok;
    switch (op) {
    case MARMOT_HIP_UNARY_GELU:
        ok = launch_unary<MARMOT_HIP_UNARY_GELU>(dev, dtype, d_x, d_out, n);
        break;
    case MARMOT_HIP_UNARY_GELU_TANH:
        ok = launch_unary<MARMOT_HIP_UNARY_GELU_TANH>(dev, dtype, d_x, d_out, n);
        break;
    case MARMOT_HIP_UNARY_SILU:
        ok = launch_unary<MARMOT_HIP_UNARY_SILU>(dev, dtype, d_x, d_out, n);
        break;
    default:
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "unary: unknown operation %d", op);
    }
    if (!ok) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "unary: unsupported dtype %d", dtype);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_softmax_typed(marmot_hip_device_t *dev, int dtype, const void *d_x, size_t outer, size_t axis,
                             size_t inner, void *d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (axis == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Softmax axis dimension must be non-zero");
    }
    if (dtype != MARMOT_HIP_DTYPE_F32 && dtype != MARMOT_HIP_DTYPE_F16 && dtype != MARMOT_HIP_DTYPE_BF16) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "softmax: unsupported dtype %d", dtype);
    }
    const size_t rows = outer * inner;
    if (rows == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (rows > 0x7fffffffull) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "softmax: more than 2^31 - 1 rows");
    }
    MH_HIP(hipSetDevice(dev->device_index));
    if (dtype == MARMOT_HIP_DTYPE_F16) {
        return launch_softmax<MARMOT_HIP_DTYPE_F16>(dev, d_x, rows, axis, inner, d_out);
    }
    if (dtype == MARMOT_HIP_DTYPE_BF16) {
        return launch_softmax<MARMOT_HIP_DTYPE_BF16>(dev, d_x, rows, axis, inner, d_out);
    }
    return launch_softmax<MARMOT_HIP_DTYPE_F32>(dev, d_x, rows, axis, inner, d_out);
}

int marmot_hip_softmax(marmot_hip_device_t *dev, const float *d_x, size_t outer, size_t axis, size_t inner,
                       float *d_out) {
    return marmot_hip_softmax_typed(dev, MARMOT_HIP_DTYPE_F32, d_x, outer, axis, inner, d_out);
}

int marmot_hip_convert(marmot_hip_device_t *dev, void *d_dst, int dst_dtype, const void *d_src, int src_dtype,
                       size_t n) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_dst == nullptr || d_src == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (n == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    bool ok;
    switch (dst_dtype) {
    case MARMOT_HIP_DTYPE_F32:
        ok = launch_convert_to<MARMOT_HIP_DTYPE_F32>(dev, d_dst, d_src, src_dtype, n);
        break;
    case MARMOT_HIP_DTYPE_F16:
        ok = launch_convert_to<MARMOT_HIP_DTYPE_F16>(dev, d_dst, d_src, src_dtype, n);
        break;
    case MARMOT_HIP_DTYPE_BF16:
        ok = launch_convert_to<MARMOT_HIP_DTYPE_BF16>(dev, d_dst, d_src, src_dtype, n);
        break;
    default:
        ok = false;
        break;
    }
    if (!ok) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "convert: %d -> %d is not among FLOAT32 / FLOAT16 / BFLOAT16",
                         src_dtype, dst_dtype);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_gather_rows(marmot_hip_device_t *dev, const void *d_x, size_t rows_in, size_t row_bytes,
                           size_t in_stride_bytes, const void *d_idx, int idx_dtype, size_t idx_stride, size_t rows_out,
                           void *d_out, size_t out_stride_bytes) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_idx == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (idx_dtype != MARMOT_HIP_DTYPE_I32 && idx_dtype != MARMOT_HIP_DTYPE_U32) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "gather_rows indices dtype unsupported");
    }
    if (rows_out == 0 || row_bytes == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (rows_in == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "gather_rows index out of range");
    }
    if (rows_out > 65535) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "gather_rows: more than 65535 rows per call");
    }
    MH_HIP(hipSetDevice(dev->device_index));
    // Out-of-range indices are reported through a device flag read back after the launch; that takes a stream
    // synchronization and is skipped while the stream is being captured into a graph (the rows are zeroed then).
    int *flag = nullptr;
    if (!dev->capturing) {
        void *ws = nullptr;
        const int st = workspace_reserve(dev, 256, &ws);
        if (st != MARMOT_HIP_SUCCESS) {
            return st;
        }
        flag = (int *)ws;
        MH_HIP(hipMemsetAsync(flag, 0, sizeof(int), dev->stream));
    }
    const int idx_signed = idx_dtype == MARMOT_HIP_DTYPE_I32;
    const uintptr_t align = (uintptr_t)d_x | (uintptr_t)d_out | row_bytes | in_stride_bytes | out_stride_bytes;
    const uint8_t *x = (const uint8_t *)d_x;
    uint8_t *out = (uint8_t *)d_out;
    if ((align & 15) == 0) {
        const size_t units = row_bytes / 16;
        const dim3 grid((unsigned)((units + 255) / 256 > 64 ? 64 : (units + 255) / 256), (unsigned)rows_out);
        hipLaunchKernelGGL((k_gather_rows<uint4>), grid, dim3(256), 0, dev->stream, x, rows_in, units, in_stride_bytes,
                           d_idx, idx_signed, idx_stride, out, out_stride_bytes, flag);
    } else if ((align & 3) == 0) {
        const size_t units = row_bytes / 4;
        const dim3 grid((unsigned)((units + 255) / 256 > 64 ? 64 : (units + 255) / 256), (unsigned)rows_out);
        hipLaunchKernelGGL((k_gather_rows<uint32_t>), grid, dim3(256), 0, dev->stream, x, rows_in, units,
                           in_stride_bytes, d_idx, idx_signed, idx_stride, out, out_stride_bytes, flag);
    } else if ((align & 1) == 0) {
        const size_t units = row_bytes / 2;
        const dim3 grid((unsigned)((units + 255) / 256 > 64 ? 64 : (units + 255) / 256), (unsigned)rows_out);
        hipLaunchKernelGGL((k_gather_rows<uint16_t>), grid, dim3(256), 0, dev->stream, x, rows_in, units,
                           in_stride_bytes, d_idx, idx_signed, idx_stride, out, out_stride_bytes, flag);
    } else {
        const size_t units = row_bytes;
        const dim3 grid((unsigned)((units + 255) / 256 > 64 ? 64 : (units + 255) / 256), (unsigned)rows_out);
        hipLaunchKernelGGL((k_gather_rows<uint8_t>), grid, dim3(256), 0, dev->stream, x, rows_in, units,
                           in_stride_bytes, d_idx, idx_signed, idx_stride, out, out_stride_bytes, flag);
    }
    MH_HIP(hipGetLastError());
    if (flag != nullptr) {
        int host_flag = 0;
        MH_HIP(hipMemcpyAsync(&host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, dev->stream));
        MH_HIP(hipStreamSynchronize(dev->stream));
        if (host_flag != 0) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "gather_rows index out of range");
        }
    }
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_slice(marmot_hip_device_t *dev, const void *d_x, size_t elem_size, int ndim, const size_t *in_shape,
                     const size_t *starts, const size_t *sizes, void *d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_out == nullptr || in_shape == nullptr || starts == nullptr || sizes == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Null pointer in slice");
    }
    if (ndim < 1 || ndim > 8) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "slice: 1 to 8 dimensions");
    }
    if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "slice: element size must be 1, 2, 4 or 8 bytes");
    }
    SliceParams p = {};
    p.ndim = ndim;
    p.n = 1;
    size_t stride = 1;
    for (int d = ndim - 1; d >= 0; --d) {
        if (starts[d] > in_shape[d] || sizes[d] > in_shape[d] - starts[d]) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "slice: box outside the input in dimension %d", d);
        }
        p.sizes[d] = sizes[d];
        p.in_stride[d] = stride;
        p.in_first += starts[d] * stride;
        p.n *= sizes[d];
        stride *= in_shape[d];
    }
    if (p.n == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    const dim3 grid(grid_for(p.n)), block(256);
    switch (elem_size) {
    case 1:
        hipLaunchKernelGGL((k_slice<uint8_t>), grid, block, 0, dev->stream, (const uint8_t *)d_x, (uint8_t *)d_out, p);
        break;
    case 2:
        hipLaunchKernelGGL((k_slice<uint16_t>), grid, block, 0, dev->stream, (const uint16_t *)d_x, (uint16_t *)d_out, p);
        break;
    case 4:
        hipLaunchKernelGGL((k_slice<uint32_t>), grid, block, 0, dev->stream, (const uint32_t *)d_x, (uint32_t *)d_out, p);
        break;
    default:
        hipLaunchKernelGGL((k_slice<uint64_t>), grid, block, 0, dev->stream, (const uint64_t *)d_x, (uint64_t *)d_out, p);
        break;
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

} // extern "C"

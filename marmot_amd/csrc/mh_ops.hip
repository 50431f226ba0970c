// The fp32 operations that sit between the quantized linears of a decoder layer, and their fused forms that hand the
// next linear its activations already quantized:
//   * RMS normalization (cpu_rmsnorm_impl / cpu_rmsnorm_gemma_impl, normalization_dispatch.c:129-181,
//     normalization_scalar.c:469-510, 780-791): out = (x [+ residual]) * inv_rms * (weight + weight_offset),
//     inv_rms = 1 / sqrt(mean((x [+ residual])^2) + eps); optionally the rows are also written as packed Q8_K / Q8_0
//     activations (the input of the q/k/v or gate/up projections), one launch for both.
//   * gated products swiglu / geglu (cpu_swiglu_f32_scalar / cpu_geglu_f32_scalar, elementwise_f32_scalar.c:11-20,
//     147-214), optionally straight into packed activations (the input of the down projection);
//   * residual add (cpu_add_f32, elementwise_f32_scalar.c);
//   * rotary embedding of fp32 / fp16 rows (cpu_rope, src/backends/cpu/ops/rope/rope_dispatch.c:145-372).
// fp32 arithmetic per element is the reference's expression, rounded operation by operation (-ffp-contract=off); the
// sum of squares of a row is formed by 256 threads (strided partial sums, then a fixed-order tree), not sequentially,
// so inv_rms can differ from the scalar CPU loop in the last bits.
#include "mh_actquant.h"

#include <math.h>

namespace mh {

struct RmsNormParams {
    const float *x;
    const float *residual;  // nullptr: none
    const float *weight;    // nullptr: none
    float weight_offset;
    float eps;
    size_t rows, cols;
    float *out;  // nullptr: packed output only
    int act_kind;  // 0: no packed output, else MARMOT_HIP_KIND_Q8_K / MARMOT_HIP_KIND_Q8_0
    ActScratch packed;
};

// One workgroup of 256 threads per row. The sum of squares: every thread adds its own values in index order, the 64
// partial sums of a wavefront meet in a butterfly, the four wavefront sums are added as (0 + 1) + (2 + 3).
__device__ __forceinline__ float rms_total(float sum, float *red, int lane, int wave) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        sum += __shfl_xor(sum, off);
    }
    if (lane == 0) {
        red[wave] = sum;
    }
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// Rows of up to RMS_ROW_CHUNKS x 1024 values whose length is a multiple of 4: the row is read once, with 16-byte loads
// that are all in flight together, and stays in registers between the sum and the scaling. Thread t holds values
// 4 (t + 256 j) .. + 3 for j = 0, 1, ...: for wavefront w and lane l that is block w + 4 j, values 4 l .. 4 l + 3 of a
// 256-value block, the order in which the Q8_K packer takes them.
constexpr int RMS_ROW_CHUNKS = 8;

template <int ACT>
__global__ __launch_bounds__(256) void k_rms_norm_row_in_registers(const RmsNormParams p) {
    static_assert(ACT == 0 || ACT == MARMOT_HIP_KIND_Q8_K, "the Q8_0 packer takes single values");
    __shared__ float red[4];
    warm_kernel_arguments<sizeof(RmsNormParams), sizeof(RmsNormParams)>();
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float4 *x = (const float4 *)(p.x + row * p.cols);
    const float4 *res = p.residual != nullptr ? (const float4 *)(p.residual + row * p.cols) : nullptr;
    const float4 *weight = (const float4 *)p.weight;
    const int chunks = (int)(p.cols / 4);
    float4 v[RMS_ROW_CHUNKS], w[RMS_ROW_CHUNKS];
#pragma unroll
    for (int j = 0; j < RMS_ROW_CHUNKS; ++j) {
        const int c = tid + 256 * j;
        v[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        w[j] = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
        if (c < chunks) {
            v[j] = x[c];
            if (weight != nullptr) {
                w[j] = weight[c];
            }
        }
    }
    if (res != nullptr) {
#pragma unroll
        for (int j = 0; j < RMS_ROW_CHUNKS; ++j) {
            const int c = tid + 256 * j;
            if (c < chunks) {
                const float4 r = res[c];
                v[j].x += r.x;
                v[j].y += r.y;
                v[j].z += r.z;
                v[j].w += r.w;
            }
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < RMS_ROW_CHUNKS; ++j) {
        sum += v[j].x * v[j].x;
        sum += v[j].y * v[j].y;
        sum += v[j].z * v[j].z;
        sum += v[j].w * v[j].w;
    }
    const float total = rms_total(sum, red, lane, wave);
    const float mean_sq = total / (float)p.cols;
    const float inv_rms = 1.0f / sqrtf(mean_sq + p.eps);
#pragma unroll
    for (int j = 0; j < RMS_ROW_CHUNKS; ++j) {
        const int c = tid + 256 * j;
        float4 o;
        o.x = v[j].x * inv_rms;
        o.y = v[j].y * inv_rms;
        o.z = v[j].z * inv_rms;
        o.w = v[j].w * inv_rms;
        if (weight != nullptr) {
            o.x = o.x * (w[j].x + p.weight_offset);
            o.y = o.y * (w[j].y + p.weight_offset);
            o.z = o.z * (w[j].z + p.weight_offset);
            o.w = o.w * (w[j].w + p.weight_offset);
        }
        if (c >= chunks) {
            o = make_float4(0.0f, 0.0f, 0.0f, 0.0f);  // beyond the row, whatever inv_rms is
        } else if (p.out != nullptr) {
            ((float4 *)(p.out + row * p.cols))[c] = o;
        }
        if constexpr (ACT == MARMOT_HIP_KIND_Q8_K) {
            const size_t b = (size_t)wave + 4 * (size_t)j;  // uniform over the wavefront
            if (b < p.packed.nb) {
                const float q[4] = {o.x, o.y, o.z, o.w};
                q8k_block_store<false>(q, lane, row, b, p.packed.nb, nullptr, p.packed);
            }
        }
    }
}

// Any row length: the row is read twice (the second time from the caches). Results are bit-identical to the register
// kernel's where both apply.
template <int ACT>
__global__ __launch_bounds__(256) void k_rms_norm(const RmsNormParams p) {
    __shared__ float red[4];
    warm_kernel_arguments<sizeof(RmsNormParams), sizeof(RmsNormParams)>();
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *x = p.x + row * p.cols;
    const float *res = p.residual != nullptr ? p.residual + row * p.cols : nullptr;
    // the same partition of the row as the register kernel: thread t adds values 4 (t + 256 j) .. + 3, j = 0, 1, ...
    float sum = 0.0f;
    for (size_t c = tid; 4 * c < p.cols; c += 256) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const size_t i = 4 * c + e;
            if (i < p.cols) {
                float v = x[i];
                if (res != nullptr) {
                    v += res[i];
                }
                sum += v * v;
            }
        }
    }
    const float total = rms_total(sum, red, lane, wave);
    const float mean_sq = total / (float)p.cols;
    const float inv_rms = 1.0f / sqrtf(mean_sq + p.eps);
    auto value = [&](size_t i) {
        float v = x[i];
        if (res != nullptr) {
            v += res[i];
        }
        v = v * inv_rms;
        if (p.weight != nullptr) {
            v = v * (p.weight[i] + p.weight_offset);
        }
        return v;
    };
    if constexpr (ACT == 0) {
        for (size_t i = tid; i < p.cols; i += 256) {
            p.out[row * p.cols + i] = value(i);
        }
    } else if constexpr (ACT == MARMOT_HIP_KIND_Q8_K) {
        // wavefront w quantizes blocks w, w + 4, ...: 4 consecutive values per lane
        const size_t nb = p.packed.nb;
        for (size_t b = wave; b < nb; b += 4) {
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const size_t col = b * QK_K + (size_t)lane * 4 + i;
                v[i] = col < p.cols ? value(col) : 0.0f;
                if (p.out != nullptr && col < p.cols) {
                    p.out[row * p.cols + col] = v[i];
                }
            }
            q8k_block_store<false>(v, lane, row, b, nb, nullptr, p.packed);
        }
    } else {
        // 32 lanes per block: thread t quantizes value t % 32 of blocks t / 32, t / 32 + 8, ...
        const size_t nb = p.packed.nb;
        const int lane32 = tid & 31;
        for (size_t b = tid >> 5; b < nb; b += 8) {
            const size_t col = b * QK + lane32;
            const float v = col < p.cols ? value(col) : 0.0f;
            if (p.out != nullptr && col < p.cols) {
                p.out[row * p.cols + col] = v;
            }
            q8_0_block_store<false>(v, col < p.cols, lane32, row, b, nb, nullptr, p.packed);
        }
    }
}

// out[r][c] = act(gate[r][c]) * up[r][c]; rows of the three arrays may be strided (elements)
template <bool GEGLU>
__device__ __forceinline__ float glu_value(float g, float u) {
    float a;
    if constexpr (GEGLU) {
        // cpu_gelu_tanh_f32 (elementwise_f32_scalar.c:15-20)
        const float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
        a = 0.5f * g * (1.0f + tanhf(inner));
    } else {
        a = g / (1.0f + expf(-g));  // cpu_silu_f32 (elementwise_f32_scalar.c:11-13)
    }
    return a * u;
}

template <bool GEGLU>
__global__ __launch_bounds__(256) void k_glu(const float *__restrict__ gate, const float *__restrict__ up,
                                             float *__restrict__ out, size_t rows, size_t cols, size_t gate_stride,
                                             size_t up_stride, size_t out_stride) {
    const size_t n = rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / cols, c = i - r * cols;
        out[r * out_stride + c] = glu_value<GEGLU>(gate[r * gate_stride + c], up[r * up_stride + c]);
    }
}

// Four values per thread with 16-byte accesses: row length and strides are multiples of 4, the arrays 16-byte
// aligned, and rows * cols / 4 plus one grid stride (at most 2^24) fits 32 bits. Strides here count float4 elements.
template <bool GEGLU>
__global__ __launch_bounds__(256) void k_glu4(const float4 *__restrict__ gate, const float4 *__restrict__ up,
                                              float4 *__restrict__ out, uint32_t n4, uint32_t cols4,
                                              uint32_t gate_stride4, uint32_t up_stride4, uint32_t out_stride4) {
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n4; i += gridDim.x * 256u) {
        const uint32_t r = i / cols4, c = i - r * cols4;
        const float4 g = gate[(size_t)r * gate_stride4 + c], u = up[(size_t)r * up_stride4 + c];
        float4 o;
        o.x = glu_value<GEGLU>(g.x, u.x);
        o.y = glu_value<GEGLU>(g.y, u.y);
        o.z = glu_value<GEGLU>(g.z, u.z);
        o.w = glu_value<GEGLU>(g.w, u.w);
        out[(size_t)r * out_stride4 + c] = o;
    }
}

__global__ __launch_bounds__(256) void k_add(const float *__restrict__ a, const float *__restrict__ b,
                                             float *__restrict__ out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        out[i] = a[i] + b[i];
    }
}

__global__ __launch_bounds__(256) void k_add4(const float4 *__restrict__ a, const float4 *__restrict__ b,
                                              float4 *__restrict__ out, size_t n4) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
        const float4 x = a[i], y = b[i];
        out[i] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    }
}

// Rotary embedding of rows (cpu_rope, src/backends/cpu/ops/rope/rope_dispatch.c:287-372): one thread per pair of a
// row. NORM pairs are neighbours (2i, 2i+1) and move as one 8-byte (fp32) or 4-byte (fp16) access when PAIRED (row
// starts and strides keep them aligned); NEOX pairs (i, i + dim/2) are two accesses, each contiguous across threads.
// INDEX is uint32_t when rows * dim / 2 fits it (the division by the row length is then a 32-bit one).
struct RopeRowsParams {
    const void *x;
    void *out;
    const void *positions;
    const float *freqs;
    float attn_scale;
    int positions_dtype;
    size_t rows, half, x_stride, out_stride;
};

template <bool F16, bool NEOX, bool PAIRED, typename INDEX>
__global__ __launch_bounds__(256) void k_rope_rows(const RopeRowsParams p) {
    const INDEX half = (INDEX)p.half;
    const INDEX total = (INDEX)(p.rows * p.half);
    const INDEX step = (INDEX)gridDim.x * 256u;
    for (INDEX t = (INDEX)blockIdx.x * 256u + threadIdx.x; t < total; t += step) {
        const INDEX row = t / half;
        const INDEX i = t - row * half;
        float pos;
        if (p.positions_dtype == MARMOT_HIP_DTYPE_F32) {
            pos = ((const float *)p.positions)[row];
        } else if (p.positions_dtype == MARMOT_HIP_DTYPE_I32) {
            pos = (float)((const int32_t *)p.positions)[row];
        } else {
            pos = (float)((const int64_t *)p.positions)[row];
        }
        const float angle = pos * p.freqs[i];
        float sin_theta, cos_theta;
        sincosf(angle, &sin_theta, &cos_theta);
        cos_theta *= p.attn_scale;
        sin_theta *= p.attn_scale;
        const size_t even = NEOX ? i : 2 * (size_t)i, odd = NEOX ? (size_t)i + p.half : 2 * (size_t)i + 1;
        const size_t in0 = (size_t)row * p.x_stride, out0 = (size_t)row * p.out_stride;
        float x_even, x_odd;
        if constexpr (F16) {
            const uint16_t *x = (const uint16_t *)p.x;
            if constexpr (PAIRED) {
                const uint32_t both = *(const uint32_t *)(x + in0 + even);
                x_even = h2f((uint16_t)(both & 0xffffu));
                x_odd = h2f((uint16_t)(both >> 16));
            } else {
                x_even = h2f(x[in0 + even]);
                x_odd = h2f(x[in0 + odd]);
            }
        } else {
            const float *x = (const float *)p.x;
            if constexpr (PAIRED) {
                const float2 both = *(const float2 *)(x + in0 + even);
                x_even = both.x;
                x_odd = both.y;
            } else {
                x_even = x[in0 + even];
                x_odd = x[in0 + odd];
            }
        }
        const float r_even = x_even * cos_theta - x_odd * sin_theta;
        const float r_odd = x_even * sin_theta + x_odd * cos_theta;
        if constexpr (F16) {
            uint16_t *out = (uint16_t *)p.out;
            if constexpr (PAIRED) {
                *(uint32_t *)(out + out0 + even) = (uint32_t)f2h(r_even) | ((uint32_t)f2h(r_odd) << 16);
            } else {
                out[out0 + even] = f2h(r_even);
                out[out0 + odd] = f2h(r_odd);
            }
        } else {
            float *out = (float *)p.out;
            if constexpr (PAIRED) {
                *(float2 *)(out + out0 + even) = make_float2(r_even, r_odd);
            } else {
                out[out0 + even] = r_even;
                out[out0 + odd] = r_odd;
            }
        }
    }
}

template <bool F16, bool NEOX, bool PAIRED>
static void launch_rope_rows(marmot_hip_device *dev, const RopeRowsParams &p) {
    const size_t total = p.rows * p.half;
    size_t g = (total + 255) / 256;
    const dim3 grid((unsigned)(g > 65536 ? 65536 : g)), block(256);
    if (total < 0xfe000000ull) {  // the index plus one grid stride (at most 2^24) stays below 2^32
        hipLaunchKernelGGL((k_rope_rows<F16, NEOX, PAIRED, uint32_t>), grid, block, 0, dev->stream, p);
    } else {
        hipLaunchKernelGGL((k_rope_rows<F16, NEOX, PAIRED, size_t>), grid, block, 0, dev->stream, p);
    }
}

static unsigned elementwise_grid(size_t n) {
    size_t g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

} // namespace mh

using namespace mh;

extern "C" {

static int rms_norm_launch(marmot_hip_device_t *dev, const float *d_x, const float *d_residual, const float *d_weight,
                           float weight_offset, float eps, size_t rows, size_t cols, float *d_out, int act_kind,
                           void *d_packed) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || (d_out == nullptr && d_packed == nullptr)) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RMSNorm requires an input and an output");
    }
    if (rows == 0 || cols == 0) {
        return MARMOT_HIP_SUCCESS;  // cpu_norm_no_work
    }
    if (rows > 0x7fffffffu) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RMSNorm: %zu rows exceed one launch", rows);
    }
    MH_HIP(hipSetDevice(dev->device_index));
    RmsNormParams p;
    p.x = d_x;
    p.residual = d_residual;
    p.weight = d_weight;
    p.weight_offset = weight_offset;
    p.eps = eps;
    p.rows = rows;
    p.cols = cols;
    p.out = d_out;
    p.act_kind = act_kind;
    if (act_kind != 0) {
        act_scratch_layout(act_kind, rows, cols, d_packed, &p.packed);
    }
    const dim3 grid((unsigned)rows), block(256);
    const bool aligned16 = ((((uintptr_t)d_x) | ((uintptr_t)d_residual) | ((uintptr_t)d_weight) | ((uintptr_t)d_out)) & 15) == 0;
    if (act_kind != MARMOT_HIP_KIND_Q8_0 && cols % 4 == 0 && cols <= (size_t)RMS_ROW_CHUNKS * 1024 && aligned16) {
        if (act_kind == 0) {
            hipLaunchKernelGGL((k_rms_norm_row_in_registers<0>), grid, block, 0, dev->stream, p);
        } else {
            hipLaunchKernelGGL((k_rms_norm_row_in_registers<MARMOT_HIP_KIND_Q8_K>), grid, block, 0, dev->stream, p);
        }
    } else if (act_kind == 0) {
        hipLaunchKernelGGL((k_rms_norm<0>), grid, block, 0, dev->stream, p);
    } else if (act_kind == MARMOT_HIP_KIND_Q8_K) {
        hipLaunchKernelGGL((k_rms_norm<MARMOT_HIP_KIND_Q8_K>), grid, block, 0, dev->stream, p);
    } else {
        hipLaunchKernelGGL((k_rms_norm<MARMOT_HIP_KIND_Q8_0>), grid, block, 0, dev->stream, p);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_rms_norm(marmot_hip_device_t *dev, const float *d_x, const float *d_residual, const float *d_weight,
                        float weight_offset, float eps, size_t rows, size_t cols, float *d_out) {
    if (d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RMSNorm requires an output");
    }
    return rms_norm_launch(dev, d_x, d_residual, d_weight, weight_offset, eps, rows, cols, d_out, 0, nullptr);
}

int marmot_hip_rms_norm_pack(marmot_hip_device_t *dev, const float *d_x, const float *d_residual,
                             const float *d_weight, float weight_offset, float eps, size_t rows, size_t cols,
                             int weight_kind, float *d_out, void *d_packed) {
    if (d_packed == nullptr || (((uintptr_t)d_packed) & 255) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "rms_norm_pack: d_packed must be 256-byte aligned");
    }
    if (marmot_hip_packed_activation_bytes(weight_kind, 1, 1) == 0) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "rms_norm_pack: unsupported quant kind %d", weight_kind);
    }
    const int act_kind = is_k_quant(weight_kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    return rms_norm_launch(dev, d_x, d_residual, d_weight, weight_offset, eps, rows, cols, d_out, act_kind, d_packed);
}

int marmot_hip_glu(marmot_hip_device_t *dev, int ffn_type, const float *d_gate, const float *d_up, size_t rows,
                   size_t cols, size_t gate_stride, size_t up_stride, size_t out_stride, float *d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_gate == nullptr || d_up == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (ffn_type != MARMOT_HIP_FFN_SWIGLU && ffn_type != MARMOT_HIP_FFN_GEGLU) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "glu: type %d is not SwiGLU or GeGLU", ffn_type);
    }
    if (gate_stride < cols || up_stride < cols || out_stride < cols) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "glu: row stride shorter than a row");
    }
    if (rows == 0 || cols == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    const dim3 block(256);
    const bool by4 = cols % 4 == 0 && gate_stride % 4 == 0 && up_stride % 4 == 0 && out_stride % 4 == 0 &&
        ((((uintptr_t)d_gate) | ((uintptr_t)d_up) | ((uintptr_t)d_out)) & 15) == 0 && rows * cols / 4 < 0xfe000000ull &&
        gate_stride / 4 < 0xffffffffull && up_stride / 4 < 0xffffffffull && out_stride / 4 < 0xffffffffull;
    if (by4) {
        const uint32_t n4 = (uint32_t)(rows * cols / 4), c4 = (uint32_t)(cols / 4);
        const dim3 grid4(elementwise_grid(n4));
        if (ffn_type == MARMOT_HIP_FFN_GEGLU) {
            hipLaunchKernelGGL((k_glu4<true>), grid4, block, 0, dev->stream, (const float4 *)d_gate,
                               (const float4 *)d_up, (float4 *)d_out, n4, c4, (uint32_t)(gate_stride / 4),
                               (uint32_t)(up_stride / 4), (uint32_t)(out_stride / 4));
        } else {
            hipLaunchKernelGGL((k_glu4<false>), grid4, block, 0, dev->stream, (const float4 *)d_gate,
                               (const float4 *)d_up, (float4 *)d_out, n4, c4, (uint32_t)(gate_stride / 4),
                               (uint32_t)(up_stride / 4), (uint32_t)(out_stride / 4));
        }
        MH_HIP(hipGetLastError());
        return MARMOT_HIP_SUCCESS;
    }
    const dim3 grid(elementwise_grid(rows * cols));
    if (ffn_type == MARMOT_HIP_FFN_GEGLU) {
        hipLaunchKernelGGL((k_glu<true>), grid, block, 0, dev->stream, d_gate, d_up, d_out, rows, cols, gate_stride,
                           up_stride, out_stride);
    } else {
        hipLaunchKernelGGL((k_glu<false>), grid, block, 0, dev->stream, d_gate, d_up, d_out, rows, cols, gate_stride,
                           up_stride, out_stride);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_swiglu_pack(marmot_hip_device_t *dev, const float *d_gate, const float *d_up, size_t rows, size_t cols,
                           int weight_kind, void *d_packed) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_gate == nullptr || d_up == nullptr || d_packed == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if ((((uintptr_t)d_packed) & 255) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "swiglu_pack: d_packed must be 256-byte aligned");
    }
    if (marmot_hip_packed_activation_bytes(weight_kind, 1, 1) == 0) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "swiglu_pack: unsupported quant kind %d", weight_kind);
    }
    if (rows == 0 || cols == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    const int act_kind = is_k_quant(weight_kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    ActScratch act;
    act_scratch_layout(act_kind, rows, cols, d_packed, &act);
    return launch_quantize_glu_soa(dev, act_kind, d_gate, d_up, false, rows, cols, act);
}

int marmot_hip_add(marmot_hip_device_t *dev, const float *d_a, const float *d_b, size_t n, float *d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_a == nullptr || d_b == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (n == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    if (n % 4 == 0 && ((((uintptr_t)d_a) | ((uintptr_t)d_b) | ((uintptr_t)d_out)) & 15) == 0) {
        hipLaunchKernelGGL(k_add4, dim3(elementwise_grid(n / 4)), dim3(256), 0, dev->stream, (const float4 *)d_a,
                           (const float4 *)d_b, (float4 *)d_out, n / 4);
    } else {
        hipLaunchKernelGGL(k_add, dim3(elementwise_grid(n)), dim3(256), 0, dev->stream, d_a, d_b, d_out, n);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_rope(marmot_hip_device_t *dev, const void *d_x, int dtype, size_t rows, size_t dim,
                    size_t x_row_stride, size_t out_row_stride, const marmot_hip_rope_t *rope, void *d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_out == nullptr || rope == nullptr || rope->d_positions == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "rope: input, output, parameters and positions are required");
    }
    if (dtype != MARMOT_HIP_DTYPE_F32 && dtype != MARMOT_HIP_DTYPE_F16) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "rope: rows must be FLOAT32 or FLOAT16");
    }
    if (dim % 2 != 0) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "rope: the rotated dimension %zu is odd", dim);
    }
    if (rows == 0 || dim == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "rope: the input must not be empty");
    }
    if (rope->positions_dtype != MARMOT_HIP_DTYPE_F32 && rope->positions_dtype != MARMOT_HIP_DTYPE_I32 &&
        rope->positions_dtype != MARMOT_HIP_DTYPE_I64) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "rope: positions must be FLOAT32, INT32 or INT64");
    }
    if (x_row_stride < dim || out_row_stride < dim) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "rope: row stride shorter than a row");
    }
    if (rope->d_freqs == nullptr || rope->head_dim != dim) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT,
                         "rope: needs the %zu frequencies of the rotated dimension (head_dim %u given)", dim / 2,
                         rope->head_dim);
    }
    if (rope->rope_type != 0 && rope->rope_type != 1) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "rope: unknown rope type %d", rope->rope_type);
    }
    MH_HIP(hipSetDevice(dev->device_index));
    RopeRowsParams p;
    p.x = d_x;
    p.out = d_out;
    p.positions = rope->d_positions;
    p.freqs = rope->d_freqs;
    p.attn_scale = rope->attn_scale;
    p.positions_dtype = rope->positions_dtype;
    p.rows = rows;
    p.half = dim / 2;
    p.x_stride = x_row_stride;
    p.out_stride = out_row_stride;
    const bool f16 = dtype == MARMOT_HIP_DTYPE_F16;
    const uintptr_t pair_mask = f16 ? 3 : 7;
    const bool paired = rope->rope_type == 0 && (((uintptr_t)d_x | (uintptr_t)d_out) & pair_mask) == 0 &&
        x_row_stride % 2 == 0 && out_row_stride % 2 == 0;
    if (rope->rope_type == 1) {
        f16 ? launch_rope_rows<true, true, false>(dev, p) : launch_rope_rows<false, true, false>(dev, p);
    } else if (paired) {
        f16 ? launch_rope_rows<true, false, true>(dev, p) : launch_rope_rows<false, false, true>(dev, p);
    } else {
        f16 ? launch_rope_rows<true, false, false>(dev, p) : launch_rope_rows<false, false, false>(dev, p);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

} // extern "C"

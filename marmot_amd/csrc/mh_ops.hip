// The fp32 operations that sit between the quantized linears of a decoder layer, and their fused forms that hand the
// next linear its activations already quantized:
//   * RMS normalization (cpu_rmsnorm_impl / cpu_rmsnorm_gemma_impl, normalization_dispatch.c:129-181,
//     normalization_scalar.c:469-510, 780-791): out = (x [+ residual]) * inv_rms * (weight + weight_offset),
//     inv_rms = 1 / sqrt(mean((x [+ residual])^2) + eps); optionally the rows are also written as packed Q8_K / Q8_0
//     activations (the input of the q/k/v or gate/up projections), one launch for both.
//   * gated products swiglu / geglu (cpu_swiglu_f32_scalar / cpu_geglu_f32_scalar, elementwise_f32_scalar.c:11-20,
//     147-214), optionally straight into packed activations (the input of the down projection);
//   * residual add (cpu_add_f32, elementwise_f32_scalar.c).
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

// One workgroup of 256 threads per row.
template <int ACT>
__global__ __launch_bounds__(256) void k_rms_norm(const RmsNormParams p) {
    __shared__ float red[4];
    warm_kernel_arguments<sizeof(RmsNormParams), sizeof(RmsNormParams)>();
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *x = p.x + row * p.cols;
    const float *res = p.residual != nullptr ? p.residual + row * p.cols : nullptr;
    float sum = 0.0f;
    for (size_t i = tid; i < p.cols; i += 256) {
        float v = x[i];
        if (res != nullptr) {
            v += res[i];
        }
        sum += v * v;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        sum += __shfl_xor(sum, off);
    }
    if (lane == 0) {
        red[wave] = sum;
    }
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
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
__global__ __launch_bounds__(256) void k_glu(const float *__restrict__ gate, const float *__restrict__ up,
                                             float *__restrict__ out, size_t rows, size_t cols, size_t gate_stride,
                                             size_t up_stride, size_t out_stride) {
    const size_t n = rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / cols, c = i - r * cols;
        const float g = gate[r * gate_stride + c];
        float a;
        if constexpr (GEGLU) {
            // cpu_gelu_tanh_f32 (elementwise_f32_scalar.c:15-20)
            const float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
            a = 0.5f * g * (1.0f + tanhf(inner));
        } else {
            a = g / (1.0f + expf(-g));  // cpu_silu_f32 (elementwise_f32_scalar.c:11-13)
        }
        out[r * out_stride + c] = a * up[r * up_stride + c];
    }
}

__global__ __launch_bounds__(256) void k_add(const float *__restrict__ a, const float *__restrict__ b,
                                             float *__restrict__ out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        out[i] = a[i] + b[i];
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
    if (act_kind == 0) {
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
    const dim3 grid(elementwise_grid(rows * cols)), block(256);
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
    hipLaunchKernelGGL(k_add, dim3(elementwise_grid(n)), dim3(256), 0, dev->stream, d_a, d_b, d_out, n);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

} // extern "C"

// marmot_hip_matmul_quantized: validation, route selection, and the direct (unquantized fp16 activation)
// small-batch kernel. Compile with -ffp-contract=off (the direct route dequantizes weights exactly like the
// reference before multiplying).
#include "mh_common.h"
#include "mh_dequant.h"

namespace mh {

// Scratch of marmot_hip_matmul_quantized_noalloc: device memory that exists from the moment the library is loaded, one
// copy per GPU, held until the process ends. In host code the array's name is only a handle: the address each device
// uses comes from hipGetSymbolAddress (static_scratch_init) and is what kernels and helpers receive.
static __device__ __align__(256) uint8_t scratch[MARMOT_HIP_NOALLOC_SCRATCH_BYTES];

int static_scratch_init(marmot_hip_device *dev) {
    void *ptr = nullptr;
    MH_HIP(hipSetDevice(dev->device_index));
    MH_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    dev->static_scratch = ptr;
    dev->static_scratch_bytes = MARMOT_HIP_NOALLOC_SCRATCH_BYTES;
    return MARMOT_HIP_SUCCESS;
}

// ------------------------------------------------------------------------------------------------
// Direct route: out[n, m] = sum_k dequant(W[m, k]) * (float)x_f16[n, k], fp32 accumulate.
// Counterpart of cpu_vec_dot_{scheme}_f16 (vec_dot_impl.h:220-286, 351-450, 866-1128): the same per-value fp32 weights
// (for Q2_K, Q3_K, Q5_K and Q6_K the ones those functions decode, see direct_f16_weight), summed in a different order. One wavefront per weight row; a lane visits 8
// consecutive k at a time (one 16-byte load of fp16 activations per column).
// ------------------------------------------------------------------------------------------------
struct DirectParams {
    const uint8_t *w;
    const uint16_t *x;
    void *out;
    const void *bias;
    int bias_is_f16;
    int out_is_f16;
    size_t n0;
    size_t K;
    size_t M;
    size_t nb;
};

template <int KIND, int NC>
__global__ __launch_bounds__(256) void k_matvec_direct_f16(const DirectParams p) {
    warm_kernel_arguments<sizeof(DirectParams), sizeof(DirectParams)>();
    constexpr int BV = KindTraits<KIND>::BV;
    constexpr int BB = KindTraits<KIND>::BB;
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= p.M) {
        return;
    }
    const uint8_t *rowp = p.w + row * p.nb * BB;
    float acc[NC];
#pragma unroll
    for (int n = 0; n < NC; ++n) {
        acc[n] = 0.0f;
    }
    for (size_t k0 = (size_t)lane * 8; k0 < p.K; k0 += 64 * 8) {
        const size_t b = k0 / BV;
        const int v0 = (int)(k0 - b * BV);
        const uint8_t *blk = rowp + b * BB;
        float wv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            wv[i] = (k0 + i < p.K) ? direct_f16_weight<KIND>(blk, v0 + i) : 0.0f;
        }
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            const uint16_t *xp = p.x + (p.n0 + n) * p.K + k0;
            if (k0 + 8 <= p.K && (((uintptr_t)xp) & 15) == 0) {
                const uint4 xv = *(const uint4 *)xp;
                const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[n] += wv[2 * i] * h2f((uint16_t)(xs[i] & 0xffffu));
                    acc[n] += wv[2 * i + 1] * h2f((uint16_t)(xs[i] >> 16));
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (k0 + i < p.K) {
                        acc[n] += wv[i] * h2f(xp[i]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int n = 0; n < NC; ++n) {
        const float s = wave_sum(acc[n]);
        if (lane == 0) {
            const size_t idx = (p.n0 + n) * p.M + row;
            if (!p.out_is_f16) {
                float v = s;
                if (p.bias != nullptr) {
                    v += ((const float *)p.bias)[row];
                }
                ((float *)p.out)[idx] = v;
            } else {
                uint16_t h = f2h(s);
                if (p.bias != nullptr) {
                    const float bv =
                        p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[row]) : ((const float *)p.bias)[row];
                    h = f2h(h2f(h) + bv);
                }
                ((uint16_t *)p.out)[idx] = h;
            }
        }
    }
}

template <int KIND>
static int launch_direct_kind(marmot_hip_device *dev, DirectParams p, size_t N) {
    const dim3 grid((unsigned)((p.M + 3) / 4)), block(256);
    size_t n0 = 0;
    while (n0 < N) {
        p.n0 = n0;
        const size_t left = N - n0;
        if (left >= 4) {
            hipLaunchKernelGGL((k_matvec_direct_f16<KIND, 4>), grid, block, 0, dev->stream, p);
            n0 += 4;
        } else if (left >= 2) {
            hipLaunchKernelGGL((k_matvec_direct_f16<KIND, 2>), grid, block, 0, dev->stream, p);
            n0 += 2;
        } else {
            hipLaunchKernelGGL((k_matvec_direct_f16<KIND, 1>), grid, block, 0, dev->stream, p);
            n0 += 1;
        }
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int launch_matvec_f16(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K, size_t M,
                      const void *d_bias, int bias_dtype, void *d_out, int out_dtype) {
    DirectParams p;
    p.w = (const uint8_t *)d_w;
    p.x = (const uint16_t *)d_x;
    p.out = d_out;
    p.bias = d_bias;
    p.bias_is_f16 = bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.n0 = 0;
    p.K = K;
    p.M = M;
    p.nb = (K + block_values(kind) - 1) / block_values(kind);
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_K:
        set_route("matvec_q4_k_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q4_K>(dev, p, N);
    case MARMOT_HIP_KIND_Q8_0:
        set_route("matvec_q8_0_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q8_0>(dev, p, N);
    case MARMOT_HIP_KIND_Q4_0:
        set_route("matvec_q4_0_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q4_0>(dev, p, N);
    case MARMOT_HIP_KIND_Q8_1:
        set_route("matvec_q8_1_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q8_1>(dev, p, N);
    case MARMOT_HIP_KIND_Q4_1:
        set_route("matvec_q4_1_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q4_1>(dev, p, N);
    case MARMOT_HIP_KIND_Q5_0:
        set_route("matvec_q5_0_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q5_0>(dev, p, N);
    case MARMOT_HIP_KIND_Q5_1:
        set_route("matvec_q5_1_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q5_1>(dev, p, N);
    case MARMOT_HIP_KIND_Q2_K:
        set_route("matvec_q2_k_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q2_K>(dev, p, N);
    case MARMOT_HIP_KIND_Q3_K:
        set_route("matvec_q3_k_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q3_K>(dev, p, N);
    case MARMOT_HIP_KIND_Q5_K:
        set_route("matvec_q5_k_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q5_K>(dev, p, N);
    case MARMOT_HIP_KIND_Q6_K:
        set_route("matvec_q6_k_f16_direct");
        return launch_direct_kind<MARMOT_HIP_KIND_Q6_K>(dev, p, N);
    default:
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED,
                         "quantized matmul: fp16 activations without packing are not offered for quant kind %d", kind);
    }
}

static int validate_matmul(const marmot_hip_device *dev, int kind, const void *d_weight, const void *d_input,
                           int in_dtype, size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype,
                           const void *d_out, int out_dtype) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_weight == nullptr || d_input == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (!is_weight_kind(kind)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "Quantized matmul kernel not available for quant kind %d",
                         kind);
    }
    const bool in_f32 = in_dtype == MARMOT_HIP_DTYPE_F32, in_f16 = in_dtype == MARMOT_HIP_DTYPE_F16;
    const bool out_f32 = out_dtype == MARMOT_HIP_DTYPE_F32, out_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    if (!((in_f32 && out_f32) || (in_f16 && (out_f32 || out_f16)))) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE,
                         "Quantized matmul requires FLOAT32 input or FLOAT16 activations with FLOAT16/FLOAT32 output");
    }
    if (d_bias != nullptr) {
        const bool ok = (bias_dtype == MARMOT_HIP_DTYPE_F32) || (bias_dtype == MARMOT_HIP_DTYPE_F16 && out_f16);
        if (!ok) {
            return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "Matmul bias dtype is not compatible with the output");
        }
    }
    if (K == 0 || M == 0) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "Quantized matmul dimension mismatch on K");
    }
    (void)N;
    return MARMOT_HIP_SUCCESS;
}

static int matmul_impl(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, const void *d_input,
                       int in_dtype, size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype, void *d_out0,
                       void *d_out1, int out_dtype, uint32_t flags) {
    if (N == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    const bool direct = in_dtype == MARMOT_HIP_DTYPE_F16 && (flags & MARMOT_HIP_MATMUL_FORCE_PACK) == 0;
    if (direct) {
        for (int which = 0; which < (d_w1 != nullptr ? 2 : 1); ++which) {
            const void *w = which ? d_w1 : d_w0;
            void *o = which ? d_out1 : d_out0;
            int st;
            if (gemm_f16_supported(dev, kind, N, K, M)) {
                st = launch_gemm_f16(dev, kind, w, d_input, N, K, M, d_bias, bias_dtype, o, out_dtype);
            } else if (gemm_f16_any_supported(dev, kind, N, K, M) && (((uintptr_t)d_input) & 15) == 0 &&
                       (((uintptr_t)w) & 3) == 0) {  // (the kernel loads weight words from multiples of 4)
                st = launch_gemm_f16_any(dev, kind, w, d_input, N, K, M, d_bias, bias_dtype, o, out_dtype);
            } else {
                st = launch_matvec_f16(dev, kind, w, d_input, N, K, M, d_bias, bias_dtype, o, out_dtype);
            }
            if (st != MARMOT_HIP_SUCCESS) {
                return st;
            }
        }
        return MARMOT_HIP_SUCCESS;
    }
    // packed route. fp32 activations whose rows are whole blocks are quantized inside the matvec kernel; otherwise
    // the activations are quantized once into the workspace (shared by both weights of a dual call).
    const bool mmq = mmq_supported(dev, kind, N, K);
    const bool rows_kernel = mmq && kind == MARMOT_HIP_KIND_Q4_K && N <= 16 && !dev->knobs.no_row_kernels;
    WeightSet rows_ws;
    rows_ws.count = d_w1 != nullptr ? 2 : 1;
    rows_ws.w[0] = d_w0;
    rows_ws.w[1] = d_w1;
    rows_ws.out[0] = d_out0;
    rows_ws.out[1] = d_out1;
    rows_ws.bias[0] = d_bias;
    rows_ws.bias[1] = d_bias;
    rows_ws.bias_dtype = bias_dtype;
    if (rows_kernel && in_dtype == MARMOT_HIP_DTYPE_F32) {
        // row-owning small-batch kernel: quantizes the activations itself, no partial sums
        const int st = launch_mmq_rows_q4k(dev, rows_ws, (const float *)d_input, nullptr, N, K, M, out_dtype);
        if (st != MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
            return st;
        }
    }
    if (!mmq && in_dtype == MARMOT_HIP_DTYPE_F32 && matvec_can_fuse_quantization(dev, kind, N, K, d_input)) {
        return launch_matvec_packed(dev, kind, d_w0, d_w1, nullptr, (const float *)d_input, N, K, M, d_bias,
                                    bias_dtype, d_out0, d_out1, out_dtype);
    }
    const int act_kind = is_k_quant(kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    const size_t act_bytes = (act_scratch_layout(act_kind, N, K, nullptr, nullptr) + 255) & ~(size_t)255;
    // Q2_K, Q3_K (from five rows on) and the 32-value formats but Q8_1 (from nine): the tiled int8 GEMMs (their K-split partial
    // sums behind the activations)
    const bool q80_kind = gemm_q80_kind(kind) && N >= gemm_q80_min_rows(kind) && K % QK_K == 0;
    const size_t need = act_bytes + (mmq ? mmq_scratch_bytes(dev, kind, N, K, M, d_w1 != nullptr ? 2 : 1) : 0) +
                        (q80_kind ? gemm_i8_scratch_bytes(dev, N, K, M, d_w1 != nullptr ? 2 : 1) : 0);
    void *ws = nullptr;
    int st = workspace_reserve(dev, need, &ws);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    ActScratch act;
    act_scratch_layout(act_kind, N, K, ws, &act);
    st = launch_quantize_act_soa(dev, act_kind, d_input, in_dtype, N, K, act);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    if (q80_kind && gemm_q80_applies(dev, kind, N, K, rows_ws.w, rows_ws.count, act)) {
        return launch_gemm_q80(dev, kind, rows_ws, act, N, K, M, out_dtype, (uint8_t *)ws + act_bytes);
    }
    if (rows_kernel) {
        st = launch_mmq_rows_q4k(dev, rows_ws, nullptr, &act, N, K, M, out_dtype);
        if (st != MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
            return st;
        }
    }
    if (mmq) {
        return launch_mmq(dev, kind, d_w0, d_w1, act, N, K, M, d_bias, bias_dtype, d_out0, d_out1, out_dtype,
                          (uint8_t *)ws + act_bytes);
    }
    return launch_matvec_packed(dev, kind, d_w0, d_w1, &act, nullptr, N, K, M, d_bias, bias_dtype, d_out0, d_out1,
                                out_dtype);
}

// ------------------------------------------------------------------ rotary epilogue of the Q/K/V projection
// One thread per (projection, activation row, pair of columns). src: fp32 [N, M] (the projection before the store's
// rounding: the output itself for fp32 outputs, a workspace for fp16 outputs); dst: [N, M] of the output dtype.
// A projection that is not rotated is only converted (fp16 outputs) or skipped (fp32, src == dst).
struct RopeFinishParams {
    const float *src[3];
    void *dst[3];
    int rotate[3];
    const void *positions;
    int positions_dtype;
    const float *freqs;
    float attn_scale;
    uint32_t head_dim;
    int neox;
    int out_is_f16;
    size_t N, M;
};

__global__ __launch_bounds__(256) void k_qkv_rope_finish(const RopeFinishParams p) {
    warm_kernel_arguments<sizeof(RopeFinishParams), sizeof(RopeFinishParams)>();
    const int proj = blockIdx.z;
    const size_t n = blockIdx.y;
    const size_t pair = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (pair >= p.M / 2) {
        return;
    }
    const float *src = p.src[proj] + n * p.M;
    const bool rotate = p.rotate[proj] != 0;
    if (!rotate && !p.out_is_f16) {
        return;  // fp32 output already holds the projection
    }
    const uint32_t half = p.head_dim / 2;
    const size_t head = pair / half;
    const uint32_t i = (uint32_t)(pair - head * half);
    size_t even_index, odd_index;
    if (rotate) {
        even_index = head * p.head_dim + (p.neox ? i : 2 * i);
        odd_index = head * p.head_dim + (p.neox ? i + half : 2 * i + 1);
    } else {
        even_index = 2 * pair;
        odd_index = 2 * pair + 1;
    }
    float even = src[even_index], odd = src[odd_index];
    if (rotate) {
        float pos;
        if (p.positions_dtype == MARMOT_HIP_DTYPE_F32) {
            pos = ((const float *)p.positions)[n];
        } else if (p.positions_dtype == MARMOT_HIP_DTYPE_I32) {
            pos = (float)((const int32_t *)p.positions)[n];
        } else {
            pos = (float)((const int64_t *)p.positions)[n];
        }
        const float angle = pos * p.freqs[i];
        float sin_theta, cos_theta;
        sincosf(angle, &sin_theta, &cos_theta);
        cos_theta *= p.attn_scale;
        sin_theta *= p.attn_scale;
        const float e = even * cos_theta - odd * sin_theta;
        const float o = even * sin_theta + odd * cos_theta;
        even = e;
        odd = o;
    }
    if (p.out_is_f16) {
        uint16_t *dst = (uint16_t *)p.dst[proj] + n * p.M;
        dst[even_index] = f2h(even);
        dst[odd_index] = f2h(odd);
    } else {
        float *dst = (float *)p.dst[proj] + n * p.M;
        dst[even_index] = even;
        dst[odd_index] = odd;
    }
}

// Rotary epilogue of the Q/K/V projection. stage: the three fp32 projections [3][N][M] when the outputs are fp16
// (rounded once, after the rotation), nullptr when the fp32 outputs themselves hold them.
static int qkv_rope_finish(marmot_hip_device *dev, const marmot_hip_rope_t *rope, const float *stage, void *d_out_q,
                           void *d_out_k, void *d_out_v, size_t N, size_t M, int out_dtype) {
    const bool stage32 = stage != nullptr;
    RopeFinishParams rp;
    void *outs[3] = {d_out_q, d_out_k, d_out_v};
    for (int i = 0; i < 3; ++i) {
        rp.src[i] = stage32 ? stage + (size_t)i * N * M : (const float *)outs[i];
        rp.dst[i] = outs[i];
    }
    rp.rotate[0] = rope->apply_to_q ? 1 : 0;
    rp.rotate[1] = rope->apply_to_k ? 1 : 0;
    rp.rotate[2] = 0;
    rp.positions = rope->d_positions;
    rp.positions_dtype = rope->positions_dtype;
    rp.freqs = rope->d_freqs;
    rp.attn_scale = rope->attn_scale;
    rp.head_dim = rope->head_dim;
    rp.neox = rope->rope_type == 1;
    rp.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    rp.N = N;
    rp.M = M;
    if (N > 65535) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RoPE epilogue: more than 65535 activation rows");
    }
    const dim3 grid((unsigned)((M / 2 + 255) / 256), (unsigned)N, 3);
    hipLaunchKernelGGL(k_qkv_rope_finish, grid, dim3(256), 0, dev->stream, rp);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

} // namespace mh

using namespace mh;

extern "C" {

int marmot_hip_matmul_quantized(marmot_hip_device_t *dev, int kind, const void *d_weight, const void *d_input,
                                int in_dtype, size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype,
                                void *d_out, int out_dtype, uint32_t flags) {
    int st = validate_matmul(dev, kind, d_weight, d_input, in_dtype, N, K, M, d_bias, bias_dtype, d_out, out_dtype);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    return matmul_impl(dev, kind, d_weight, nullptr, d_input, in_dtype, N, K, M, d_bias, bias_dtype, d_out, nullptr,
                       out_dtype, flags);
}

int marmot_hip_matmul_quantized_noalloc(marmot_hip_device_t *dev, int kind, const void *d_weight, const void *d_input,
                                        int in_dtype, size_t N, size_t K, size_t M, const void *d_bias,
                                        int bias_dtype, void *d_out, int out_dtype, uint32_t flags) {
    int st = validate_matmul(dev, kind, d_weight, d_input, in_dtype, N, K, M, d_bias, bias_dtype, d_out, out_dtype);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    if (dev->branch > 0) {
        // the array exists once per device: a call in another branch of the same section could use it at the same time
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION,
                         "matmul_quantized_noalloc: only in the first branch of a branch section");
    }
    // same routes and kernels as marmot_hip_matmul_quantized; every scratch request of the call is served from this
    // device's copy of the static array (or refused when it is larger)
    dev->use_static_scratch = true;
    st = matmul_impl(dev, kind, d_weight, nullptr, d_input, in_dtype, N, K, M, d_bias, bias_dtype, d_out, nullptr,
                     out_dtype, flags);
    dev->use_static_scratch = false;
    return st;
}

size_t marmot_hip_packed_activation_bytes(int weight_kind, size_t N, size_t K) {
    if (block_values(weight_kind) == 0 || weight_kind == MARMOT_HIP_KIND_Q8_K) {
        return 0;
    }
    const int act_kind = is_k_quant(weight_kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    return act_scratch_layout(act_kind, N, K, nullptr, nullptr);
}

int marmot_hip_packed_activation_layout(int weight_kind, size_t N, size_t K, marmot_hip_packed_layout_t *layout) {
    if (layout == nullptr || block_values(weight_kind) == 0 || weight_kind == MARMOT_HIP_KIND_Q8_K) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "packed activation layout: unsupported weight kind %d",
                         weight_kind);
    }
    const int act_kind = is_k_quant(weight_kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    ActScratch act;
    uint8_t *const origin = nullptr;
    layout->total_bytes = act_scratch_layout(act_kind, N, K, origin, &act);
    layout->act_kind = act_kind;
    layout->values_offset = 0;
    layout->values_per_row = act.kp;
    layout->scales_offset = (size_t)((uint8_t *)act.d - origin);
    layout->blocks_per_row = act.nb;
    layout->sums_offset = (size_t)((uint8_t *)act.sums - origin);
    layout->sums_per_block = act_kind == MARMOT_HIP_KIND_Q8_K ? 16 : 1;
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_pack_activations(marmot_hip_device_t *dev, int weight_kind, const void *d_input, int in_dtype,
                                size_t N, size_t K, void *d_packed) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_input == nullptr || d_packed == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (marmot_hip_packed_activation_bytes(weight_kind, 1, 1) == 0) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "pack_activations: unsupported quant kind %d", weight_kind);
    }
    if (in_dtype != MARMOT_HIP_DTYPE_F32 && in_dtype != MARMOT_HIP_DTYPE_F16) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "pack_activations: input dtype %d", in_dtype);
    }
    if ((((uintptr_t)d_packed) & 255) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "pack_activations: d_packed must be 256-byte aligned");
    }
    const int act_kind = is_k_quant(weight_kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    ActScratch act;
    act_scratch_layout(act_kind, N, K, d_packed, &act);
    return launch_quantize_act_soa(dev, act_kind, d_input, in_dtype, N, K, act);
}

int marmot_hip_matmul_prepacked(marmot_hip_device_t *dev, int kind, const void *d_weight, const void *d_packed,
                                size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype, void *d_out,
                                int out_dtype) {
    // the packed route accepts what a forced-pack call would: any float input dtype has already been consumed
    int st = validate_matmul(dev, kind, d_weight, d_packed, MARMOT_HIP_DTYPE_F16, N, K, M, d_bias, bias_dtype, d_out,
                             out_dtype);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    if ((((uintptr_t)d_packed) & 255) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "matmul_prepacked: d_packed must be 256-byte aligned");
    }
    if (N == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    const int act_kind = is_k_quant(kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    ActScratch act;
    act_scratch_layout(act_kind, N, K, const_cast<void *>(d_packed), &act);
    if (mmq_supported(dev, kind, N, K)) {
        MH_HIP(hipSetDevice(dev->device_index));
        if (kind == MARMOT_HIP_KIND_Q4_K && N <= 16 && !dev->knobs.no_row_kernels) {
            WeightSet ws;
            ws.w[0] = d_weight;
            ws.out[0] = d_out;
            ws.bias[0] = d_bias;
            ws.bias_dtype = bias_dtype;
            st = launch_mmq_rows_q4k(dev, ws, nullptr, &act, N, K, M, out_dtype);
            if (st != MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                return st;
            }
        }
        return launch_mmq(dev, kind, d_weight, nullptr, act, N, K, M, d_bias, bias_dtype, d_out, nullptr, out_dtype,
                          nullptr);
    }
    {
        WeightSet ws;
        ws.w[0] = d_weight;
        ws.out[0] = d_out;
        ws.bias[0] = d_bias;
        ws.bias_dtype = bias_dtype;
        if (gemm_q80_applies(dev, kind, N, K, ws.w, 1, act)) {
            MH_HIP(hipSetDevice(dev->device_index));
            const size_t partial_bytes = gemm_i8_scratch_bytes(dev, N, K, M, 1);
            void *scratch = nullptr;
            if (partial_bytes != 0) {
                MH_TRY(workspace_reserve(dev, partial_bytes, &scratch));
            }
            return launch_gemm_q80(dev, kind, ws, act, N, K, M, out_dtype, scratch);
        }
    }
    return launch_matvec_packed(dev, kind, d_weight, nullptr, &act, nullptr, N, K, M, d_bias, bias_dtype, d_out,
                                nullptr, out_dtype);
}

int marmot_hip_matmul_quantized_dual(marmot_hip_device_t *dev, int kind, const void *d_weight_a,
                                     const void *d_weight_b, const void *d_input, int in_dtype, size_t N, size_t K,
                                     size_t M, void *d_out_a, void *d_out_b, int out_dtype, uint32_t flags) {
    if (d_weight_b == nullptr || d_out_b == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    int st = validate_matmul(dev, kind, d_weight_a, d_input, in_dtype, N, K, M, nullptr, 0, d_out_a, out_dtype);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    return matmul_impl(dev, kind, d_weight_a, d_weight_b, d_input, in_dtype, N, K, M, nullptr, 0, d_out_a, d_out_b,
                       out_dtype, flags);
}

int marmot_hip_matmul_qkv_quantized(marmot_hip_device_t *dev, int kind, const void *d_wq, const void *d_wk,
                                    const void *d_wv, const void *d_input, int in_dtype, size_t N, size_t K, size_t M,
                                    const void *d_bq, const void *d_bk, const void *d_bv, int bias_dtype,
                                    void *d_out_q, void *d_out_k, void *d_out_v, int out_dtype) {
    return marmot_hip_matmul_qkv_rope_quantized(dev, kind, d_wq, d_wk, d_wv, d_input, in_dtype, N, K, M, d_bq, d_bk,
                                                d_bv, bias_dtype, d_out_q, d_out_k, d_out_v, out_dtype, nullptr);
}

int marmot_hip_rope_frequencies(int scaling_type, float theta, float freq_scale, float ext_factor,
                                float attn_factor, float beta_fast, float beta_slow, uint32_t orig_ctx_len,
                                uint32_t head_dim, size_t M, float *freqs_out, float *attn_scale_out,
                                uint32_t *head_dim_out) {
    if (freqs_out == nullptr || attn_scale_out == nullptr || head_dim_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RoPE frequency span output is null");
    }
    // cpu_matmul_qkv_resolve_head_dim (matmul_qkv_rope.h:14-23)
    size_t hd = head_dim;
    if (hd == 0 || hd > M || (M % hd) != 0 || (hd & 1u) != 0u) {
        hd = M;
    }
    if ((hd & 1u) != 0u) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RoPE frequency cache requires even dimensions");
    }
    // rope_scaling_prepare (src/core/helpers/rope.c:61-110)
    if (freq_scale <= 0.0f) {
        freq_scale = 1.0f;
    }
    if (attn_factor <= 0.0f) {
        attn_factor = 1.0f;
    }
    if (scaling_type == 0 || scaling_type == -1) {
        freq_scale = 1.0f;
        ext_factor = 0.0f;
    } else if (scaling_type == 1 || scaling_type == 3) {
        ext_factor = 0.0f;
    }
    if (!(ext_factor != 0.0f && orig_ctx_len > 0 && theta > 0.0f && beta_fast > 0.0f && beta_slow > 0.0f)) {
        ext_factor = 0.0f;
    }
    // YaRN: correction range (rope_yarn_corr_dims, rope.c:38-59) and attention scale (rope.c:95-99)
    float corr_low = 0.0f, corr_high = 0.0f;
    float attn_scale = attn_factor;
    if (ext_factor != 0.0f) {
        const float denom = 2.0f * logf(theta);
        const float pi = 3.14159265358979323846f;
        float low_raw = 0.0f, high_raw = 0.0f;
        if (denom != 0.0f) {
            low_raw = (float)(int)hd * logf((float)(int)orig_ctx_len / (beta_fast * 2.0f * pi)) / denom;
            high_raw = (float)(int)hd * logf((float)(int)orig_ctx_len / (beta_slow * 2.0f * pi)) / denom;
        }
        corr_low = fmaxf(0.0f, floorf(low_raw));
        corr_high = fminf((float)((int)hd - 1), ceilf(high_raw));
        const float inv_scale = 1.0f / freq_scale;
        attn_scale *= 1.0f + 0.1f * logf(inv_scale);
    }
    *attn_scale_out = attn_scale;
    *head_dim_out = (uint32_t)hd;
    for (size_t i = 0; i < hd / 2; ++i) {  // compute_rope_frequencies (rope.c:112-127), host powf like the reference
        const float freq = powf(theta, -((float)(2 * i) / (float)hd));
        float scale = freq_scale;
        if (ext_factor != 0.0f) {  // rope_yarn_ramp (rope.c:28-36)
            float d = corr_high - corr_low;
            if (d < 0.001f) {
                d = 0.001f;
            }
            const float y = ((float)i - corr_low) / d;
            const float ramp = 1.0f - fminf(1.0f, fmaxf(0.0f, y));
            const float mix = ramp * ext_factor;
            scale = freq_scale + mix * (1.0f - freq_scale);
        }
        freqs_out[i] = freq * scale;
    }
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_matmul_qkv_rope_quantized(marmot_hip_device_t *dev, int kind, const void *d_wq, const void *d_wk,
                                         const void *d_wv, const void *d_input, int in_dtype, size_t N, size_t K,
                                         size_t M, const void *d_bq, const void *d_bk, const void *d_bv,
                                         int bias_dtype, void *d_out_q, void *d_out_k, void *d_out_v, int out_dtype,
                                         const marmot_hip_rope_t *rope) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_wq == nullptr || d_wk == nullptr || d_wv == nullptr || d_input == nullptr || d_out_q == nullptr ||
        d_out_k == nullptr || d_out_v == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (!is_weight_kind(kind)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "QKV projection kernel not available for quant kind %d",
                         kind);
    }
    if (in_dtype != MARMOT_HIP_DTYPE_F32 && in_dtype != MARMOT_HIP_DTYPE_F16) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "QKV projection requires FLOAT32 or FLOAT16 activations");
    }
    if (out_dtype != in_dtype) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "QKV projection outputs must have the input dtype");
    }
    const bool any_bias = d_bq != nullptr || d_bk != nullptr || d_bv != nullptr;
    if (any_bias && bias_dtype != MARMOT_HIP_DTYPE_F32 && bias_dtype != MARMOT_HIP_DTYPE_F16) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "QKV projection bias must be FLOAT32 or FLOAT16");
    }
    if (K == 0 || M == 0) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "QKV projection dimension mismatch on K");
    }
    const bool roped = rope != nullptr && (rope->apply_to_q || rope->apply_to_k);
    if (roped) {
        if (rope->d_positions == nullptr || rope->d_freqs == nullptr) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RoPE needs positions and frequencies");
        }
        if (rope->positions_dtype != MARMOT_HIP_DTYPE_F32 && rope->positions_dtype != MARMOT_HIP_DTYPE_I32 &&
            rope->positions_dtype != MARMOT_HIP_DTYPE_I64) {
            return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "RoPE positions must be FLOAT32, INT32 or INT64");
        }
        if (rope->head_dim == 0 || (rope->head_dim & 1u) != 0u || M % rope->head_dim != 0) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RoPE head dimension must be even and divide M");
        }
        if (rope->rope_type != 0 && rope->rope_type != 1) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "RoPE type must be NORM (0) or NEOX (1)");
        }
    }
    if (N == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));
    // With the rotary epilogue and fp16 outputs the projections are kept in fp32 (workspace) until the rotation has
    // been applied, so that the store rounds once, after it.
    const bool stage32 = roped && out_dtype == MARMOT_HIP_DTYPE_F16;
    const size_t stage_bytes = stage32 ? ((3 * N * M * sizeof(float) + 255) & ~(size_t)255) : 0;
    const int mm_out_dtype = stage32 ? MARMOT_HIP_DTYPE_F32 : out_dtype;
    WeightSet ws;
    ws.count = 3;
    ws.w[0] = d_wq;
    ws.w[1] = d_wk;
    ws.w[2] = d_wv;
    ws.bias[0] = d_bq;
    ws.bias[1] = d_bk;
    ws.bias[2] = d_bv;
    ws.out[0] = d_out_q;
    ws.out[1] = d_out_k;
    ws.out[2] = d_out_v;
    ws.bias_dtype = bias_dtype;
    ws.bias_first = true;
    const bool mmq = mmq_supported(dev, kind, N, K, 3);
    if (mmq && kind == MARMOT_HIP_KIND_Q4_K && in_dtype == MARMOT_HIP_DTYPE_F32 && N <= 16 &&
        !dev->knobs.no_row_kernels && (((uintptr_t)d_input) & 15) == 0 &&
        mmq_rows_supported(dev, kind, N, K, M, 3, false)) {
        void *wsp_rows = nullptr;
        if (stage_bytes != 0) {
            const int rs = workspace_reserve(dev, stage_bytes, &wsp_rows);
            if (rs != MARMOT_HIP_SUCCESS) {
                return rs;
            }
            for (int i = 0; i < 3; ++i) {
                ws.out[i] = (float *)wsp_rows + (size_t)i * N * M;
            }
        }
        const int rs = launch_mmq_rows_q4k(dev, ws, (const float *)d_input, nullptr, N, K, M, mm_out_dtype);
        if (rs != MARMOT_HIP_SUCCESS || !roped) {
            return rs;
        }
        return qkv_rope_finish(dev, rope, stage32 ? (const float *)wsp_rows : nullptr, d_out_q, d_out_k, d_out_v, N, M,
                               out_dtype);
    }
    const bool fuse_quant = !mmq && in_dtype == MARMOT_HIP_DTYPE_F32 && matvec_can_fuse_quantization(dev, kind, N, K, d_input);
    const int act_kind = is_k_quant(kind) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    const size_t act_bytes =
        fuse_quant ? 0 : ((act_scratch_layout(act_kind, N, K, nullptr, nullptr) + 255) & ~(size_t)255);
    // Q2_K, Q3_K (from five rows on) and the 32-value formats but Q8_1 (from nine): the tiled int8 GEMMs, their K-split partial
    // sums where the mmq scratch would be
    const bool q80_kind = !fuse_quant && gemm_q80_kind(kind) && N >= gemm_q80_min_rows(kind) && K % QK_K == 0;
    const size_t mmq_bytes = mmq ? ((mmq_scratch_bytes(dev, kind, N, K, M, 3) + 255) & ~(size_t)255)
        : q80_kind               ? ((gemm_i8_scratch_bytes(dev, N, K, M, 3) + 255) & ~(size_t)255)
                                 : 0;
    void *wsp = nullptr;
    int st = MARMOT_HIP_SUCCESS;
    if (act_bytes + mmq_bytes + stage_bytes != 0) {
        st = workspace_reserve(dev, act_bytes + mmq_bytes + stage_bytes, &wsp);
        if (st != MARMOT_HIP_SUCCESS) {
            return st;
        }
    }
    float *stage = (float *)((uint8_t *)wsp + act_bytes + mmq_bytes);
    if (stage32) {
        for (int i = 0; i < 3; ++i) {
            ws.out[i] = stage + (size_t)i * N * M;
        }
    }
    if (fuse_quant) {
        st = launch_matvec_set(dev, kind, ws, nullptr, (const float *)d_input, N, K, M, mm_out_dtype);
    } else {
        ActScratch act;
        act_scratch_layout(act_kind, N, K, wsp, &act);
        st = launch_quantize_act_soa(dev, act_kind, d_input, in_dtype, N, K, act);
        if (st != MARMOT_HIP_SUCCESS) {
            return st;
        }
        st = MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
        if (mmq && kind == MARMOT_HIP_KIND_Q4_K && N <= 16 && !dev->knobs.no_row_kernels) {
            st = launch_mmq_rows_q4k(dev, ws, nullptr, &act, N, K, M, mm_out_dtype);
        }
        if (st != MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
            // the row-owning kernel took it
        } else if (mmq) {
            st = launch_mmq_set(dev, kind, ws, act, N, K, M, mm_out_dtype, (uint8_t *)wsp + act_bytes);
        } else if (q80_kind && gemm_q80_applies(dev, kind, N, K, ws.w, ws.count, act)) {
            st = launch_gemm_q80(dev, kind, ws, act, N, K, M, mm_out_dtype, (uint8_t *)wsp + act_bytes);
        } else {
            st = launch_matvec_set(dev, kind, ws, &act, nullptr, N, K, M, mm_out_dtype);
        }
    }
    if (st != MARMOT_HIP_SUCCESS || !roped) {
        return st;
    }
    return qkv_rope_finish(dev, rope, stage32 ? stage : nullptr, d_out_q, d_out_k, d_out_v, N, M, out_dtype);
}

} // extern "C"

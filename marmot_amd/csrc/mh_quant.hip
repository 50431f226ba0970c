// Dequantizers (bit-exact with the reference's CPU dequantizers) and activation quantizers
// (bit-exact with its Q8_0 / Q8_K activation packers).
//
// This file must be compiled with -ffp-contract=off: every fp32 multiply / subtract below is meant to
// round on its own, exactly as the reference's scalar CPU code does.
#include "mh_actquant.h"
#include "mh_dequant.h"

#include <float.h>

namespace mh {

// ------------------------------------------------------------------------------------------------
// Dequantize: one thread per output value; `kp` = padded row length (nb * block_values).
// ------------------------------------------------------------------------------------------------

template <int KIND>
__global__ __launch_bounds__(256) void k_dequantize(const uint8_t *__restrict__ blocks, float *__restrict__ out,
                                                    size_t rows, size_t k, size_t nb) {
    constexpr int BV = KindTraits<KIND>::BV;
    constexpr int BB = KindTraits<KIND>::BB;
    const size_t kp = nb * BV;
    const size_t total = rows * kp;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t row = idx / kp;
        const size_t col = idx - row * kp;
        if (col >= k) {
            continue;
        }
        const size_t b = col / BV;
        const int v = (int)(col - b * BV);
        const uint8_t *blk = blocks + (row * nb + b) * BB;
        const float y = dequant_value<KIND>(blk, v);
        out[row * k + col] = y;
    }
}

// ------------------------------------------------------------------------------------------------
// Embedding gather from a block-quantized table (embedding_scalar.c:241-303, 381-447): one thread per output value.
// ------------------------------------------------------------------------------------------------
template <int KIND>
__global__ __launch_bounds__(256) void k_embedding_gather(const uint8_t *__restrict__ table, size_t vocab, size_t dim,
                                                          const void *__restrict__ ids, int ids_are_i64,
                                                          void *__restrict__ out, int out_is_f16, float scale,
                                                          int padding_id, int *__restrict__ error_flag) {
    warm_kernel_arguments<72, 72>();
    constexpr int BV = KindTraits<KIND>::BV;
    constexpr int BB = KindTraits<KIND>::BB;
    const size_t idx = blockIdx.y;
    const size_t col = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (col >= dim) {
        return;
    }
    const long long token = ids_are_i64 ? ((const long long *)ids)[idx] : (long long)((const int *)ids)[idx];
    bool zero = padding_id >= 0 && token == (long long)padding_id;
    if (!zero && (token < 0 || (unsigned long long)token >= (unsigned long long)vocab)) {
        zero = true;
        if (error_flag != nullptr && col == 0) {
            atomicMax(error_flag, (int)(gridDim.y - idx));  // tokens - position: the maximum names the first offender
        }
    }
    float y = 0.0f;
    if (!zero) {
        const size_t nb = (dim + BV - 1) / BV;
        const size_t b = col / BV;
        const int v = (int)(col - b * BV);
        const uint8_t *blk = table + ((size_t)token * nb + b) * BB;
        if constexpr (KIND == MARMOT_HIP_KIND_Q4_0) {
            // the embedding path's own nibble order for Q4_0 (embedding_scalar.c:221-229)
            const uint8_t packed = blk[2 + (v >> 1)];
            const int q = ((v & 1) ? (packed >> 4) : (packed & 0x0f)) - 8;
            y = h2f((uint16_t)(blk[0] | (blk[1] << 8))) * (float)q;
        } else if constexpr (KIND == MARMOT_HIP_KIND_Q4_1) {
            // the same interleaved order for Q4_1 tables (embedding_scalar.c:231-240): scale * q + min, two roundings
            const uint8_t packed = blk[4 + (v >> 1)];
            const int q = (v & 1) ? (packed >> 4) : (packed & 0x0f);
            y = h2f((uint16_t)(blk[0] | (blk[1] << 8))) * (float)q + h2f((uint16_t)(blk[2] | (blk[3] << 8)));
        } else {
            y = dequant_value<KIND>(blk, v);
        }
    }
    if (out_is_f16) {
        // the product is rounded to fp32 on its own before the conversion: merged into one mixed-precision
        // multiply-add with a +0 addend, -0 * scale would come out as +0
        float t = y * scale;
        asm volatile("" : "+v"(t));
        ((uint16_t *)out)[idx * dim + col] = zero ? (uint16_t)0 : f2h(t);
    } else {
        ((float *)out)[idx * dim + col] = zero ? 0.0f : (scale == 1.0f ? y : y * scale);
    }
}

// ------------------------------------------------------------------------------------------------
// Activation quantizers
// ------------------------------------------------------------------------------------------------

// Where the values to quantize come from.
enum ActSource {
    SRC_F32 = 0,     // fp32 activations
    SRC_F16 = 1,     // fp16 activations, widened exactly
    SRC_SWIGLU = 2,  // silu(gate) * up of two fp32 arrays (MoE expert body, moe_ops.c:318-320, 552-556)
    SRC_GEGLU = 3,   // gelu(gate) * up
};

template <int SRC>
__device__ __forceinline__ float load_act_value(const void *x, const void *x2, size_t i) {
    if constexpr (SRC == SRC_F16) {
        return h2f(((const uint16_t *)x)[i]);
    } else if constexpr (SRC == SRC_SWIGLU) {
        const float g = ((const float *)x)[i];
        const float a = g / (1.0f + expf(-g));
        return a * ((const float *)x2)[i];
    } else if constexpr (SRC == SRC_GEGLU) {
        const float g = ((const float *)x)[i];
        const float a = 0.5f * g * (1.0f + erff(g * 0.70710678118654752440f));
        return a * ((const float *)x2)[i];
    } else {
        return ((const float *)x)[i];
    }
}

// Q8_K (matmul_quant_pack.c:106-142): one wavefront per 256-value block, 4 consecutive values per lane.
// AOS = marmot_q8_k_block_t output; otherwise the library's structure-of-arrays scratch.
// PER_WAVE consecutive blocks per wavefront, all of them requested before the first is quantized.
template <int SRC, bool AOS, int PER_WAVE>
__global__ __launch_bounds__(256) void k_quantize_q8_k(const void *__restrict__ x, const void *__restrict__ x2,
                                                       size_t rows, size_t k, size_t nb,
                                                       uint8_t *__restrict__ blocks_out, ActScratch soa) {
    warm_kernel_arguments<6 * 8 + sizeof(ActScratch), 6 * 8 + sizeof(ActScratch)>();
    const int lane = threadIdx.x & 63;
    const size_t first = ((size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * PER_WAVE;
    const size_t total = rows * nb;
    if (first >= total) {
        return;
    }
    float v[PER_WAVE][4];
#pragma unroll
    for (int w = 0; w < PER_WAVE; ++w) {
        const size_t id = first + w < total ? first + w : total - 1;  // beyond the end: re-read, never stored
        const size_t row = id / nb;
        const size_t b = id - row * nb;
        const size_t col0 = b * QK_K + (size_t)lane * 4;
        bool vec = false;
        if constexpr (SRC == SRC_F32) {
            // whole 16-byte groups inside the row: one load instead of four
            vec = (k & 3) == 0 && ((((uintptr_t)x) & 15) == 0) && col0 + 3 < k;
            if (vec) {
                const float4 f = *(const float4 *)((const float *)x + row * k + col0);
                v[w][0] = f.x;
                v[w][1] = f.y;
                v[w][2] = f.z;
                v[w][3] = f.w;
            }
        }
        if (!vec) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const size_t col = col0 + i;
                v[w][i] = col < k ? load_act_value<SRC>(x, x2, row * k + col) : 0.0f;
            }
        }
    }
#pragma unroll
    for (int w = 0; w < PER_WAVE; ++w) {
        if (first + w < total) {  // uniform over the wavefront
            const size_t id = first + w;
            const size_t row = id / nb;
            q8k_block_store<AOS>(v[w], lane, row, id - row * nb, nb, blocks_out, soa);
        }
    }
}

// Q8_0 (matmul_quant_pack.c:23-62, block.c:221-232 scalar): 32 lanes per block, one value per lane.
template <int SRC, bool AOS>
__global__ __launch_bounds__(256) void k_quantize_q8_0(const void *__restrict__ x, const void *__restrict__ x2,
                                                       size_t rows, size_t k, size_t nb,
                                                       uint8_t *__restrict__ blocks_out, ActScratch soa) {
    warm_kernel_arguments<6 * 8 + sizeof(ActScratch), 6 * 8 + sizeof(ActScratch)>();
    const int lane32 = threadIdx.x & 31;
    const size_t blk_id = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    if (blk_id >= rows * nb) {
        return;
    }
    const size_t row = blk_id / nb;
    const size_t b = blk_id - row * nb;
    const size_t col = b * QK + lane32;
    const float v = col < k ? load_act_value<SRC>(x, x2, row * k + col) : 0.0f;
    q8_0_block_store<AOS>(v, col < k, lane32, row, b, nb, blocks_out, soa);
}

// The same blocks into the structure-of-arrays scratch with eight lanes per block and four consecutive values per lane
// (one 16-byte load, one dword store) for rows of whole blocks: the maximum and the sum of 32 values do not depend on the
// order in which they are combined, and every value sees the expressions of q8_0_block_store, so the codes, scales and
// sums are the same bits. (One value per lane stores single bytes: 10.8 us for 512 x 4096 values against 4 us here.)
template <int SRC>
__global__ __launch_bounds__(256) void k_quantize_q8_0_x4(const void *__restrict__ x, const void *__restrict__ x2,
                                                          size_t rows, size_t k, size_t nb, ActScratch soa) {
    const int lane8 = threadIdx.x & 7;
    const size_t blk_id = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 3;
    if (blk_id >= rows * nb) {
        return;
    }
    const size_t row = blk_id / nb;
    const size_t b = blk_id - row * nb;
    const size_t i0 = row * k + b * QK + (size_t)(4 * lane8);
    float v[4];
    if constexpr (SRC == SRC_F32) {
        const float4 f = *(const float4 *)((const float *)x + i0);
        v[0] = f.x, v[1] = f.y, v[2] = f.z, v[3] = f.w;
    } else if constexpr (SRC == SRC_F16) {
        const uint2 h = *(const uint2 *)((const uint16_t *)x + i0);
        v[0] = h2f((uint16_t)(h.x & 0xffffu)), v[1] = h2f((uint16_t)(h.x >> 16));
        v[2] = h2f((uint16_t)(h.y & 0xffffu)), v[3] = h2f((uint16_t)(h.y >> 16));
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = load_act_value<SRC>(x, x2, i0 + i);
        }
    }
    float max_abs = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) {
        max_abs = fmaxf(max_abs, __shfl_xor(max_abs, off));
    }
    float scale = max_abs / 127.0f;
    if (scale < FLT_MIN) {
        scale = 1.0f;
    }
    const float inv_scale = 1.0f / scale;
    int s = 0;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int q = (int)roundf(v[i] * inv_scale);
        q = q < -127 ? -127 : (q > 127 ? 127 : q);
        s += q;
        packed |= ((uint32_t)q & 0xffu) << (8 * i);
    }
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) {
        s += __shfl_xor(s, off);
    }
    *(uint32_t *)(soa.qs + row * soa.kp + b * QK + (size_t)(4 * lane8)) = packed;
    if (lane8 == 0) {
        soa.d[row * nb + b] = h2f(f2h(scale));
        soa.sums[row * nb + b] = (int16_t)s;
    }
}

// Plain 16-byte copy: device-to-device copies of the library, and the known-traffic kernel that profiler
// counters (FETCH_SIZE / WRITE_SIZE) are calibrated against.
__global__ __launch_bounds__(256) void k_copy16(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) {
        dst[i] = src[i];
    }
}

// Read-only stream of 16-byte loads, 8 in flight per lane, each workgroup over one contiguous run of 32 KiB: what a
// kernel that only has to fetch its operand can reach. The loaded words are folded and stored only if they match a
// value the fold cannot produce from the all-ones test pattern, so nothing is written.
struct ReadProbeParams {
    const uint4 *src;
    uint32_t *sink;
    size_t n16;
    MH_TIMELINE_FIELD
};
__global__ __launch_bounds__(256) void k_read16(const ReadProbeParams p) {
    MH_MARK_DECL
    MH_MARK(p, 0);  // timeline: wavefront started
    const uint4 *__restrict__ src = p.src;
    uint32_t *sink = p.sink;
    const size_t n16 = p.n16;
    const size_t base = (size_t)blockIdx.x * 256 * 8 + threadIdx.x;
    uint4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const size_t idx = base + (size_t)i * 256;
        v[i] = idx < n16 ? src[idx] : make_uint4(0, 0, 0, 0);
    }
    MH_MARK(p, 1);  // loads issued
    uint32_t a = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    }
    if (a == 0x12345678u) {
        sink[threadIdx.x] = a;
    }
#if defined(MH_TIMELINE)
    asm volatile("" ::"v"(a));  // the marks below must not move above the fold: it is what waits for the loads
#endif
    MH_MARK(p, 2);  // data arrived
    MH_MARK_FLUSH(p);
}

__global__ void k_fill_bytes(uint8_t *dst, uint8_t value, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        dst[i] = value;
    }
}

template <int SRC, bool AOS>
static int launch_quantize_src(marmot_hip_device *dev, int act_kind, const void *d_x, const void *d_x2, size_t rows,
                               size_t k, uint8_t *blocks_out, const ActScratch &soa) {
    if (act_kind == MARMOT_HIP_KIND_Q8_K) {
        const size_t nb = (k + QK_K - 1) / QK_K;
        const size_t blocks = rows * nb;
        // one block per wavefront: the reductions inside a block are a chain of dependent steps, and many resident
        // wavefronts hide it better than several blocks in one wavefront (measured at 512 x 4096: 7.0 us against 9.0)
        const dim3 grid((unsigned)((blocks + 3) / 4));
        hipLaunchKernelGGL((k_quantize_q8_k<SRC, AOS, 1>), grid, dim3(256), 0, dev->stream, d_x, d_x2, rows, k, nb,
                           blocks_out, soa);
    } else {
        const size_t nb = (k + QK - 1) / QK;
        const size_t blocks = rows * nb;
        const size_t elem = SRC == SRC_F16 ? 2 : 4;
        const bool aligned = (((uintptr_t)d_x) % (4 * elem)) == 0 && (d_x2 == nullptr || (((uintptr_t)d_x2) & 15) == 0);
        if (!AOS && k % QK == 0 && aligned && (((uintptr_t)soa.qs) & 3) == 0 && soa.kp % 4 == 0) {
            const dim3 grid((unsigned)((blocks + 31) / 32));
            hipLaunchKernelGGL((k_quantize_q8_0_x4<SRC>), grid, dim3(256), 0, dev->stream, d_x, d_x2, rows, k, nb, soa);
        } else {
            const dim3 grid((unsigned)((blocks + 7) / 8));
            hipLaunchKernelGGL((k_quantize_q8_0<SRC, AOS>), grid, dim3(256), 0, dev->stream, d_x, d_x2, rows, k, nb,
                               blocks_out, soa);
        }
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

template <bool AOS>
static int launch_quantize(marmot_hip_device *dev, int act_kind, const void *d_x, int in_dtype, size_t rows, size_t k,
                           uint8_t *blocks_out, const ActScratch &soa) {
    if (rows == 0 || k == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (in_dtype == MARMOT_HIP_DTYPE_F16) {
        return launch_quantize_src<SRC_F16, AOS>(dev, act_kind, d_x, nullptr, rows, k, blocks_out, soa);
    }
    return launch_quantize_src<SRC_F32, AOS>(dev, act_kind, d_x, nullptr, rows, k, blocks_out, soa);
}

int launch_quantize_glu_soa(marmot_hip_device *dev, int act_kind, const float *d_gate, const float *d_up, bool geglu,
                            size_t rows, size_t k, const ActScratch &dst) {
    if (rows == 0 || k == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (geglu) {
        return launch_quantize_src<SRC_GEGLU, false>(dev, act_kind, d_gate, d_up, rows, k, nullptr, dst);
    }
    return launch_quantize_src<SRC_SWIGLU, false>(dev, act_kind, d_gate, d_up, rows, k, nullptr, dst);
}

int launch_quantize_act_soa(marmot_hip_device *dev, int act_kind, const void *d_x, int in_dtype, size_t rows, size_t k,
                            const ActScratch &dst) {
    return launch_quantize<false>(dev, act_kind, d_x, in_dtype, rows, k, nullptr, dst);
}

} // namespace mh

using namespace mh;

extern "C" {

int marmot_hip_copy16_internal(marmot_hip_device_t *dev, void *d_dst, const void *d_src, size_t size) {
    const size_t n16 = size / 16;
    size_t grid = (n16 + 255) / 256;
    if (grid > (size_t)1 << 20) {
        grid = (size_t)1 << 20;
    }
    hipLaunchKernelGGL(k_copy16, dim3((unsigned)grid), dim3(256), 0, dev->stream, (const uint4 *)d_src, (uint4 *)d_dst,
                       n16);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_read_probe(marmot_hip_device_t *dev, const void *d_src, size_t size, void *d_sink) {
    if (dev == nullptr || d_src == nullptr || d_sink == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "read_probe: null argument");
    }
    if (size % 16 != 0 || (((uintptr_t)d_src) & 15) != 0 || size == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "read_probe: size and address must be multiples of 16");
    }
    const size_t n16 = size / 16;
    const size_t grid = (n16 + 256 * 8 - 1) / (256 * 8);
    if (grid > 0x7fffffffu) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "read_probe: %zu bytes are more than one launch covers", size);
    }
    ReadProbeParams p;
    p.src = (const uint4 *)d_src;
    p.sink = (uint32_t *)d_sink;
    p.n16 = n16;
    MH_TIMELINE_SET(p, dev);
    hipLaunchKernelGGL(k_read16, dim3((unsigned)grid), dim3(256), 0, dev->stream, p);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

// One wavefront that stores the device's constant-rate 100 MHz counter: a time stamp inside a stream or a captured graph
__global__ void k_timestamp(unsigned long long *out) {
    if (threadIdx.x == 0) {
        *out = __builtin_amdgcn_s_memrealtime();
    }
}

int marmot_hip_timestamp(marmot_hip_device_t *dev, void *d_ticks) {
    if (dev == nullptr || d_ticks == nullptr || (((uintptr_t)d_ticks) & 7) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "timestamp: null or misaligned argument");
    }
    hipLaunchKernelGGL(k_timestamp, dim3(1), dim3(64), 0, dev->stream, (unsigned long long *)d_ticks);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_fill_bytes_internal(marmot_hip_device_t *dev, void *d_dst, int value, size_t size) {
    const unsigned grid = (unsigned)((size + 256 * 16 - 1) / (256 * 16));
    hipLaunchKernelGGL(k_fill_bytes, dim3(grid < 4096 ? (grid ? grid : 1) : 4096), dim3(256), 0, dev->stream,
                       (uint8_t *)d_dst, (uint8_t)value, size);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_dequantize(marmot_hip_device_t *dev, int kind, const void *d_blocks, size_t rows, size_t k,
                          float *d_out) {
    if (dev == nullptr || d_blocks == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "dequantize: null argument");
    }
    const size_t bv = block_values(kind);
    if (bv == 0) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "dequantize: unsupported quant kind %d", kind);
    }
    if (rows == 0 || k == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    const size_t nb = (k + bv - 1) / bv;
    const size_t total = rows * nb * bv;
    size_t g = (total + 255) / 256;
    if (g > 65536) {
        g = 65536;
    }
    const dim3 grid((unsigned)g), block(256);
    const uint8_t *src = (const uint8_t *)d_blocks;
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_K:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q4_K>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q5_K:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q5_K>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q2_K:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q2_K>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q3_K:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q3_K>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q6_K:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q6_K>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q8_0:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q8_0>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q4_0:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q4_0>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q8_1:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q8_1>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q4_1:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q4_1>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q5_0:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q5_0>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q5_1:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q5_1>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    case MARMOT_HIP_KIND_Q8_K:
        hipLaunchKernelGGL((k_dequantize<MARMOT_HIP_KIND_Q8_K>), grid, block, 0, dev->stream, src, d_out, rows, k, nb);
        break;
    default:
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "dequantize: unsupported quant kind %d", kind);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_quantize_activations(marmot_hip_device_t *dev, int act_kind, const void *d_x, int in_dtype,
                                    size_t rows, size_t k, void *d_blocks_out) {
    if (dev == nullptr || d_x == nullptr || d_blocks_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "quantize_activations: null argument");
    }
    if (act_kind != MARMOT_HIP_KIND_Q8_0 && act_kind != MARMOT_HIP_KIND_Q8_K) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "quantize_activations: kind %d is not Q8_0/Q8_K",
                         act_kind);
    }
    if (in_dtype != MARMOT_HIP_DTYPE_F32 && in_dtype != MARMOT_HIP_DTYPE_F16) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "quantize_activations: input dtype %d", in_dtype);
    }
    ActScratch none;
    return launch_quantize<true>(dev, act_kind, d_x, in_dtype, rows, k, (uint8_t *)d_blocks_out, none);
}

int marmot_hip_embedding_gather_quantized(marmot_hip_device_t *dev, int kind, const void *d_table, size_t vocab,
                                          size_t dim, const void *d_ids, int ids_dtype, size_t n, void *d_out,
                                          int out_dtype, float scale, int32_t padding_id, int bounds_check) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_table == nullptr || d_ids == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "Tensor argument must not be null");
    }
    if (!is_weight_kind(kind)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "embedding gather: unsupported quant kind %d", kind);
    }
    if (ids_dtype != MARMOT_HIP_DTYPE_I32 && ids_dtype != MARMOT_HIP_DTYPE_I64) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "embedding gather: token ids must be INT32 or INT64");
    }
    if (out_dtype != MARMOT_HIP_DTYPE_F32 && out_dtype != MARMOT_HIP_DTYPE_F16) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "embedding gather: output must be FLOAT32 or FLOAT16");
    }
    if (n == 0 || dim == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (n > 65535) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "embedding gather: more than 65535 tokens per call");
    }
    MH_HIP(hipSetDevice(dev->device_index));
    // Out-of-range tokens are reported through a device flag that is read back after the launch; that needs a
    // stream synchronization and is skipped while the stream is being captured into a graph (rows are zeroed then).
    int *flag = nullptr;
    if (bounds_check != 0 && !dev->capturing) {
        void *ws = nullptr;
        const int st = workspace_reserve(dev, 256, &ws);
        if (st != MARMOT_HIP_SUCCESS) {
            return st;
        }
        flag = (int *)ws;
        MH_HIP(hipMemsetAsync(flag, 0, sizeof(int), dev->stream));
    }
    const dim3 grid((unsigned)((dim + 255) / 256), (unsigned)n), block(256);
    const uint8_t *table = (const uint8_t *)d_table;
    const int i64 = ids_dtype == MARMOT_HIP_DTYPE_I64, f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_K:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q4_K>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q5_K:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q5_K>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q2_K:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q2_K>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q3_K:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q3_K>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q6_K:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q6_K>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q8_0:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q8_0>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q8_1:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q8_1>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q5_0:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q5_0>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q5_1:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q5_1>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    case MARMOT_HIP_KIND_Q4_1:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q4_1>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    default:
        hipLaunchKernelGGL((k_embedding_gather<MARMOT_HIP_KIND_Q4_0>), grid, block, 0, dev->stream, table, vocab, dim,
                           d_ids, i64, d_out, f16, scale, (int)padding_id, flag);
        break;
    }
    MH_HIP(hipGetLastError());
    if (flag != nullptr) {
        int host_flag = 0;
        MH_HIP(hipMemcpyAsync(&host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, dev->stream));
        MH_HIP(hipStreamSynchronize(dev->stream));
        if (host_flag != 0) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT,
                             "embedding gather: token id at position %zu is out of range", n - (size_t)host_flag);
        }
    }
    return MARMOT_HIP_SUCCESS;
}

} // extern "C"

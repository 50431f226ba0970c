// K-quant weight quantizers on the device: fp32 rows -> Q4_K / Q5_K / Q6_K blocks, bit for bit what the reference's
// CPU quantizers write (q4k_gguf.c:35-131, q5k_gguf.c:35-160, q6k_gguf.c:35-61 with kquant_common.h:39-130, 150-236,
// 310-369). This is model preparation, not a per-token path: the kernels keep every floating-point sum in the
// reference's element order (one thread walks one sub-block from its first value to its last) and parallelize only
// across sub-blocks and blocks; the file is compiled without contraction, with correctly rounded division and square
// root, like the dequantizers.
#include "mh_common.h"

namespace mh {

// (uint8_t)nearbyintf(v) as the reference's x86 build evaluates it: through a 32-bit integer, then the low byte
__device__ __forceinline__ uint32_t round_to_u8(float v) {
    return (uint32_t)(int32_t)rintf(v) & 0xffu;
}

// kquant_common.h:142-148
__device__ __forceinline__ int nearest_int_magic(float value) {
    const float shifted = value + 12582912.0f;
    return (__float_as_int(shifted) & 0x007fffff) - 0x00400000;
}

// make_qkx2_quants (kquant_common.h:39-130) with squared error, for one sub-block of 32 values held by one thread.
// Returns the scale; *the_min receives -min; L the levels 0 .. nmax.
__device__ float qkx2_search32(int nmax, const float (&x)[32], const float (&w)[32], int (&L)[32], float *the_min,
                               float rmin, float rdelta, int nstep) {
    float mn = x[0], mx = x[0];
    float sum_w = w[0];
    float sum_x = sum_w * x[0];
#pragma unroll
    for (int i = 1; i < 32; ++i) {
        if (x[i] < mn) {
            mn = x[i];
        }
        if (x[i] > mx) {
            mx = x[i];
        }
        sum_w += w[i];
        sum_x += w[i] * x[i];
    }
    if (mn > 0.0f) {
        mn = 0.0f;
    }
    if (mx == mn) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            L[i] = 0;
        }
        *the_min = -mn;
        return 0.0f;
    }
    float iscale = (float)nmax / (mx - mn);
    float scale = 1.0f / iscale;
    float best_error = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        int l = (int)rintf(iscale * (x[i] - mn));
        l = l > nmax ? nmax : (l < 0 ? 0 : l);
        L[i] = l;
        float diff = scale * (float)l + mn - x[i];
        diff = diff * diff;
        best_error += w[i] * diff;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (mx - mn);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        int aux[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            int l = (int)rintf(iscale * (x[i] - mn));
            l = l > nmax ? nmax : (l < 0 ? 0 : l);
            aux[i] = l;
            const float fl = (float)l;
            sum_l += w[i] * fl;
            sum_l2 += w[i] * fl * fl;
            sum_xl += w[i] * fl * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0.0f) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                float diff = this_scale * (float)aux[i] + this_min - x[i];
                diff = diff * diff;
                cur_error += w[i] * diff;
            }
            if (cur_error < best_error) {
#pragma unroll
                for (int i = 0; i < 32; ++i) {
                    L[i] = aux[i];
                }
                best_error = cur_error;
                scale = this_scale;
                mn = this_min;
            }
        }
    }
    *the_min = -mn;
    return scale;
}

// Q4_K (BITS 4) and Q5_K (BITS 5): eight threads per 256-value block, one per 32-value sub-block; eight blocks per
// workgroup. Levels pass through LDS for the interleaved nibble / fifth-bit packing.
template <int BITS>
__global__ __launch_bounds__(64) void k_quantize_q45_k(const float *__restrict__ x, size_t rows, size_t k, size_t nb,
                                                       uint8_t *__restrict__ out) {
    constexpr int NMAX = BITS == 4 ? 15 : 31;
    constexpr int BLOCK_BYTES = BITS == 4 ? Q4_K_BYTES : Q5_K_BYTES;
    __shared__ uint8_t levels[8][QK_K];
    const int t = threadIdx.x, jb = t >> 3, j = t & 7;
    const size_t total = rows * nb;
    const size_t qb = (size_t)blockIdx.x * 8 + (size_t)jb;
    const bool valid = qb < total;
    const size_t row = valid ? qb / nb : 0, b = valid ? qb % nb : 0;
    const size_t start = b * QK_K;
    const uint32_t elems = valid ? (uint32_t)(start + QK_K <= k ? QK_K : k - start) : 0u;

    float xv[32];
#pragma unroll
    for (int l = 0; l < 32; ++l) {
        const uint32_t i = 32u * (uint32_t)j + (uint32_t)l;
        xv[l] = i < elems ? x[row * k + start + i] : 0.0f;
    }
    // weights of the search: average magnitude of the sub-block plus |x|
    float sum_x2 = 0.0f;
#pragma unroll
    for (int l = 0; l < 32; ++l) {
        sum_x2 += xv[l] * xv[l];
    }
    const float av_x = sqrtf(sum_x2 / 32.0f);
    float wv[32];
#pragma unroll
    for (int l = 0; l < 32; ++l) {
        wv[l] = av_x + fabsf(xv[l]);
    }
    int L[32];
    float my_min;
    const float my_scale =
        BITS == 4 ? qkx2_search32(NMAX, xv, wv, L, &my_min, -1.0f, 0.1f, 20) : qkx2_search32(NMAX, xv, wv, L, &my_min, -0.5f, 0.1f, 15);

    // block maxima in sub-block order, 6-bit scale / min of every sub-block
    const int base = t & ~7;
    float max_scale = 0.0f, max_min = 0.0f;
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
        const float s = __shfl(my_scale, base + jj);
        const float m = __shfl(my_min, base + jj);
        if (s > max_scale) {
            max_scale = s;
        }
        if (m > max_min) {
            max_min = m;
        }
    }
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint32_t ls = round_to_u8(inv_scale * my_scale);
    uint32_t lm = round_to_u8(inv_min * my_min);
    ls = ls > 63u ? 63u : ls;
    lm = lm > 63u ? 63u : lm;
    const uint16_t d_h = f2h(max_scale / 63.0f);
    const uint16_t dmin_h = f2h(max_min / 63.0f);
    const uint32_t ls_hi = (uint32_t)__shfl((int)ls, base + ((j + 4) & 7));  // sub-block j + 4, read by j < 4
    const uint32_t lm_hi = (uint32_t)__shfl((int)lm, base + ((j + 4) & 7));

    // levels again with the stored (rounded) scale and min; a sub-block whose stored scale is zero keeps the search's
    const float d = h2f(d_h) * (float)ls;
    if (d != 0.0f) {
        const float dm = h2f(dmin_h) * (float)lm;
#pragma unroll
        for (int l = 0; l < 32; ++l) {
            int q = (int)rintf((xv[l] + dm) / d);
            q = q > NMAX ? NMAX : (q < 0 ? 0 : q);
            L[l] = q;
        }
    }
#pragma unroll
    for (int l = 0; l < 32; ++l) {
        levels[jb][32 * j + l] = (uint8_t)L[l];
    }
    __syncthreads();
    if (!valid) {
        return;
    }
    uint8_t *blk = out + qb * BLOCK_BYTES;
    if (j == 0) {
        *(uint16_t *)blk = d_h;
        *(uint16_t *)(blk + 2) = dmin_h;
    }
    if (j < 4) {  // get_scale_min_k4 packing (kquant_common.h:29-37 read backwards)
        blk[4 + j] = (uint8_t)(ls | ((ls_hi >> 4) << 6));
        blk[4 + j + 4] = (uint8_t)(lm | ((lm_hi >> 4) << 6));
        blk[4 + j + 8] = (uint8_t)((ls_hi & 0xFu) | ((lm_hi & 0xFu) << 4));
    }
    const uint8_t *lv = levels[jb];
    const uint32_t qs_offset = (elems + 1u) / 2u;  // bytes from here on are zero in a partial block
    uint8_t *qs = blk + (BITS == 4 ? 16 : 48);
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const uint32_t i = 16u * (uint32_t)j + (uint32_t)c;  // byte of qs: group i / 32, position i % 32
        const uint32_t g = i >> 5, l = i & 31u;
        uint32_t l1 = lv[64 * g + l], l2 = lv[64 * g + l + 32];
        if (BITS == 5) {
            l1 = l1 > 15u ? l1 - 16u : l1;
            l2 = l2 > 15u ? l2 - 16u : l2;
        }
        const uint32_t v = l1 | (l2 << 4);
        qs[i] = (uint8_t)(i < qs_offset ? v : 0u);
    }
    if (BITS == 5) {
        uint8_t *qh = blk + 16;
        // a partial block keeps (elems + 63) / 64 bytes of qh, as the reference does; a full block keeps all 32
        const uint32_t qh_offset = elems < (uint32_t)QK_K ? (elems + 63u) / 64u : 32u;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t jj = 4u * (uint32_t)j + (uint32_t)c;
            uint32_t bits = 0;
#pragma unroll
            for (uint32_t g = 0; g < 4; ++g) {
                bits |= (lv[64 * g + jj] > 15u ? 1u : 0u) << (2 * g);
                bits |= (lv[64 * g + jj + 32] > 15u ? 2u : 0u) << (2 * g);
            }
            qh[jj] = (uint8_t)(jj < qh_offset ? bits : 0u);
        }
    }
}

__device__ __forceinline__ int clamp_qx(int v, int nmax) {
    return v > nmax - 1 ? nmax - 1 : (v < -nmax ? -nmax : v);
}

// make_qx_quants with rmse_type 1 and no weights (kquant_common.h:150-236) for 16 values, nmax 32
__device__ float qx_search16(const float (&x)[16], int (&L)[16]) {
    constexpr int nmax = 32;
    float mx = 0.0f, amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            mx = x[i];
        }
    }
    if (amax < 1e-15f) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            L[i] = 0;
        }
        return 0.0f;
    }
    const float iscale = -((float)nmax) / mx;
    float sumlx = 0.0f, suml2 = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int l = clamp_qx(nearest_int_magic(iscale * x[i]), nmax);
        L[i] = l + nmax;
        const float w = x[i] * x[i];
        sumlx += w * x[i] * (float)l;
        suml2 += w * (float)l * (float)l;
    }
    float scale = suml2 > 0.0f ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) {
            continue;
        }
        const float trial_iscale = -((float)nmax + 0.1f * (float)is) / mx;
        float trial_sumlx = 0.0f, trial_suml2 = 0.0f;
        int aux[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int l = clamp_qx(nearest_int_magic(trial_iscale * x[i]), nmax);
            aux[i] = l;
            const float w = x[i] * x[i];
            trial_sumlx += w * x[i] * (float)l;
            trial_suml2 += w * (float)l * (float)l;
        }
        if (trial_suml2 > 0.0f && trial_sumlx * trial_sumlx > best * trial_suml2) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                L[i] = aux[i] + nmax;
            }
            scale = trial_sumlx / trial_suml2;
            best = scale * trial_sumlx;
        }
    }
    return scale;
}

// Q6_K: sixteen threads per 256-value block, one per 16-value sub-block; four blocks per workgroup
__global__ __launch_bounds__(64) void k_quantize_q6_k(const float *__restrict__ x, size_t rows, size_t k, size_t nb,
                                                      uint8_t *__restrict__ out) {
    __shared__ uint8_t levels[4][QK_K];
    __shared__ float sub_scales[4][16];
    const int t = threadIdx.x, jb = t >> 4, s = t & 15;
    const size_t total = rows * nb;
    const size_t qb = (size_t)blockIdx.x * 4 + (size_t)jb;
    const bool valid = qb < total;
    const size_t row = valid ? qb / nb : 0, b = valid ? qb % nb : 0;
    const size_t start = b * QK_K;
    const uint32_t elems = valid ? (uint32_t)(start + QK_K <= k ? QK_K : k - start) : 0u;

    float xv[16];
#pragma unroll
    for (int l = 0; l < 16; ++l) {
        const uint32_t i = 16u * (uint32_t)s + (uint32_t)l;
        xv[l] = i < elems ? x[row * k + start + i] : 0.0f;
    }
    int L[16];
    const float my_scale = qx_search16(xv, L);
    sub_scales[jb][s] = my_scale;
    __syncthreads();
    // the scale of largest magnitude, first occurrence in sub-block order
    float max_scale = 0.0f, max_abs_scale = 0.0f;
#pragma unroll
    for (int ib = 0; ib < 16; ++ib) {
        const float sc = sub_scales[jb][ib];
        const float a = fabsf(sc);
        if (a > max_abs_scale) {
            max_abs_scale = a;
            max_scale = sc;
        }
    }
    const bool zero_block = max_abs_scale < 1e-15f;
    uint16_t d_h = 0;
    int sc8 = 0;
    if (!zero_block) {
        const float iscale = -128.0f / max_scale;
        d_h = f2h(1.0f / iscale);
        sc8 = nearest_int_magic(iscale * my_scale);
        sc8 = sc8 > 127 ? 127 : (sc8 < -128 ? -128 : sc8);
        const float d = h2f(d_h) * (float)sc8;
        if (d != 0.0f) {
#pragma unroll
            for (int l = 0; l < 16; ++l) {
                L[l] = clamp_qx(nearest_int_magic(xv[l] / d), 32) + 32;
            }
        }
    }
#pragma unroll
    for (int l = 0; l < 16; ++l) {
        levels[jb][16 * s + l] = (uint8_t)(zero_block ? 0 : L[l]);
    }
    __syncthreads();
    if (!valid) {
        return;
    }
    uint8_t *blk = out + qb * Q6_K_BYTES;  // ql[128], qh[64], scales[16], d
    const uint8_t *lv = levels[jb];
    const uint32_t ql_offset = (elems + 1u) / 2u, qh_offset = (elems + 3u) / 4u;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint32_t i = 8u * (uint32_t)s + (uint32_t)c;  // byte of ql: half i / 64, upper pair (i % 64) / 32
        const uint32_t h = i >> 6, up = (i >> 5) & 1u, l = i & 31u;
        const uint32_t lo = lv[128 * h + 32 * up + l] & 0xFu, hi = lv[128 * h + 32 * up + l + 64] & 0xFu;
        blk[i] = (uint8_t)(!zero_block && i < ql_offset ? (lo | (hi << 4)) : 0u);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t i = 4u * (uint32_t)s + (uint32_t)c;  // byte of qh: half i / 32
        const uint32_t h = i >> 5, l = i & 31u;
        const uint32_t v = (uint32_t)(lv[128 * h + l] >> 4) | ((uint32_t)(lv[128 * h + l + 32] >> 4) << 2) |
            ((uint32_t)(lv[128 * h + l + 64] >> 4) << 4) | ((uint32_t)(lv[128 * h + l + 96] >> 4) << 6);
        blk[128 + i] = (uint8_t)(!zero_block && i < qh_offset ? v : 0u);
    }
    blk[192 + s] = (uint8_t)(int8_t)(zero_block ? 0 : sc8);
    if (s == 0) {
        blk[208] = (uint8_t)(d_h & 0xffu);
        blk[209] = (uint8_t)(d_h >> 8);
    }
}

} // namespace mh

using namespace mh;

int marmot_hip_quantize_weights(marmot_hip_device_t *dev, int kind, const float *d_x, size_t rows, size_t k,
                                void *d_blocks_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_blocks_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "quantize_weights: null argument");
    }
    if (kind != MARMOT_HIP_KIND_Q4_K && kind != MARMOT_HIP_KIND_Q5_K && kind != MARMOT_HIP_KIND_Q6_K) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "quantize_weights: kind %d is not Q4_K / Q5_K / Q6_K", kind);
    }
    if (rows == 0 || k == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    const size_t nb = (k + QK_K - 1) / QK_K;
    size_t total = 0;
    if (__builtin_mul_overflow(rows, nb, &total) || total > (size_t)0x7fffffff * 4) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "quantize_weights: too many blocks");
    }
    MH_HIP(hipSetDevice(dev->device_index));
    uint8_t *out = (uint8_t *)d_blocks_out;
    if (kind == MARMOT_HIP_KIND_Q6_K) {
        hipLaunchKernelGGL(k_quantize_q6_k, dim3((unsigned)((total + 3) / 4)), dim3(64), 0, dev->stream, d_x, rows, k, nb,
                           out);
    } else if (kind == MARMOT_HIP_KIND_Q4_K) {
        hipLaunchKernelGGL(k_quantize_q45_k<4>, dim3((unsigned)((total + 7) / 8)), dim3(64), 0, dev->stream, d_x, rows, k,
                           nb, out);
    } else {
        hipLaunchKernelGGL(k_quantize_q45_k<5>, dim3((unsigned)((total + 7) / 8)), dim3(64), 0, dev->stream, d_x, rows, k,
                           nb, out);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

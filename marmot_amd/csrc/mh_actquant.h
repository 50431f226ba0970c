// Per-block activation quantizers shared by the stand-alone quantization kernels and the kernels that produce
// quantized activations directly (normalization, gated products).
#pragma once
#include "mh_common.h"

#include <float.h>

namespace mh {

// One 256-value block of Q8_K activations (matmul_quant_pack.c:106-142) by one wavefront: lane l holds values
// 4 l .. 4 l + 3 of the block (zero beyond the row's end). AOS: marmot_q8_k_block_t output; otherwise the library's
// structure-of-arrays scratch.
template <bool AOS>
__device__ __forceinline__ void q8k_block_store(const float (&v)[4], int lane, size_t row, size_t b, size_t nb,
                                                uint8_t *__restrict__ blocks_out, const ActScratch &soa) {
    // value of largest magnitude, first occurrence wins (strict > in index order)
    float best_abs = 0.0f;
    float best_val = 0.0f;
    int best_idx = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float ax = fabsf(v[i]);
        if (ax > best_abs) {
            best_abs = ax;
            best_val = v[i];
            best_idx = lane * 4 + i;
        }
    }
    // Across the wavefront: the largest magnitude by data-parallel-primitive moves inside each row of 16 lanes (no LDS
    // round trips) and a scalar maximum over the four rows; the first lane that holds it is the lowest index, since
    // lanes hold consecutive values; its signed value comes over as a scalar.
    float wmax = best_abs;
    wmax = fmaxf(wmax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, wmax), 0xB1, 0xF, 0xF, true)));
    wmax = fmaxf(wmax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, wmax), 0x4E, 0xF, 0xF, true)));
    wmax = fmaxf(wmax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, wmax), 0x141, 0xF, 0xF, true)));
    wmax = fmaxf(wmax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, wmax), 0x140, 0xF, 0xF, true)));
    {
        const int wi = __builtin_bit_cast(int, wmax);
        const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(wi, 0));
        const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(wi, 16));
        const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(wi, 32));
        const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(wi, 48));
        wmax = fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
    }
    const unsigned long long holders = __ballot(best_abs == wmax);
    const int first = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(holders | (1ull << 63)));
    best_val = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, best_val), first));
    best_abs = wmax;
    (void)best_idx;

    int q[4] = {0, 0, 0, 0};
    float d = 0.0f;
    if (best_abs > 0.0f) {
        const float iscale = -127.0f / best_val;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int t = nearest_int_clamped(iscale * v[i]);
            q[i] = t > 127 ? 127 : t;
        }
        d = 1.0f / iscale;
    }
    int s = q[0] + q[1] + q[2] + q[3];
    s += __builtin_amdgcn_update_dpp(0, s, 0xB1, 0xF, 0xF, true);  // lane ^ 1
    s += __builtin_amdgcn_update_dpp(0, s, 0x4E, 0xF, 0xF, true);  // lane ^ 2: lanes 4j..4j+3 hold the sum of values 16j..16j+15
    const uint32_t packed = (uint32_t)(uint8_t)(int8_t)q[0] | ((uint32_t)(uint8_t)(int8_t)q[1] << 8) |
        ((uint32_t)(uint8_t)(int8_t)q[2] << 16) | ((uint32_t)(uint8_t)(int8_t)q[3] << 24);

    if constexpr (AOS) {
        uint8_t *blk = blocks_out + (row * nb + b) * Q8_K_BYTES;
        __builtin_memcpy(blk + 4 + lane * 4, &packed, 4);
        if ((lane & 3) == 0) {
            const int16_t bs = (int16_t)s;
            __builtin_memcpy(blk + 4 + 256 + (lane >> 2) * 2, &bs, 2);
        }
        if (lane == 0) {
            __builtin_memcpy(blk, &d, 4);
        }
    } else {
        *(uint32_t *)(soa.qs + row * soa.kp + b * QK_K + lane * 4) = packed;
        if ((lane & 3) == 0) {
            soa.sums[(row * nb + b) * 16 + (lane >> 2)] = (int16_t)s;
        }
        if (lane == 0) {
            soa.d[row * nb + b] = d;
        }
    }
}

// One 32-value block of Q8_0 activations (matmul_quant_pack.c:23-62, block.c:221-232 scalar) by 32 adjacent lanes, one
// value per lane (in_range false beyond the row's end: the value is zero and so is its code).
template <bool AOS>
__device__ __forceinline__ void q8_0_block_store(float v, bool in_range, int lane32, size_t row, size_t b, size_t nb,
                                                 uint8_t *__restrict__ blocks_out, const ActScratch &soa) {
    float max_abs = fabsf(v);
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) {
        max_abs = fmaxf(max_abs, __shfl_xor(max_abs, off));
    }
    float scale = max_abs / 127.0f;
    if (scale < FLT_MIN) {
        scale = 1.0f;
    }
    const float inv_scale = 1.0f / scale;
    int q = (int)roundf(v * inv_scale);
    q = q < -127 ? -127 : (q > 127 ? 127 : q);
    if (!in_range) {
        q = 0;
    }
    int s = q;
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) {
        s += __shfl_xor(s, off);
    }
    const uint16_t hs = f2h(scale);
    if constexpr (AOS) {
        uint8_t *blk = blocks_out + (row * nb + b) * Q8_0_BYTES;
        blk[2 + lane32] = (uint8_t)(int8_t)q;
        if (lane32 == 0) {
            __builtin_memcpy(blk, &hs, 2);
        }
    } else {
        soa.qs[row * soa.kp + b * QK + lane32] = (int8_t)q;
        if (lane32 == 0) {
            soa.d[row * nb + b] = h2f(hs);
            soa.sums[row * nb + b] = (int16_t)s;
        }
    }
}

} // namespace mh

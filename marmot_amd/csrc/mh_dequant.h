// Per-value dequantizers shared by the dequantize kernels and the direct (unquantized-activation) matmul
// route. Arithmetic and operation order follow the reference's CPU dequantizers exactly; translation units
// that include this header must be compiled with -ffp-contract=off.
#pragma once

#include "mh_common.h"

namespace mh {

// Q4_K (q4k_gguf.c:133-166): d1 = d*sc; m1 = dmin*m; y = d1*q - m1
__device__ __forceinline__ float dequant_value_q4_k(const uint8_t *blk, int v) {
    const BlockQ4_K *b = (const BlockQ4_K *)blk;
    const int j = v >> 5;          // sub-block 0..7
    const int l = v & 31;
    const int g = j >> 1;          // 64-value group
    uint8_t sc, m;
    const uint8_t *s = b->scales;
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (uint8_t)((s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4));
        m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
    const float d = h2f(b->d);
    const float dmin = h2f(b->dmin);
    const float d1 = d * (float)sc;
    const float m1 = dmin * (float)m;
    const uint8_t byte = b->qs[32 * g + l];
    const int q = (j & 1) ? (byte >> 4) : (byte & 0xF);
    return d1 * (float)q - m1;
}

// Q2_K (q2k_gguf.c:113-149): y = (d * sc) * q - dmin * m; group v / 16 holds sc | m << 4
__device__ __forceinline__ float dequant_value_q2_k(const uint8_t *blk, int v) {
    const BlockQ2_K *b = (const BlockQ2_K *)blk;
    const int c = v >> 7, j = (v >> 5) & 3, l = v & 31;
    const uint8_t sc = b->scales[v >> 4];
    const float dl = h2f(b->d) * (float)(sc & 0xF);
    const float ml = h2f(b->dmin) * (float)(sc >> 4);
    const int q = (b->qs[32 * c + l] >> (2 * j)) & 3;
    return dl * (float)q - ml;
}

// the six-bit scale of group is (0..15) of a Q3_K block, offset 32 removed (q3k_gguf.c:140-149)
__device__ __forceinline__ int q3k_group_scale(const uint8_t *scales, int is) {
    const int low = is < 8 ? (scales[is] & 0xF) : (scales[is - 8] >> 4);
    const int high = (scales[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
    return (low | (high << 4)) - 32;
}

// Q3_K (q3k_gguf.c:126-175): y = (d * sc) * (q2 - (high bit set ? 0 : 4))
__device__ __forceinline__ float dequant_value_q3_k(const uint8_t *blk, int v) {
    const BlockQ3_K *b = (const BlockQ3_K *)blk;
    const int c = v >> 7, j = (v >> 5) & 3, l = v & 31;
    const float dl = h2f(b->d) * (float)q3k_group_scale(b->scales, v >> 4);
    const int q2 = (b->qs[32 * c + l] >> (2 * j)) & 3;
    const int q = q2 - (((b->hmask[l] >> (v >> 5)) & 1) ? 0 : 4);
    return dl * (float)q;
}

// Q5_K (q5k_gguf.c:162-198): the Q4_K formula with a fifth bit from qh
__device__ __forceinline__ float dequant_value_q5_k(const uint8_t *blk, int v) {
    const BlockQ5_K *b = (const BlockQ5_K *)blk;
    const int j = v >> 5;
    const int l = v & 31;
    const int g = j >> 1;
    uint8_t sc, m;
    const uint8_t *s = b->scales;
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (uint8_t)((s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4));
        m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
    const float d = h2f(b->d);
    const float dmin = h2f(b->dmin);
    const float d1 = d * (float)sc;
    const float m1 = dmin * (float)m;
    const uint8_t byte = b->qs[32 * g + l];
    const int q = ((j & 1) ? (byte >> 4) : (byte & 0xF)) | (((b->qh[l] >> j) & 1) << 4);
    return d1 * (float)q - m1;
}

// Q6_K (q6k_gguf.c:63-99): y = (d * sc) * q
__device__ __forceinline__ float dequant_value_q6_k(const uint8_t *blk, int v) {
    const BlockQ6_K *b = (const BlockQ6_K *)blk;
    const int hh = v >> 7;         // half 0..1
    const int w = v & 127;
    const int j = w >> 5;          // 0..3: which of q1..q4
    const int l = w & 31;
    const uint8_t *ql = b->ql + 64 * hh;
    const uint8_t *qh = b->qh + 32 * hh;
    const int8_t *sc = b->scales + 8 * hh;
    const uint8_t lo = (j & 1) ? ql[l + 32] : ql[l];
    const int nib = (j & 2) ? (lo >> 4) : (lo & 0xF);
    const int hi2 = (qh[l] >> (2 * j)) & 3;
    const int q = (int)(int8_t)(nib | (hi2 << 4)) - 32;
    const float d = h2f(b->d);
    return d * (float)sc[(l >> 4) + 2 * j] * (float)q;
}

// Q8_0 (q8_gguf.c:189-200): y = (float)q * scale
__device__ __forceinline__ float dequant_value_q8_0(const uint8_t *blk, int v) {
    const BlockQ8_0 *b = (const BlockQ8_0 *)blk;
    return (float)b->qs[v] * h2f(b->scale);
}

// Q8_1 (q8_gguf.c:202-213): y = (float)q * scale
__device__ __forceinline__ float dequant_value_q8_1(const uint8_t *blk, int v) {
    const BlockQ8_1 *b = (const BlockQ8_1 *)blk;
    return (float)b->qs[v] * h2f(b->scale);
}

// Q4_0 (q4_gguf.c:367-394): y = (q - 8) * scale
__device__ __forceinline__ float dequant_value_q4_0(const uint8_t *blk, int v) {
    const BlockQ4_0 *b = (const BlockQ4_0 *)blk;
    const uint8_t packed = b->qs[v & 15];
    const int q = (v < 16) ? (packed & 0x0F) : (packed >> 4);
    return (float)(q - 8) * h2f(b->scale);
}

// Q4_1 (q4_gguf.c:396-424): y = q * scale + min
__device__ __forceinline__ float dequant_value_q4_1(const uint8_t *blk, int v) {
    const BlockQ4_1 *b = (const BlockQ4_1 *)blk;
    const uint8_t packed = b->qs[v & 15];
    const int q = (v < 16) ? (packed & 0x0F) : (packed >> 4);
    return (float)q * h2f(b->scale) + h2f(b->min);
}

// the five-bit value v of a Q5_0 / Q5_1 block: nibble v % 16 (low for v < 16) plus bit v of qh (q5_gguf.c:255-265)
__device__ __forceinline__ int q5_legacy_value(const uint8_t *qh, const uint8_t *qs, int v) {
    const uint8_t packed = qs[v & 15];
    const int nib = (v < 16) ? (packed & 0x0F) : (packed >> 4);
    return nib | (((qh[v >> 3] >> (v & 7)) & 1) << 4);
}

// Q5_0 (q5_gguf.c:242-279): y = (q - 16) * scale
__device__ __forceinline__ float dequant_value_q5_0(const uint8_t *blk, int v) {
    const BlockQ5_0 *b = (const BlockQ5_0 *)blk;
    return (float)(q5_legacy_value(b->qh, b->qs, v) - 16) * h2f(b->scale);
}

// Q5_1 (q5_gguf.c:281-318): y = q * scale + min
__device__ __forceinline__ float dequant_value_q5_1(const uint8_t *blk, int v) {
    const BlockQ5_1 *b = (const BlockQ5_1 *)blk;
    return (float)q5_legacy_value(b->qh, b->qs, v) * h2f(b->scale) + h2f(b->min);
}

// Q8_K (q8k_gguf.c): y = d * q
__device__ __forceinline__ float dequant_value_q8_k(const uint8_t *blk, int v) {
    const BlockQ8_K *b = (const BlockQ8_K *)blk;
    float d;
    __builtin_memcpy(&d, &b->d, 4);
    return d * (float)b->qs[v];
}

template <int KIND>
__device__ __forceinline__ float dequant_value(const uint8_t *blk, int v) {
    if constexpr (KIND == MARMOT_HIP_KIND_Q4_K) {
        return dequant_value_q4_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q2_K) {
        return dequant_value_q2_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q3_K) {
        return dequant_value_q3_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q5_K) {
        return dequant_value_q5_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q6_K) {
        return dequant_value_q6_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q8_0) {
        return dequant_value_q8_0(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q4_0) {
        return dequant_value_q4_0(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q8_1) {
        return dequant_value_q8_1(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q4_1) {
        return dequant_value_q4_1(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q5_0) {
        return dequant_value_q5_0(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q5_1) {
        return dequant_value_q5_1(blk, v);
    } else {
        return dequant_value_q8_k(blk, v);
    }
}

// ---- weights as the reference's fp16 direct dots see them
// cpu_vec_dot_{q2_k,q3_k,q5_k,q6_k}_f16 (vec_dot_impl.h:866-971, 1025-1128) decode their blocks with index patterns
// of their own, which differ from the dequantizers above; the reference's matmul golden for fp16 activations records
// what they compute. A backend that replaces that path has to return the same numbers, so the direct fp16 route
// mirrors the functions as written. Value v (0..255) of a block:
//   Q2_K: one scale / min pair per 128 values (scales[v / 128]), 2-bit values in sequential order (bits 2 (v % 4) of
//         qs[v / 4]);
__device__ __forceinline__ float direct_f16_weight_q2_k(const uint8_t *blk, int v) {
    const BlockQ2_K *b = (const BlockQ2_K *)blk;
    const uint8_t sc = b->scales[v >> 7];
    const float dl = h2f(b->d) * (float)(sc & 0xF);
    const float ml = h2f(b->dmin) * (float)(sc >> 4);
    const int q = (b->qs[v >> 2] >> ((v & 3) * 2)) & 3;
    return dl * (float)q - ml;
}
//   Q3_K: the high-bit mask advances once per 128 values instead of once per 32;
__device__ __forceinline__ float direct_f16_weight_q3_k(const uint8_t *blk, int v) {
    const BlockQ3_K *b = (const BlockQ3_K *)blk;
    const int c = v >> 7, j = (v >> 5) & 3, li = v & 31;  // li = l + 16 * half
    const float dl = h2f(b->d) * (float)q3k_group_scale(b->scales, v >> 4);
    const int q2 = (b->qs[32 * c + li] >> (2 * j)) & 3;
    const int q = q2 - (((b->hmask[li] >> c) & 1) ? 0 : 4);
    return dl * (float)q;
}
//   Q5_K: the fifth bit is bit 0 of byte 8 g + l (+ 32 for the high nibbles) counted from the start of qh, which for
//         most values is a byte of another element or of qs;
__device__ __forceinline__ float direct_f16_weight_q5_k(const uint8_t *blk, int v) {
    const BlockQ5_K *b = (const BlockQ5_K *)blk;
    const int j = v >> 5, l = v & 31, g = j >> 1;
    uint8_t sc, m;
    const uint8_t *s = b->scales;
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (uint8_t)((s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4));
        m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
    const float d1 = h2f(b->d) * (float)sc;
    const float m1 = h2f(b->dmin) * (float)m;
    const uint8_t byte = b->qs[32 * g + l];
    const int h = b->qh[8 * g + l + ((j & 1) ? 32 : 0)] & 1;  // runs past qh[32] into qs: still inside the block
    const int q = ((j & 1) ? (byte >> 4) : (byte & 0xF)) | (h << 4);
    return d1 * (float)q - m1;
}
//   Q6_K: one scale per 128 values (scales[v / 128]), nibbles and high pairs in sequential order.
__device__ __forceinline__ float direct_f16_weight_q6_k(const uint8_t *blk, int v) {
    const BlockQ6_K *b = (const BlockQ6_K *)blk;
    const float scale = h2f(b->d) * (float)b->scales[v >> 7];
    const int nib = (v & 1) ? (b->ql[v >> 1] >> 4) : (b->ql[v >> 1] & 0xF);
    const int hi2 = (b->qh[v >> 2] >> ((v & 3) * 2)) & 3;
    const int q = (int)(int8_t)(nib | (hi2 << 4)) - 32;
    return scale * (float)q;
}

// the weight the reference's fp16 direct dot multiplies with activation v of a block
template <int KIND>
__device__ __forceinline__ float direct_f16_weight(const uint8_t *blk, int v) {
    if constexpr (KIND == MARMOT_HIP_KIND_Q2_K) {
        return direct_f16_weight_q2_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q3_K) {
        return direct_f16_weight_q3_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q5_K) {
        return direct_f16_weight_q5_k(blk, v);
    } else if constexpr (KIND == MARMOT_HIP_KIND_Q6_K) {
        return direct_f16_weight_q6_k(blk, v);
    } else {
        return dequant_value<KIND>(blk, v);
    }
}

template <int KIND>
struct KindTraits {
    static constexpr int BV = (KIND == MARMOT_HIP_KIND_Q4_0 || KIND == MARMOT_HIP_KIND_Q8_0 ||
                               KIND == MARMOT_HIP_KIND_Q4_1 || KIND == MARMOT_HIP_KIND_Q5_0 ||
                               KIND == MARMOT_HIP_KIND_Q5_1 || KIND == MARMOT_HIP_KIND_Q8_1)
        ? QK
        : QK_K;
    static constexpr int BB = KIND == MARMOT_HIP_KIND_Q4_0 ? Q4_0_BYTES
        : KIND == MARMOT_HIP_KIND_Q4_1                     ? Q4_1_BYTES
        : KIND == MARMOT_HIP_KIND_Q5_0                     ? Q5_0_BYTES
        : KIND == MARMOT_HIP_KIND_Q5_1                     ? Q5_1_BYTES
        : KIND == MARMOT_HIP_KIND_Q8_1                     ? Q8_1_BYTES
        : KIND == MARMOT_HIP_KIND_Q8_0                     ? Q8_0_BYTES
        : KIND == MARMOT_HIP_KIND_Q2_K                     ? Q2_K_BYTES
        : KIND == MARMOT_HIP_KIND_Q3_K                     ? Q3_K_BYTES
        : KIND == MARMOT_HIP_KIND_Q4_K                     ? Q4_K_BYTES
        : KIND == MARMOT_HIP_KIND_Q5_K                     ? Q5_K_BYTES
        : KIND == MARMOT_HIP_KIND_Q6_K                     ? Q6_K_BYTES
                                                           : Q8_K_BYTES;
};

} // namespace mh

/*
 * marmot_oracle — TEST INFRASTRUCTURE ONLY (see marmot_oracle.h).
 *
 * CPU restatement of marmot's quantized-matmul arithmetic in its scalar
 * configuration. Build with -ffp-contract=off so every fp32 operation is
 * rounded separately, as in the reference's scalar build.
 */
#include "marmot_oracle.h"

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define QK 32
#define QK_K 256
#define TILE_COLS 16  /* matmul_quant_internal.h:11 */
#define BLOCK_ROWS 64 /* matmul_quant_internal.h:12 */
#define KC_BLOCKS 64  /* matmul_quant_internal.h:13 */
#define MR 8          /* matmul_quant_internal.h:15-21 */

/* error codes: include/marmot/types.h:210-220 */
#define MO_OK 0
#define MO_ERR_INVALID_ARGUMENT (-1)
#define MO_ERR_OUT_OF_MEMORY (-2)
#define MO_ERR_DIMENSION_MISMATCH (-7)
#define MO_ERR_INVALID_OPERATION (-5)
#define MO_ERR_UNSUPPORTED_DTYPE (-6)
#define MO_ERR_NOT_IMPLEMENTED (-8)

/* ---- block layouts: include/marmot/quant_block.h:20-125 ---- */
#pragma pack(push, 1)
typedef struct {
    uint16_t scale;
    uint8_t qs[16];
} blk_q4_0; /* 18 B */
typedef struct {
    uint16_t scale;
    int8_t qs[32];
} blk_q8_0; /* 34 B */
typedef struct {
    uint16_t scale;
    uint16_t min;
    uint8_t qs[16];
} blk_q4_1; /* 20 B */
typedef struct {
    uint16_t scale;
    uint8_t qh[4];
    uint8_t qs[16];
} blk_q5_0; /* 22 B */
typedef struct {
    uint16_t scale;
    uint16_t min;
    uint8_t qh[4];
    uint8_t qs[16];
} blk_q5_1; /* 24 B */
typedef struct {
    uint16_t scale;
    uint16_t sum; /* f16(sum(q) * scale): carried, not used by the dequantizer or the dots */
    int8_t qs[32];
} blk_q8_1; /* 36 B */
typedef struct {
    uint16_t d;
    uint16_t dmin;
    uint8_t scales[12];
    uint8_t qs[128];
} blk_q4_k; /* 144 B */
typedef struct {
    uint16_t d;
    uint16_t dmin;
    uint8_t scales[12];
    uint8_t qh[32];
    uint8_t qs[128];
} blk_q5_k; /* 176 B */
typedef struct {
    uint8_t scales[16]; /* scale (low nibble) and min (high nibble) of each group of 16 */
    uint8_t qs[64];
    uint16_t d;
    uint16_t dmin;
} blk_q2_k; /* 84 B */
typedef struct {
    uint8_t hmask[32];
    uint8_t qs[64];
    uint8_t scales[12];
    uint16_t d;
} blk_q3_k; /* 110 B */
typedef struct {
    uint8_t ql[128];
    uint8_t qh[64];
    int8_t scales[16];
    uint16_t d;
} blk_q6_k; /* 210 B */
typedef struct {
    float d;
    int8_t qs[256];
    int16_t bsums[16];
} blk_q8_k; /* 292 B */
#pragma pack(pop)

_Static_assert(sizeof(blk_q4_0) == 18, "Q4_0");
_Static_assert(sizeof(blk_q8_0) == 34, "Q8_0");
_Static_assert(sizeof(blk_q4_1) == 20, "Q4_1");
_Static_assert(sizeof(blk_q5_0) == 22, "Q5_0");
_Static_assert(sizeof(blk_q5_1) == 24, "Q5_1");
_Static_assert(sizeof(blk_q8_1) == 36, "Q8_1");
_Static_assert(sizeof(blk_q4_k) == 144, "Q4_K");
_Static_assert(sizeof(blk_q5_k) == 176, "Q5_K");
_Static_assert(sizeof(blk_q2_k) == 84, "Q2_K");
_Static_assert(sizeof(blk_q3_k) == 110, "Q3_K");
_Static_assert(sizeof(blk_q6_k) == 210, "Q6_K");
_Static_assert(sizeof(blk_q8_k) == 292, "Q8_K");

size_t mo_block_values(int kind) {
    switch (kind) {
    case MO_KIND_Q4_0:
    case MO_KIND_Q4_1:
    case MO_KIND_Q5_0:
    case MO_KIND_Q5_1:
    case MO_KIND_Q8_0:
    case MO_KIND_Q8_1:
        return QK;
    case MO_KIND_Q2_K:
    case MO_KIND_Q3_K:
    case MO_KIND_Q4_K:
    case MO_KIND_Q5_K:
    case MO_KIND_Q6_K:
    case MO_KIND_Q8_K:
        return QK_K;
    default:
        return 0;
    }
}

size_t mo_block_bytes(int kind) {
    switch (kind) {
    case MO_KIND_Q4_0:
        return sizeof(blk_q4_0);
    case MO_KIND_Q4_1:
        return sizeof(blk_q4_1);
    case MO_KIND_Q5_0:
        return sizeof(blk_q5_0);
    case MO_KIND_Q5_1:
        return sizeof(blk_q5_1);
    case MO_KIND_Q8_1:
        return sizeof(blk_q8_1);
    case MO_KIND_Q8_0:
        return sizeof(blk_q8_0);
    case MO_KIND_Q4_K:
        return sizeof(blk_q4_k);
    case MO_KIND_Q5_K:
        return sizeof(blk_q5_k);
    case MO_KIND_Q2_K:
        return sizeof(blk_q2_k);
    case MO_KIND_Q3_K:
        return sizeof(blk_q3_k);
    case MO_KIND_Q6_K:
        return sizeof(blk_q6_k);
    case MO_KIND_Q8_K:
        return sizeof(blk_q8_k);
    default:
        return 0;
    }
}

/* matmul_quant_dispatch.c:423-427 */
size_t mo_row_bytes(int kind, size_t k) {
    const size_t bv = mo_block_values(kind);
    if (bv == 0) {
        return 0;
    }
    return ((k + bv - 1) / bv) * mo_block_bytes(kind);
}

/* ---- fp16 ---- */
float mo_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t mo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        if (absx > 0x7f800000u) {
            return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu));
        }
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* < 2^-25 (or exactly 2^-25 tie -> even 0) */
        return sign;
    }
    int32_t exp = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7fffffu) | 0x800000u;
    uint32_t shift;
    uint32_t half_exp;
    if (exp < -14) { /* subnormal half */
        shift = (uint32_t)(13 + (-14 - exp));
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = (uint32_t)(exp + 15);
    }
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) {
        q++;
    }
    uint32_t out;
    if (half_exp == 0) {
        out = q; /* may carry into exponent 1: correct */
    } else {
        out = ((half_exp - 1) << 10) + q; /* q has the implicit bit at 0x400 */
    }
    return (uint16_t)(sign | out);
}

/* ---- small helpers ---- */

/* quantization/common/kquant_common.h:142-148 (and matmul_quant_pack.c:11-21 with clamping) */
static inline int nearest_int_magic(float value) {
    const float shifted = value + 12582912.0f;
    int bits;
    memcpy(&bits, &shifted, sizeof(int));
    return (bits & 0x007fffff) - 0x00400000;
}

static inline int nearest_int_clamped(float value) {
    if (value > 4194303.0f) {
        value = 4194303.0f;
    } else if (value < -4194303.0f) {
        value = -4194303.0f;
    }
    return nearest_int_magic(value);
}

/* quantization/common/kquant_common.h:29-37 */
static inline void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ======================= Q8_0 ======================= */

/* q8_gguf.c:127-153, quant_utils.c:55-73, block.c:221-232 (scalar: roundf, clamp +-127) */
static void q8_0_quantize_block(const float *values, uint32_t elems, blk_q8_0 *block) {
    float max_abs = 0.0f;
    for (uint32_t i = 0; i < elems; ++i) {
        const float a = fabsf(values[i]);
        if (a > max_abs) {
            max_abs = a;
        }
    }
    float scale = max_abs <= 0.0f ? 0.0f : max_abs / 127.0f;
    if (scale < FLT_MIN) {
        scale = 1.0f;
    }
    const float inv_scale = 1.0f / scale;
    memset(block, 0, sizeof(*block));
    block->scale = mo_f32_to_f16(scale);
    for (uint32_t i = 0; i < elems; ++i) {
        const float v = values[i] * inv_scale;
        int32_t q = (int32_t)roundf(v);
        if (q < -127) {
            q = -127;
        } else if (q > 127) {
            q = 127;
        }
        block->qs[i] = (int8_t)q;
    }
}

/* q8_gguf.c:189-200 */
static void q8_0_dequantize_block(const blk_q8_0 *block, uint32_t elems, float *out) {
    const float scale = mo_f16_to_f32(block->scale);
    for (uint32_t i = 0; i < elems; ++i) {
        out[i] = (float)block->qs[i] * scale;
    }
}

/* q8_gguf.c:155-187: the Q8_0 values plus f16(sum(q) * scale) with the unrounded scale */
static void q8_1_quantize_block(const float *values, uint32_t elems, blk_q8_1 *block) {
    blk_q8_0 tmp;
    q8_0_quantize_block(values, elems, &tmp);
    float max_abs = 0.0f;
    for (uint32_t i = 0; i < elems; ++i) {
        const float a = fabsf(values[i]);
        if (a > max_abs) {
            max_abs = a;
        }
    }
    float scale = max_abs <= 0.0f ? 0.0f : max_abs / 127.0f;
    if (scale < FLT_MIN) {
        scale = 1.0f;
    }
    memset(block, 0, sizeof(*block));
    block->scale = tmp.scale;
    memcpy(block->qs, tmp.qs, sizeof(tmp.qs));
    int32_t sum = 0;
    for (uint32_t i = 0; i < elems; ++i) {
        sum += block->qs[i];
    }
    block->sum = mo_f32_to_f16((float)sum * scale);
}

/* q8_gguf.c:202-213 */
static void q8_1_dequantize_block(const blk_q8_1 *block, uint32_t elems, float *out) {
    const float scale = mo_f16_to_f32(block->scale);
    for (uint32_t i = 0; i < elems; ++i) {
        out[i] = (float)block->qs[i] * scale;
    }
}

/* ======================= Q4_0 ======================= */

/* q4_gguf.c:249-312 */
static void q4_0_quantize_block(const float *values, uint32_t elems, blk_q4_0 *block) {
    float bv[QK] = {0};
    memcpy(bv, values, elems * sizeof(float));
    float amax = 0.0f;
    float max_val = 0.0f;
    for (uint32_t i = 0; i < QK; ++i) {
        const float a = fabsf(bv[i]);
        if (a > amax) {
            amax = a;
            max_val = bv[i];
        }
    }
    float scale = 0.0f;
    float inv_scale = 0.0f;
    if (amax > 0.0f) {
        scale = -max_val / 8.0f;
        if (scale != 0.0f) {
            inv_scale = 1.0f / scale;
        }
    }
    block->scale = mo_f32_to_f16(scale);
    uint8_t qv[QK];
    for (uint32_t i = 0; i < QK; ++i) {
        const float x = bv[i] * inv_scale;
        int32_t q = (int32_t)(int8_t)(x + 8.5f);
        if (q < 0) {
            q = 0;
        } else if (q > 15) {
            q = 15;
        }
        qv[i] = (uint8_t)q;
    }
    for (uint32_t j = 0; j < QK / 2; ++j) {
        block->qs[j] = (uint8_t)(((qv[j + QK / 2] & 0x0F) << 4) | (qv[j] & 0x0F));
    }
}

/* q4_gguf.c:367-394 (scalar branch) */
static void q4_0_dequantize_block(const blk_q4_0 *block, uint32_t elems, float *out) {
    const float scale = mo_f16_to_f32(block->scale);
    float decoded[QK];
    for (uint32_t j = 0; j < QK / 2; ++j) {
        const uint8_t packed = block->qs[j];
        decoded[j] = (float)((int)(packed & 0x0F) - 8) * scale;
        decoded[j + QK / 2] = (float)((int)(packed >> 4) - 8) * scale;
    }
    memcpy(out, decoded, elems * sizeof(float));
}

/* ======================= Q4_1, Q5_0, Q5_1 ======================= */

/* block.c:27-39 */
static void block_minmax(const float *data, uint32_t len, float *min_val, float *max_val) {
    float lo = data[0], hi = data[0];
    for (uint32_t i = 1; i < len; ++i) {
        const float v = data[i];
        if (v < lo) {
            lo = v;
        }
        if (v > hi) {
            hi = v;
        }
    }
    *min_val = lo;
    *max_val = hi;
}

/* q4_gguf.c:314-365 (scalar branch) */
static void q4_1_quantize_block(const float *values, uint32_t elems, blk_q4_1 *block) {
    float min_val, max_val;
    block_minmax(values, elems, &min_val, &max_val);
    float scale = (max_val - min_val) / 15.0f;
    if (scale < FLT_MIN) {
        scale = 1.0f;
    }
    const float inv_scale = (scale != 0.0f) ? 1.0f / scale : 0.0f;
    block->scale = mo_f32_to_f16(scale);
    block->min = mo_f32_to_f16(min_val);
    uint8_t qv[QK] = {0};
    for (uint32_t i = 0; i < elems; ++i) {
        const float x = (values[i] - min_val) * inv_scale;
        int32_t q = (int32_t)(int8_t)(x + 0.5f);
        if (q < 0) {
            q = 0;
        } else if (q > 15) {
            q = 15;
        }
        qv[i] = (uint8_t)q;
    }
    for (uint32_t j = 0; j < QK / 2; ++j) {
        const uint8_t q0 = j < elems ? (uint8_t)(qv[j] & 0x0F) : 0;
        const uint8_t q1 = j + QK / 2 < elems ? (uint8_t)(qv[j + QK / 2] & 0x0F) : 0;
        block->qs[j] = (uint8_t)((q1 << 4) | q0);
    }
}

/* q4_gguf.c:396-424 (scalar branch) */
static void q4_1_dequantize_block(const blk_q4_1 *block, uint32_t elems, float *out) {
    const float scale = mo_f16_to_f32(block->scale);
    const float min_val = mo_f16_to_f32(block->min);
    float decoded[QK];
    for (uint32_t j = 0; j < QK / 2; ++j) {
        const uint8_t packed = block->qs[j];
        decoded[j] = (float)(packed & 0x0F) * scale + min_val;
        decoded[j + QK / 2] = (float)(packed >> 4) * scale + min_val;
    }
    memcpy(out, decoded, elems * sizeof(float));
}

/* the five-bit values of a Q5_0 / Q5_1 block: q5_gguf.c:255-265, 294-304 */
static void q5_unpack(const uint8_t *qh_bytes, const uint8_t *qs, uint8_t *qv) {
    uint32_t qh;
    memcpy(&qh, qh_bytes, sizeof(qh));
    for (uint32_t j = 0; j < QK / 2; ++j) {
        qv[j] = (uint8_t)((qs[j] & 0x0F) | (((qh >> j) & 1u) << 4));
        qv[j + QK / 2] = (uint8_t)((qs[j] >> 4) | (((qh >> (j + QK / 2)) & 1u) << 4));
    }
}

static void q5_pack(const uint8_t *qv, uint32_t elems, uint8_t *qh_bytes, uint8_t *qs) {
    uint32_t qh = 0;
    for (uint32_t j = 0; j < QK / 2; ++j) {
        const uint8_t q0 = j < elems ? qv[j] : 0;
        const uint8_t q1 = j + QK / 2 < elems ? qv[j + QK / 2] : 0;
        qs[j] = (uint8_t)((q0 & 0x0F) | ((q1 & 0x0F) << 4));
        qh |= ((uint32_t)((q0 & 0x10u) >> 4)) << j;
        qh |= ((uint32_t)((q1 & 0x10u) >> 4)) << (j + QK / 2);
    }
    memcpy(qh_bytes, &qh, sizeof(qh));
}

/* q5_gguf.c:121-187, block.c:195-206 */
static void q5_0_quantize_block(const float *values, uint32_t elems, blk_q5_0 *block) {
    float amax = 0.0f;
    float max_val = 0.0f;
    for (uint32_t i = 0; i < elems; ++i) {
        const float a = fabsf(values[i]);
        if (a > amax) {
            amax = a;
            max_val = values[i];
        }
    }
    const float d = max_val / -16.0f;
    const float scale = (d != 0.0f) ? d : 1.0f;
    const float inv_scale = 1.0f / scale;
    memset(block, 0, sizeof(*block));
    block->scale = mo_f32_to_f16(scale);
    uint8_t qv[QK] = {0};
    for (uint32_t i = 0; i < elems; ++i) {
        const float shifted = values[i] * inv_scale + 16.5f;
        int32_t q = (int32_t)shifted;
        if (q < 0) {
            q = 0;
        } else if (q > 31) {
            q = 31;
        }
        qv[i] = (uint8_t)q; /* the reference stores q - 16 and adds 16 back with a clamp to [0, 31] */
    }
    q5_pack(qv, elems, block->qh, block->qs);
}

/* q5_gguf.c:242-279 (scalar branch) */
static void q5_0_dequantize_block(const blk_q5_0 *block, uint32_t elems, float *out) {
    const float scale = mo_f16_to_f32(block->scale);
    uint8_t qv[QK];
    q5_unpack(block->qh, block->qs, qv);
    float decoded[QK];
    for (uint32_t i = 0; i < QK; ++i) {
        decoded[i] = (float)((int32_t)qv[i] - 16) * scale;
    }
    memcpy(out, decoded, elems * sizeof(float));
}

/* q5_gguf.c:189-240, block.c:208-219 */
static void q5_1_quantize_block(const float *values, uint32_t elems, blk_q5_1 *block) {
    float min_val, max_val;
    block_minmax(values, elems, &min_val, &max_val);
    float scale = (max_val - min_val) / 31.0f;
    if (scale < FLT_MIN) {
        scale = 1.0f;
    }
    const float inv_scale = (scale != 0.0f) ? 1.0f / scale : 0.0f;
    memset(block, 0, sizeof(*block));
    block->scale = mo_f32_to_f16(scale);
    block->min = mo_f32_to_f16(min_val);
    uint8_t qv[QK] = {0};
    for (uint32_t i = 0; i < elems; ++i) {
        const float value = (values[i] - min_val) * inv_scale;
        int32_t q = (int32_t)roundf(value);
        if (q < 0) {
            q = 0;
        } else if (q > 31) {
            q = 31;
        }
        qv[i] = (uint8_t)q;
    }
    q5_pack(qv, elems, block->qh, block->qs);
}

/* q5_gguf.c:281-318 (scalar branch) */
static void q5_1_dequantize_block(const blk_q5_1 *block, uint32_t elems, float *out) {
    const float scale = mo_f16_to_f32(block->scale);
    const float min_val = mo_f16_to_f32(block->min);
    uint8_t qv[QK];
    q5_unpack(block->qh, block->qs, qv);
    float decoded[QK];
    for (uint32_t i = 0; i < QK; ++i) {
        decoded[i] = (float)qv[i] * scale + min_val;
    }
    memcpy(out, decoded, elems * sizeof(float));
}

/* ======================= Q4_K ======================= */

/* kquant_common.h:39-130 */
static float make_qkx2_quants(
    int n, int nmax, const float *x, const float *weights, uint8_t *L, float *the_min, uint8_t *Laux, float rmin,
    float rdelta, int nstep, int use_mad
) {
    float min = x[0];
    float max = x[0];
    float sum_w = weights[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < min) {
            min = x[i];
        }
        if (x[i] > max) {
            max = x[i];
        }
        const float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0) {
        min = 0;
    }
    if (max == min) {
        for (int i = 0; i < n; ++i) {
            L[i] = 0;
        }
        *the_min = -min;
        return 0.0f;
    }
    float iscale = nmax / (max - min);
    float scale = 1.0f / iscale;
    float best_error = 0;
    for (int i = 0; i < n; ++i) {
        int l = (int)nearbyintf(iscale * (x[i] - min));
        L[i] = (uint8_t)(l > nmax ? nmax : l < 0 ? 0 : l);
        float diff = scale * L[i] + min - x[i];
        diff = use_mad ? fabsf(diff) : diff * diff;
        best_error += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (max - min);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = (int)nearbyintf(iscale * (x[i] - min));
            l = l > nmax ? nmax : l < 0 ? 0 : l;
            Laux[i] = (uint8_t)l;
            const float w = weights[i];
            sum_l += w * l;
            sum_l2 += w * l * l;
            sum_xl += w * l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0;
            for (int i = 0; i < n; ++i) {
                float diff = this_scale * Laux[i] + this_min - x[i];
                diff = use_mad ? fabsf(diff) : diff * diff;
                cur_error += weights[i] * diff;
            }
            if (cur_error < best_error) {
                for (int i = 0; i < n; ++i) {
                    L[i] = Laux[i];
                }
                best_error = cur_error;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

/* q4k_gguf.c:35-131 */
static void q4_k_quantize_block(const float *values, uint32_t elems, blk_q4_k *block) {
    float bv[QK_K];
    memcpy(bv, values, elems * sizeof(float));
    if (elems < QK_K) {
        memset(bv + elems, 0, (QK_K - elems) * sizeof(float));
    }
    uint8_t L[QK_K];
    memset(L, 0, sizeof(L));
    uint8_t Laux[32];
    float weights[32];
    float scales[QK_K / 32];
    float mins[QK_K / 32];
    memset(block, 0, sizeof(*block));

    float max_scale = 0.0f;
    float max_min = 0.0f;
    for (int j = 0; j < QK_K / 32; ++j) {
        float sum_x2 = 0.0f;
        for (int l = 0; l < 32; ++l) {
            const float v = bv[32 * j + l];
            sum_x2 += v * v;
        }
        const float av_x = sqrtf(sum_x2 / 32.0f);
        for (int l = 0; l < 32; ++l) {
            weights[l] = av_x + fabsf(bv[32 * j + l]);
        }
        scales[j] = make_qkx2_quants(32, 15, bv + 32 * j, weights, L + 32 * j, &mins[j], Laux, -1.0f, 0.1f, 20, 0);
        if (scales[j] > max_scale) {
            max_scale = scales[j];
        }
        if (mins[j] > max_min) {
            max_min = mins[j];
        }
    }

    const float inv_scale = max_scale > 0 ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0 ? 63.0f / max_min : 0.0f;
    for (int j = 0; j < QK_K / 32; ++j) {
        uint8_t ls = (uint8_t)nearbyintf(inv_scale * scales[j]);
        uint8_t lm = (uint8_t)nearbyintf(inv_min * mins[j]);
        ls = ls > 63 ? 63 : ls;
        lm = lm > 63 ? 63 : lm;
        if (j < 4) {
            block->scales[j] = ls;
            block->scales[j + 4] = lm;
        } else {
            block->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            block->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
            block->scales[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    block->d = mo_f32_to_f16(max_scale / 63.0f);
    block->dmin = mo_f32_to_f16(max_min / 63.0f);

    for (int j = 0; j < QK_K / 32; ++j) {
        uint8_t sc, m;
        get_scale_min_k4(j, block->scales, &sc, &m);
        const float d = mo_f16_to_f32(block->d) * sc;
        if (d == 0) {
            continue;
        }
        const float dm = mo_f16_to_f32(block->dmin) * m;
        for (int ii = 0; ii < 32; ++ii) {
            int l = (int)nearbyintf((bv[32 * j + ii] + dm) / d);
            l = l > 15 ? 15 : (l < 0 ? 0 : l);
            L[32 * j + ii] = (uint8_t)l;
        }
    }

    for (int j = 0; j < QK_K; j += 64) {
        for (int l = 0; l < 32; ++l) {
            block->qs[(j / 2) + l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
        }
    }
    if (elems < QK_K) {
        const size_t qs_offset = (elems + 1) / 2;
        if (qs_offset < sizeof(block->qs)) {
            memset(block->qs + qs_offset, 0, sizeof(block->qs) - qs_offset);
        }
    }
}

/* q4k_gguf.c:133-166: d1 = d*sc; m1 = dmin*m; y = d1*q - m1, each op rounded */
static void q4_k_dequantize_block(const blk_q4_k *block, uint32_t elems, float *out) {
    const uint8_t *q = block->qs;
    const float d = mo_f16_to_f32(block->d);
    const float min = mo_f16_to_f32(block->dmin);
    size_t written = 0;
    int is = 0;
    for (size_t j = 0; j < QK_K && written < elems; j += 64) {
        uint8_t sc, m;
        get_scale_min_k4(is + 0, block->scales, &sc, &m);
        const float d1 = d * sc;
        const float m1 = min * m;
        get_scale_min_k4(is + 1, block->scales, &sc, &m);
        const float d2 = d * sc;
        const float m2 = min * m;
        for (int l = 0; l < 32 && written < elems; ++l, ++written) {
            out[written] = d1 * (q[l] & 0xF) - m1;
        }
        for (int l = 0; l < 32 && written < elems; ++l, ++written) {
            out[written] = d2 * (q[l] >> 4) - m2;
        }
        q += 32;
        is += 2;
    }
}

/* ======================= Q5_K ======================= */

/* q5k_gguf.c:35-160: the Q4_K search with 31 levels (rmin -0.5, 15 steps); the fifth bit of value 64g + l
 * (low nibble) is bit 2g of qh[l], of value 64g + 32 + l (high nibble) bit 2g + 1 */
static void q5_k_quantize_block(const float *values, uint32_t elems, blk_q5_k *block) {
    float bv[QK_K];
    memcpy(bv, values, elems * sizeof(float));
    if (elems < QK_K) {
        memset(bv + elems, 0, (QK_K - elems) * sizeof(float));
    }
    uint8_t L[QK_K];
    memset(L, 0, sizeof(L));
    uint8_t Laux[32];
    float weights[32];
    float scales[QK_K / 32];
    float mins[QK_K / 32];
    memset(block, 0, sizeof(*block));

    float max_scale = 0.0f;
    float max_min = 0.0f;
    for (int j = 0; j < QK_K / 32; ++j) {
        float sum_x2 = 0.0f;
        for (int l = 0; l < 32; ++l) {
            const float v = bv[32 * j + l];
            sum_x2 += v * v;
        }
        const float av_x = sqrtf(sum_x2 / 32.0f);
        for (int l = 0; l < 32; ++l) {
            weights[l] = av_x + fabsf(bv[32 * j + l]);
        }
        scales[j] = make_qkx2_quants(32, 31, bv + 32 * j, weights, L + 32 * j, &mins[j], Laux, -0.5f, 0.1f, 15, 0);
        if (scales[j] > max_scale) {
            max_scale = scales[j];
        }
        if (mins[j] > max_min) {
            max_min = mins[j];
        }
    }

    const float inv_scale = max_scale > 0 ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0 ? 63.0f / max_min : 0.0f;
    for (int j = 0; j < QK_K / 32; ++j) {
        uint8_t ls = (uint8_t)nearbyintf(inv_scale * scales[j]);
        uint8_t lm = (uint8_t)nearbyintf(inv_min * mins[j]);
        ls = ls > 63 ? 63 : ls;
        lm = lm > 63 ? 63 : lm;
        if (j < 4) {
            block->scales[j] = ls;
            block->scales[j + 4] = lm;
        } else {
            block->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            block->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
            block->scales[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    block->d = mo_f32_to_f16(max_scale / 63.0f);
    block->dmin = mo_f32_to_f16(max_min / 63.0f);

    for (int j = 0; j < QK_K / 32; ++j) {
        uint8_t sc, m;
        get_scale_min_k4(j, block->scales, &sc, &m);
        const float d = mo_f16_to_f32(block->d) * sc;
        if (d == 0) {
            continue;
        }
        const float dm = mo_f16_to_f32(block->dmin) * m;
        for (int ii = 0; ii < 32; ++ii) {
            int l = (int)nearbyintf((bv[32 * j + ii] + dm) / d);
            l = l > 31 ? 31 : (l < 0 ? 0 : l);
            L[32 * j + ii] = (uint8_t)l;
        }
    }

    uint8_t *ql = block->qs;
    for (int g = 0; g < QK_K / 64; ++g) {
        for (int j = 0; j < 32; ++j) {
            int l1 = L[64 * g + j];
            int l2 = L[64 * g + j + 32];
            if (l1 > 15) {
                l1 -= 16;
                block->qh[j] |= (uint8_t)(1u << (2 * g));
            }
            if (l2 > 15) {
                l2 -= 16;
                block->qh[j] |= (uint8_t)(2u << (2 * g));
            }
            ql[j] = (uint8_t)(l1 | (l2 << 4));
        }
        ql += 32;
    }
    if (elems < QK_K) {
        const size_t qs_offset = (elems + 1) / 2;
        const size_t qh_offset = (elems + 63) / 64;
        if (qs_offset < sizeof(block->qs)) {
            memset(block->qs + qs_offset, 0, sizeof(block->qs) - qs_offset);
        }
        if (qh_offset < sizeof(block->qh)) {
            memset(block->qh + qh_offset, 0, sizeof(block->qh) - qh_offset);
        }
    }
}

/* q5k_gguf.c:162-198: d1 = d*sc; m1 = dmin*m; y = d1*q - m1, each op rounded */
static void q5_k_dequantize_block(const blk_q5_k *block, uint32_t elems, float *out) {
    const uint8_t *ql = block->qs;
    const float d = mo_f16_to_f32(block->d);
    const float min = mo_f16_to_f32(block->dmin);
    size_t written = 0;
    for (int g = 0; g < QK_K / 64 && written < elems; ++g) {
        uint8_t sc, m;
        get_scale_min_k4(2 * g, block->scales, &sc, &m);
        const float d1 = d * sc;
        const float m1 = min * m;
        get_scale_min_k4(2 * g + 1, block->scales, &sc, &m);
        const float d2 = d * sc;
        const float m2 = min * m;
        for (int l = 0; l < 32 && written < elems; ++l, ++written) {
            const int q = (ql[l] & 0xF) | (((block->qh[l] >> (2 * g)) & 1) << 4);
            out[written] = d1 * q - m1;
        }
        for (int l = 0; l < 32 && written < elems; ++l, ++written) {
            const int q = (ql[l] >> 4) | (((block->qh[l] >> (2 * g + 1)) & 1) << 4);
            out[written] = d2 * q - m2;
        }
        ql += 32;
    }
}

/* ======================= Q2_K ======================= */

/* q2k_gguf.c:35-111: 16 groups of 16 values, 2-bit values with a 4-bit scale and a 4-bit min per group (search with
 * absolute deviations); value 128 c + 32 j + l sits in bits 2 j of qs[32 c + l] */
static void q2_k_quantize_block(const float *values, uint32_t elems, blk_q2_k *block) {
    float bv[QK_K];
    memcpy(bv, values, elems * sizeof(float));
    if (elems < QK_K) {
        memset(bv + elems, 0, (QK_K - elems) * sizeof(float));
    }
    uint8_t L[QK_K];
    memset(L, 0, sizeof(L));
    uint8_t Laux[16];
    float weights[16];
    float scales[QK_K / 16];
    float mins[QK_K / 16];
    memset(block, 0, sizeof(*block));

    float max_scale = 0.0f;
    float max_min = 0.0f;
    for (int j = 0; j < QK_K / 16; ++j) {
        for (int l = 0; l < 16; ++l) {
            weights[l] = fabsf(bv[16 * j + l]);
        }
        scales[j] = make_qkx2_quants(16, 3, bv + 16 * j, weights, L + 16 * j, &mins[j], Laux, -0.5f, 0.1f, 15, 1);
        if (scales[j] > max_scale) {
            max_scale = scales[j];
        }
        if (mins[j] > max_min) {
            max_min = mins[j];
        }
    }
    const float inv_scale = max_scale > 0 ? 15.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0 ? 15.0f / max_min : 0.0f;
    const float d = inv_scale > 0 ? 1.0f / inv_scale : 0.0f;
    const float dm = inv_min > 0 ? 1.0f / inv_min : 0.0f;
    block->d = mo_f32_to_f16(d);
    block->dmin = mo_f32_to_f16(dm);
    for (int j = 0; j < QK_K / 16; ++j) {
        uint8_t ls = (uint8_t)nearbyintf(inv_scale * scales[j]);
        uint8_t lm = (uint8_t)nearbyintf(inv_min * mins[j]);
        ls = ls > 15 ? 15 : ls;
        lm = lm > 15 ? 15 : lm;
        block->scales[j] = (uint8_t)(ls | (lm << 4));
    }
    for (int j = 0; j < QK_K / 16; ++j) {
        const uint8_t sc = block->scales[j] & 0xF;
        const uint8_t m = block->scales[j] >> 4;
        const float dl = d * sc; /* the unrounded d and dm, as the reference uses them here */
        const float ml = dm * m;
        if (dl != 0.0f) {
            for (int ii = 0; ii < 16; ++ii) {
                const int l = (int)nearbyintf((bv[16 * j + ii] + ml) / dl);
                L[16 * j + ii] = (uint8_t)(l > 3 ? 3 : (l < 0 ? 0 : l));
            }
        }
    }
    for (int j = 0; j < QK_K; j += 128) {
        for (int l = 0; l < 32; ++l) {
            block->qs[j / 4 + l] =
                (uint8_t)(L[j + l] | (L[j + l + 32] << 2) | (L[j + l + 64] << 4) | (L[j + l + 96] << 6));
        }
    }
}

/* q2k_gguf.c:113-149: y = (d * sc) * q - dmin * m */
static void q2_k_dequantize_block(const blk_q2_k *block, uint32_t elems, float *out) {
    const float d = mo_f16_to_f32(block->d);
    const float min = mo_f16_to_f32(block->dmin);
    const uint8_t *q = block->qs;
    size_t written = 0;
    int is = 0;
    for (size_t n = 0; n < QK_K && written < elems; n += 128) {
        int shift = 0;
        for (int j = 0; j < 4 && written < elems; ++j) {
            for (int half = 0; half < 2; ++half) {
                const uint8_t sc = block->scales[is++];
                const float dl = d * (sc & 0xF);
                const float ml = min * (sc >> 4);
                for (int l = 0; l < 16 && written < elems; ++l, ++written) {
                    out[written] = dl * ((int8_t)((q[l + 16 * half] >> shift) & 3)) - ml;
                }
            }
            shift += 2;
        }
        q += 32;
    }
}

/* ======================= Q3_K ======================= */

/* kquant_common.h:230-297 (do_rmse branch) */
static float make_q3_quants_rmse(int n, int nmax, const float *x, int8_t *L) {
    float max = 0;
    float amax = 0;
    for (int i = 0; i < n; ++i) {
        const float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax == 0) {
        for (int i = 0; i < n; ++i) {
            L[i] = 0;
        }
        return 0.0f;
    }
    const float iscale = -nmax / max;
    float sumlx = 0;
    float suml2 = 0;
    for (int i = 0; i < n; ++i) {
        int l = (int)nearbyintf(iscale * x[i]);
        l = l > (nmax - 1) ? (nmax - 1) : l < -nmax ? -nmax : l;
        L[i] = (int8_t)l;
        const float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    for (int itry = 0; itry < 5; ++itry) {
        int n_changed = 0;
        for (int i = 0; i < n; ++i) {
            const float w = x[i] * x[i];
            float slx = sumlx - w * x[i] * L[i];
            if (slx > 0) {
                float sl2 = suml2 - w * L[i] * L[i];
                int new_l = (int)nearbyintf(x[i] * sl2 / slx);
                new_l = new_l > (nmax - 1) ? (nmax - 1) : new_l < -nmax ? -nmax : new_l;
                if (new_l != L[i]) {
                    slx += w * x[i] * new_l;
                    sl2 += w * new_l * new_l;
                    if (sl2 > 0 && slx * slx * suml2 > sumlx * sumlx * sl2) {
                        L[i] = (int8_t)new_l;
                        sumlx = slx;
                        suml2 = sl2;
                        ++n_changed;
                    }
                }
            }
        }
        if (n_changed == 0) {
            break;
        }
    }
    for (int i = 0; i < n; ++i) {
        L[i] = (int8_t)(L[i] + nmax);
    }
    return suml2 > 0 ? sumlx / suml2 : 0.0f;
}

/* the 16 six-bit group scales of a Q3_K block (still offset by 32): q3k_gguf.c:140-149 */
static void q3_k_unpack_scales(const uint8_t *packed, int8_t *scales) {
    uint32_t aux[4];
    memcpy(aux, packed, 12);
    const uint32_t kmask1 = 0x03030303;
    const uint32_t kmask2 = 0x0f0f0f0f;
    const uint32_t tmp = aux[2];
    aux[2] = ((aux[0] >> 4) & kmask2) | (((tmp >> 4) & kmask1) << 4);
    aux[3] = ((aux[1] >> 4) & kmask2) | (((tmp >> 6) & kmask1) << 4);
    aux[0] = (aux[0] & kmask2) | (((tmp >> 0) & kmask1) << 4);
    aux[1] = (aux[1] & kmask2) | (((tmp >> 2) & kmask1) << 4);
    memcpy(scales, aux, 16);
}

/* q3k_gguf.c:35-124 */
static void q3_k_quantize_block(const float *values, uint32_t elems, blk_q3_k *block) {
    float bv[QK_K];
    memcpy(bv, values, elems * sizeof(float));
    if (elems < QK_K) {
        memset(bv + elems, 0, (QK_K - elems) * sizeof(float));
    }
    int8_t L[QK_K];
    float scales[QK_K / 16];
    memset(block, 0, sizeof(*block));
    float max_scale = 0.0f;
    float amax = 0.0f;
    for (int j = 0; j < QK_K / 16; ++j) {
        scales[j] = make_q3_quants_rmse(16, 4, bv + 16 * j, L + 16 * j);
        const float scale = fabsf(scales[j]);
        if (scale > amax) {
            amax = scale;
            max_scale = scales[j];
        }
    }
    if (max_scale != 0.0f) {
        const float iscale = -32.0f / max_scale;
        for (int j = 0; j < QK_K / 16; ++j) {
            int l = (int)nearbyintf(iscale * scales[j]);
            l = l > 31 ? 31 : (l < -32 ? -32 : l);
            int shifted = l + 32;
            if (j < 8) {
                block->scales[j] = (uint8_t)(shifted & 0xF);
            } else {
                block->scales[j - 8] |= (uint8_t)((shifted & 0xF) << 4);
            }
            shifted >>= 4;
            block->scales[j % 4 + 8] |= (uint8_t)(shifted << (2 * (j / 4)));
        }
        block->d = mo_f32_to_f16(1.0f / iscale);
    } else {
        block->d = mo_f32_to_f16(0.0f);
    }
    for (int j = 0; j < QK_K / 16; ++j) {
        int sc = j < 8 ? (block->scales[j] & 0xF) : (block->scales[j - 8] >> 4);
        sc = (sc | (((block->scales[8 + j % 4] >> (2 * (j / 4))) & 3) << 4)) - 32;
        const float d = mo_f16_to_f32(block->d) * sc;
        if (d == 0) {
            continue;
        }
        for (int ii = 0; ii < 16; ++ii) {
            int l = (int)nearbyintf(bv[16 * j + ii] / d);
            l = l > 3 ? 3 : (l < -4 ? -4 : l);
            L[16 * j + ii] = (int8_t)(l + 4);
        }
    }
    int m = 0;
    uint8_t hm = 1;
    for (int j = 0; j < QK_K; ++j) {
        if (L[j] > 3) {
            block->hmask[m] |= hm;
            L[j] = (int8_t)(L[j] - 4);
        }
        if (++m == QK_K / 8) {
            m = 0;
            hm = (uint8_t)(hm << 1);
        }
    }
    for (int j = 0; j < QK_K; j += 128) {
        for (int l = 0; l < 32; ++l) {
            block->qs[j / 4 + l] =
                (uint8_t)(L[j + l] | (L[j + l + 32] << 2) | (L[j + l + 64] << 4) | (L[j + l + 96] << 6));
        }
    }
    if (elems < QK_K) {
        const size_t qs_offset = (elems + 3) / 4;
        const size_t hmask_offset = (elems + 7) / 8;
        if (qs_offset < sizeof(block->qs)) {
            memset(block->qs + qs_offset, 0, sizeof(block->qs) - qs_offset);
        }
        if (hmask_offset < sizeof(block->hmask)) {
            memset(block->hmask + hmask_offset, 0, sizeof(block->hmask) - hmask_offset);
        }
    }
}

/* q3k_gguf.c:126-175: y = (d * (sc - 32)) * (q2 - (high bit ? 0 : 4)); the high bit of value 32 t + l is bit t of
 * hmask[l] */
static void q3_k_dequantize_block(const blk_q3_k *block, uint32_t elems, float *out) {
    const float d_all = mo_f16_to_f32(block->d);
    const uint8_t *q = block->qs;
    const uint8_t *hm = block->hmask;
    int8_t scales[16];
    q3_k_unpack_scales(block->scales, scales);
    size_t written = 0;
    int is = 0;
    uint8_t m = 1;
    for (size_t n = 0; n < QK_K && written < elems; n += 128) {
        int shift = 0;
        for (int j = 0; j < 4 && written < elems; ++j) {
            for (int half = 0; half < 2; ++half) {
                const float dl = d_all * (scales[is++] - 32);
                for (int l = 0; l < 16 && written < elems; ++l, ++written) {
                    const int li = l + 16 * half;
                    out[written] = dl * ((int8_t)((q[li] >> shift) & 3) - ((hm[li] & m) ? 0 : 4));
                }
            }
            shift += 2;
            m = (uint8_t)(m << 1);
        }
        q += 32;
    }
}

/* ======================= Q6_K ======================= */

static inline int clamp_qx(int value, int nmax) {
    if (value > nmax - 1) {
        return nmax - 1;
    }
    if (value < -nmax) {
        return -nmax;
    }
    return value;
}

/* kquant_common.h:150-236 with rmse_type == 1, weights == NULL */
static float make_qx_quants_rmse1(int n, int nmax, const float *x, int8_t *L) {
    float max = 0.0f;
    float amax = 0.0f;
    for (int i = 0; i < n; ++i) {
        const float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax < 1e-15f) {
        memset(L, 0, (size_t)n);
        return 0.0f;
    }
    const float iscale = -((float)nmax) / max;
    float sumlx = 0.0f;
    float suml2 = 0.0f;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int_magic(iscale * x[i]);
        l = clamp_qx(l, nmax);
        L[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = (suml2 > 0.0f) ? (sumlx / suml2) : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) {
            continue;
        }
        const float trial_iscale = -(nmax + 0.1f * (float)is) / max;
        float trial_sumlx = 0.0f;
        float trial_suml2 = 0.0f;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int_magic(trial_iscale * x[i]);
            l = clamp_qx(l, nmax);
            const float w = x[i] * x[i];
            trial_sumlx += w * x[i] * l;
            trial_suml2 += w * l * l;
        }
        if (trial_suml2 > 0.0f && trial_sumlx * trial_sumlx > best * trial_suml2) {
            for (int i = 0; i < n; ++i) {
                int l = nearest_int_magic(trial_iscale * x[i]);
                l = clamp_qx(l, nmax);
                L[i] = (int8_t)(l + nmax);
            }
            scale = trial_sumlx / trial_suml2;
            best = scale * trial_sumlx;
        }
    }
    return scale;
}

/* q6k_gguf.c:35-61 + kquant_common.h:310-369 */
static void q6_k_quantize_block(const float *values, uint32_t elems, blk_q6_k *y) {
    float x[QK_K];
    memcpy(x, values, elems * sizeof(float));
    if (elems < QK_K) {
        memset(x + elems, 0, (QK_K - elems) * sizeof(float));
    }
    memset(y, 0, sizeof(*y));

    int8_t L[QK_K];
    float scales[QK_K / 16];
    float max_scale = 0.0f;
    float max_abs_scale = 0.0f;
    for (int ib = 0; ib < QK_K / 16; ++ib) {
        const float scale = make_qx_quants_rmse1(16, 32, x + 16 * ib, L + 16 * ib);
        scales[ib] = scale;
        const float abs_scale = fabsf(scale);
        if (abs_scale > max_abs_scale) {
            max_abs_scale = abs_scale;
            max_scale = scale;
        }
    }
    if (max_abs_scale < 1e-15f) {
        memset(y, 0, sizeof(*y));
        return;
    }
    const float iscale = -128.0f / max_scale;
    y->d = mo_f32_to_f16(1.0f / iscale);
    for (int ib = 0; ib < QK_K / 16; ++ib) {
        int sc = nearest_int_magic(iscale * scales[ib]);
        sc = sc > 127 ? 127 : (sc < -128 ? -128 : sc);
        y->scales[ib] = (int8_t)sc;
    }
    for (int j = 0; j < QK_K / 16; ++j) {
        const float d = mo_f16_to_f32(y->d) * y->scales[j];
        if (d == 0.0f) {
            continue;
        }
        for (int ii = 0; ii < 16; ++ii) {
            int l = nearest_int_magic(x[16 * j + ii] / d);
            l = clamp_qx(l, 32);
            L[16 * j + ii] = (int8_t)(l + 32);
        }
    }
    uint8_t *ql = y->ql;
    uint8_t *qh = y->qh;
    for (int j = 0; j < QK_K; j += 128) {
        for (int l = 0; l < 32; ++l) {
            const uint8_t q1 = L[j + l + 0] & 0xF;
            const uint8_t q2 = L[j + l + 32] & 0xF;
            const uint8_t q3 = L[j + l + 64] & 0xF;
            const uint8_t q4 = L[j + l + 96] & 0xF;
            ql[l + 0] = (uint8_t)(q1 | (q3 << 4));
            ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
            qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) | ((L[j + l + 64] >> 4) << 4) |
                              ((L[j + l + 96] >> 4) << 6));
        }
        ql += 64;
        qh += 32;
    }
    if (elems < QK_K) {
        const size_t ql_offset = (elems + 1) / 2;
        const size_t qh_offset = (elems + 3) / 4;
        if (ql_offset < sizeof(y->ql)) {
            memset(y->ql + ql_offset, 0, sizeof(y->ql) - ql_offset);
        }
        if (qh_offset < sizeof(y->qh)) {
            memset(y->qh + qh_offset, 0, sizeof(y->qh) - qh_offset);
        }
    }
}

/* q6k_gguf.c:63-99: y = (d * sc) * q, left to right */
static void q6_k_dequantize_block(const blk_q6_k *block, uint32_t elems, float *out) {
    const float d = mo_f16_to_f32(block->d);
    const uint8_t *ql = block->ql;
    const uint8_t *qh = block->qh;
    const int8_t *sc = block->scales;
    for (size_t n = 0; n < QK_K && n < elems; n += 128) {
        for (int l = 0; l < 32; ++l) {
            const int is = l / 16;
            const int8_t q1 = (int8_t)((int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32);
            const int8_t q2 = (int8_t)((int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            const int8_t q3 = (int8_t)((int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            const int8_t q4 = (int8_t)((int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            if (n + l + 0 < elems) {
                out[n + l + 0] = d * sc[is + 0] * q1;
            }
            if (n + l + 32 < elems) {
                out[n + l + 32] = d * sc[is + 2] * q2;
            }
            if (n + l + 64 < elems) {
                out[n + l + 64] = d * sc[is + 4] * q3;
            }
            if (n + l + 96 < elems) {
                out[n + l + 96] = d * sc[is + 6] * q4;
            }
        }
        ql += 64;
        qh += 32;
        sc += 8;
    }
}

/* ======================= Q8_K (activation) ======================= */

/* matmul_quant_pack.c:106-142 */
static void q8_k_pack_block(const float *bv, blk_q8_k *dst) {
    float max_val = 0.0f;
    float abs_max = 0.0f;
    for (size_t i = 0; i < QK_K; ++i) {
        const float ax = fabsf(bv[i]);
        if (ax > abs_max) {
            abs_max = ax;
            max_val = bv[i];
        }
    }
    if (abs_max <= 0.0f) {
        dst->d = 0.0f;
        memset(dst->qs, 0, sizeof(dst->qs));
        memset(dst->bsums, 0, sizeof(dst->bsums));
        return;
    }
    const float iscale = -127.0f / max_val;
    for (size_t i = 0; i < QK_K; ++i) {
        int v = nearest_int_clamped(iscale * bv[i]);
        if (v > 127) {
            v = 127;
        }
        dst->qs[i] = (int8_t)v;
    }
    for (size_t b = 0; b < QK_K / 16; ++b) {
        int sum = 0;
        for (size_t i = 0; i < 16; ++i) {
            sum += dst->qs[b * 16 + i];
        }
        dst->bsums[b] = (int16_t)sum;
    }
    dst->d = 1.0f / iscale;
}

static inline float load_act(const void *x, int in_dtype, size_t i) {
    if (in_dtype == MO_DTYPE_F16) {
        return mo_f16_to_f32(((const uint16_t *)x)[i]);
    }
    return ((const float *)x)[i];
}

/* matmul_quant_pack.c:144-196 */
void mo_pack_q8_k(const void *x, int in_dtype, size_t k, void *blocks_out) {
    blk_q8_k *blocks = (blk_q8_k *)blocks_out;
    const size_t nb = (k + QK_K - 1) / QK_K;
    float bv[QK_K];
    for (size_t b = 0; b < nb; ++b) {
        const size_t start = b * QK_K;
        const size_t len = (start + QK_K <= k) ? QK_K : (k - start);
        for (size_t i = 0; i < len; ++i) {
            bv[i] = load_act(x, in_dtype, start + i);
        }
        if (len < QK_K) {
            memset(bv + len, 0, (QK_K - len) * sizeof(float));
        }
        q8_k_pack_block(bv, &blocks[b]);
    }
}

/* matmul_quant_pack.c:23-104 */
void mo_pack_q8_0(const void *x, int in_dtype, size_t k, void *blocks_out) {
    blk_q8_0 *blocks = (blk_q8_0 *)blocks_out;
    const size_t nb = (k + QK - 1) / QK;
    float bv[QK];
    for (size_t b = 0; b < nb; ++b) {
        const size_t start = b * QK;
        const size_t len = (start + QK <= k) ? QK : (k - start);
        for (size_t i = 0; i < len; ++i) {
            bv[i] = load_act(x, in_dtype, start + i);
        }
        if (len < QK) {
            memset(bv + len, 0, (QK - len) * sizeof(float));
        }
        float max_abs = 0.0f;
        for (size_t i = 0; i < len; ++i) {
            const float a = fabsf(bv[i]);
            if (a > max_abs) {
                max_abs = a;
            }
        }
        float scale = max_abs / 127.0f;
        if (scale < FLT_MIN) {
            scale = 1.0f;
        }
        const float inv_scale = 1.0f / scale;
        blk_q8_0 *dst = &blocks[b];
        memset(dst, 0, sizeof(*dst));
        dst->scale = mo_f32_to_f16(scale);
        for (size_t i = 0; i < len; ++i) {
            const float v = bv[i] * inv_scale;
            int32_t q = (int32_t)roundf(v);
            if (q < -127) {
                q = -127;
            } else if (q > 127) {
                q = 127;
            }
            dst->qs[i] = (int8_t)q;
        }
    }
}

/* ======================= blockwise drivers ======================= */

/* ops/quantize_core.c:199-265 */
int mo_quantize_rows(int kind, const float *x, size_t rows, size_t k, void *out) {
    const size_t bv = mo_block_values(kind);
    const size_t bb = mo_block_bytes(kind);
    if (bv == 0 || x == NULL || out == NULL) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    const size_t nb = (k + bv - 1) / bv;
    uint8_t *dst = (uint8_t *)out;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t b = 0; b < nb; ++b) {
            const size_t start = b * bv;
            const uint32_t elems = (uint32_t)((start + bv <= k) ? bv : (k - start));
            const float *src = x + r * k + start;
            void *blk = dst + (r * nb + b) * bb;
            switch (kind) {
            case MO_KIND_Q8_0:
                q8_0_quantize_block(src, elems, (blk_q8_0 *)blk);
                break;
            case MO_KIND_Q4_0:
                q4_0_quantize_block(src, elems, (blk_q4_0 *)blk);
                break;
            case MO_KIND_Q8_1:
                q8_1_quantize_block(src, elems, (blk_q8_1 *)blk);
                break;
            case MO_KIND_Q4_1:
                q4_1_quantize_block(src, elems, (blk_q4_1 *)blk);
                break;
            case MO_KIND_Q5_0:
                q5_0_quantize_block(src, elems, (blk_q5_0 *)blk);
                break;
            case MO_KIND_Q5_1:
                q5_1_quantize_block(src, elems, (blk_q5_1 *)blk);
                break;
            case MO_KIND_Q4_K:
                q4_k_quantize_block(src, elems, (blk_q4_k *)blk);
                break;
            case MO_KIND_Q5_K:
                q5_k_quantize_block(src, elems, (blk_q5_k *)blk);
                break;
            case MO_KIND_Q2_K:
                q2_k_quantize_block(src, elems, (blk_q2_k *)blk);
                break;
            case MO_KIND_Q3_K:
                q3_k_quantize_block(src, elems, (blk_q3_k *)blk);
                break;
            case MO_KIND_Q6_K:
                q6_k_quantize_block(src, elems, (blk_q6_k *)blk);
                break;
            case MO_KIND_Q8_K: {
                float tmp[QK_K];
                memcpy(tmp, src, elems * sizeof(float));
                if (elems < QK_K) {
                    memset(tmp + elems, 0, (QK_K - elems) * sizeof(float));
                }
                q8_k_pack_block(tmp, (blk_q8_k *)blk);
                break;
            }
            default:
                return MO_ERR_NOT_IMPLEMENTED;
            }
        }
    }
    return MO_OK;
}

/* ops/quantize_core.c:267-331 */
int mo_dequantize_rows(int kind, const void *blocks, size_t rows, size_t k, float *out) {
    const size_t bv = mo_block_values(kind);
    const size_t bb = mo_block_bytes(kind);
    if (bv == 0 || blocks == NULL || out == NULL) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    const size_t nb = (k + bv - 1) / bv;
    const uint8_t *src = (const uint8_t *)blocks;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t b = 0; b < nb; ++b) {
            const size_t start = b * bv;
            const uint32_t elems = (uint32_t)((start + bv <= k) ? bv : (k - start));
            const void *blk = src + (r * nb + b) * bb;
            float *dst = out + r * k + start;
            switch (kind) {
            case MO_KIND_Q8_0:
                q8_0_dequantize_block((const blk_q8_0 *)blk, elems, dst);
                break;
            case MO_KIND_Q4_0:
                q4_0_dequantize_block((const blk_q4_0 *)blk, elems, dst);
                break;
            case MO_KIND_Q8_1:
                q8_1_dequantize_block((const blk_q8_1 *)blk, elems, dst);
                break;
            case MO_KIND_Q4_1:
                q4_1_dequantize_block((const blk_q4_1 *)blk, elems, dst);
                break;
            case MO_KIND_Q5_0:
                q5_0_dequantize_block((const blk_q5_0 *)blk, elems, dst);
                break;
            case MO_KIND_Q5_1:
                q5_1_dequantize_block((const blk_q5_1 *)blk, elems, dst);
                break;
            case MO_KIND_Q4_K:
                q4_k_dequantize_block((const blk_q4_k *)blk, elems, dst);
                break;
            case MO_KIND_Q5_K:
                q5_k_dequantize_block((const blk_q5_k *)blk, elems, dst);
                break;
            case MO_KIND_Q2_K:
                q2_k_dequantize_block((const blk_q2_k *)blk, elems, dst);
                break;
            case MO_KIND_Q3_K:
                q3_k_dequantize_block((const blk_q3_k *)blk, elems, dst);
                break;
            case MO_KIND_Q6_K:
                q6_k_dequantize_block((const blk_q6_k *)blk, elems, dst);
                break;
            case MO_KIND_Q8_K: {
                /* q8k_gguf.c dequant: y = d * q */
                const blk_q8_k *q = (const blk_q8_k *)blk;
                for (uint32_t i = 0; i < elems; ++i) {
                    dst[i] = q->d * (float)q->qs[i];
                }
                break;
            }
            default:
                return MO_ERR_NOT_IMPLEMENTED;
            }
        }
    }
    return MO_OK;
}

/* ======================= block dots ======================= */

/* vec_dot_impl.h:452-479 */
float mo_vec_dot_q8_0_q8_0(const void *w, const void *a, size_t nblocks) {
    const blk_q8_0 *wb = (const blk_q8_0 *)w;
    const blk_q8_0 *ab = (const blk_q8_0 *)a;
    float total = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        int32_t sum = 0;
        for (int i = 0; i < QK; ++i) {
            sum += (int32_t)wb[b].qs[i] * (int32_t)ab[b].qs[i];
        }
        const float block_scale = mo_f16_to_f32(wb[b].scale) * mo_f16_to_f32(ab[b].scale);
        total += (float)sum * block_scale;
    }
    return total;
}

/* vec_dot_impl.h:481-510 */
float mo_vec_dot_q8_1_q8_0(const void *w, const void *a, size_t nblocks) {
    const blk_q8_1 *wb = (const blk_q8_1 *)w;
    const blk_q8_0 *ab = (const blk_q8_0 *)a;
    float total = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        int32_t sum = 0;
        for (int i = 0; i < QK; ++i) {
            sum += (int32_t)wb[b].qs[i] * (int32_t)ab[b].qs[i];
        }
        const float block_scale = mo_f16_to_f32(wb[b].scale) * mo_f16_to_f32(ab[b].scale);
        total += (float)sum * block_scale;
    }
    return total;
}

/* vec_dot_impl.h:157-186 */
float mo_vec_dot_q4_0_q8_0(const void *w, const void *a, size_t nblocks) {
    const blk_q4_0 *wb = (const blk_q4_0 *)w;
    const blk_q8_0 *ab = (const blk_q8_0 *)a;
    float total = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        int32_t sum = 0;
        for (int i = 0; i < QK / 2; ++i) {
            const uint8_t packed = wb[b].qs[i];
            sum += ((int32_t)(packed & 0x0f) - 8) * (int32_t)ab[b].qs[i];
            sum += ((int32_t)(packed >> 4) - 8) * (int32_t)ab[b].qs[i + QK / 2];
        }
        const float block_scale = mo_f16_to_f32(wb[b].scale) * mo_f16_to_f32(ab[b].scale);
        total += (float)sum * block_scale;
    }
    return total;
}

/* The 32-value formats with an offset or a fifth bit against Q8_0 activations: integer dot of the unsigned (Q4_1,
 * Q5_1) or recentred (Q5_0) weight values, times the two scales; the *_1 formats add min * scale_a * sum(a)
 * (vec_dot_impl.h:186-217, 288-349). */
static float legacy_dot(int kind, const void *w, const void *a, size_t nblocks) {
    const blk_q8_0 *ab = (const blk_q8_0 *)a;
    float total = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        uint8_t qv[QK];
        float scale_w, min_w = 0.0f;
        int centre = 0;
        if (kind == MO_KIND_Q4_1) {
            const blk_q4_1 *wb = (const blk_q4_1 *)w + b;
            for (int i = 0; i < QK / 2; ++i) {
                qv[i] = wb->qs[i] & 0x0f;
                qv[i + QK / 2] = wb->qs[i] >> 4;
            }
            scale_w = mo_f16_to_f32(wb->scale);
            min_w = mo_f16_to_f32(wb->min);
        } else if (kind == MO_KIND_Q5_0) {
            const blk_q5_0 *wb = (const blk_q5_0 *)w + b;
            q5_unpack(wb->qh, wb->qs, qv);
            scale_w = mo_f16_to_f32(wb->scale);
            centre = 16;
        } else {
            const blk_q5_1 *wb = (const blk_q5_1 *)w + b;
            q5_unpack(wb->qh, wb->qs, qv);
            scale_w = mo_f16_to_f32(wb->scale);
            min_w = mo_f16_to_f32(wb->min);
        }
        const float scale_a = mo_f16_to_f32(ab[b].scale);
        int32_t sum_q = 0, sum_a = 0;
        for (int i = 0; i < QK; ++i) {
            sum_q += ((int32_t)qv[i] - centre) * (int32_t)ab[b].qs[i];
            sum_a += (int32_t)ab[b].qs[i];
        }
        const float block_scale = scale_w * scale_a;
        if (kind == MO_KIND_Q5_0) {
            total += (float)sum_q * block_scale;
        } else {
            const float bias_scale = min_w * scale_a;
            total += block_scale * (float)sum_q + bias_scale * (float)sum_a;
        }
    }
    return total;
}

float mo_vec_dot_q4_1_q8_0(const void *w, const void *a, size_t nblocks) {
    return legacy_dot(MO_KIND_Q4_1, w, a, nblocks);
}

float mo_vec_dot_q5_0_q8_0(const void *w, const void *a, size_t nblocks) {
    return legacy_dot(MO_KIND_Q5_0, w, a, nblocks);
}

float mo_vec_dot_q5_1_q8_0(const void *w, const void *a, size_t nblocks) {
    return legacy_dot(MO_KIND_Q5_1, w, a, nblocks);
}

/* vec_dot_impl.h:541-563, 689-732 */
float mo_vec_dot_q4_k_q8_k(const void *w, const void *a, size_t nblocks) {
    const blk_q4_k *wb = (const blk_q4_k *)w;
    const blk_q8_k *ab = (const blk_q8_k *)a;
    float sum_all = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        uint8_t scales[8];
        uint8_t mins[8];
        for (int j = 0; j < 8; ++j) {
            get_scale_min_k4(j, wb[b].scales, &scales[j], &mins[j]);
        }
        int32_t sumi = 0;
        for (int j = 0; j < QK_K / 16; ++j) {
            sumi += (int32_t)ab[b].bsums[j] * (int32_t)mins[j / 2];
        }
        int32_t block_sum = 0;
        for (int sg = 0; sg < 8; ++sg) {
            const uint8_t *q4 = wb[b].qs + (sg / 2) * 32;
            const int8_t *q8 = ab[b].qs + sg * 32;
            const int high = sg & 1;
            int32_t dot = 0;
            for (int l = 0; l < 32; ++l) {
                const int32_t wv = high ? (q4[l] >> 4) : (q4[l] & 0x0F);
                dot += wv * (int32_t)q8[l];
            }
            block_sum += (int32_t)scales[sg] * dot;
        }
        const float d = ab[b].d * mo_f16_to_f32(wb[b].d);
        const float dmin = ab[b].d * mo_f16_to_f32(wb[b].dmin);
        sum_all += d * (float)block_sum - dmin * (float)sumi;
    }
    return sum_all;
}

/* vec_dot_impl.h:565-618 */
float mo_vec_dot_q2_k_q8_k(const void *w, const void *a, size_t nblocks) {
    const blk_q2_k *wb = (const blk_q2_k *)w;
    const blk_q8_k *ab = (const blk_q8_k *)a;
    float sum_all = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        const uint8_t *q2 = wb[b].qs;
        const uint8_t *sc = wb[b].scales;
        const int8_t *q8 = ab[b].qs;
        int32_t summs = 0;
        for (int j = 0; j < 16; ++j) {
            summs += (int32_t)ab[b].bsums[j] * (int32_t)(sc[j] >> 4);
        }
        const float dall = ab[b].d * mo_f16_to_f32(wb[b].d);
        const float dmin = ab[b].d * mo_f16_to_f32(wb[b].dmin);
        int32_t isum = 0;
        int is = 0;
        for (int chunk = 0; chunk < QK_K / 128; ++chunk) {
            int shift = 0;
            for (int j = 0; j < 4; ++j) {
                for (int half = 0; half < 2; ++half) {
                    const int32_t dsc = sc[is++] & 0xF;
                    int32_t dot = 0;
                    for (int l = 0; l < 16; ++l) {
                        dot += (int32_t)q8[l + 16 * half] * (int32_t)((q2[l + 16 * half] >> shift) & 3);
                    }
                    isum += dsc * dot;
                }
                shift += 2;
                q8 += 32;
            }
            q2 += 32;
        }
        sum_all += dall * (float)isum - dmin * (float)summs;
    }
    return sum_all;
}

/* vec_dot_impl.h:620-687 */
float mo_vec_dot_q3_k_q8_k(const void *w, const void *a, size_t nblocks) {
    const blk_q3_k *wb = (const blk_q3_k *)w;
    const blk_q8_k *ab = (const blk_q8_k *)a;
    float sum_all = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        const uint8_t *q3 = wb[b].qs;
        const uint8_t *hm = wb[b].hmask;
        const int8_t *q8 = ab[b].qs;
        int8_t scales[16];
        q3_k_unpack_scales(wb[b].scales, scales);
        int32_t block_sum = 0;
        uint8_t m = 1;
        int scale_index = 0;
        for (int chunk = 0; chunk < QK_K / 128; ++chunk) {
            int shift = 0;
            for (int j = 0; j < 4; ++j) {
                for (int half = 0; half < 2; ++half) {
                    int32_t dot = 0;
                    for (int l = 0; l < 16; ++l) {
                        const int li = l + 16 * half;
                        int8_t val = (int8_t)((q3[li] >> shift) & 3);
                        if ((hm[li] & m) == 0) {
                            val = (int8_t)(val - 4);
                        }
                        dot += (int32_t)val * (int32_t)q8[li];
                    }
                    block_sum += (int32_t)(scales[scale_index] - 32) * dot;
                    scale_index++;
                }
                q8 += 32;
                shift += 2;
                m = (uint8_t)(m << 1);
            }
            q3 += 32;
        }
        const float d = ab[b].d * mo_f16_to_f32(wb[b].d);
        sum_all += d * (float)block_sum;
    }
    return sum_all;
}

/* vec_dot_impl.h:734-781 */
float mo_vec_dot_q5_k_q8_k(const void *w, const void *a, size_t nblocks) {
    const blk_q5_k *wb = (const blk_q5_k *)w;
    const blk_q8_k *ab = (const blk_q8_k *)a;
    float sum_all = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        uint8_t scales[8];
        uint8_t mins[8];
        for (int j = 0; j < 8; ++j) {
            get_scale_min_k4(j, wb[b].scales, &scales[j], &mins[j]);
        }
        int32_t sumi = 0;
        for (int j = 0; j < QK_K / 16; ++j) {
            sumi += (int32_t)ab[b].bsums[j] * (int32_t)mins[j / 2];
        }
        int32_t block_sum = 0;
        for (int sg = 0; sg < 8; ++sg) {
            const uint8_t *q4 = wb[b].qs + (sg / 2) * 32;
            const int8_t *q8 = ab[b].qs + sg * 32;
            const int high = sg & 1;
            int32_t dot = 0;
            for (int l = 0; l < 32; ++l) {
                const int32_t hi = ((wb[b].qh[l] >> sg) & 1) ? 16 : 0;
                const int32_t wv = (high ? (q4[l] >> 4) : (q4[l] & 0x0F)) + hi;
                dot += wv * (int32_t)q8[l];
            }
            block_sum += (int32_t)scales[sg] * dot;
        }
        const float d = ab[b].d * mo_f16_to_f32(wb[b].d);
        const float dmin = ab[b].d * mo_f16_to_f32(wb[b].dmin);
        sum_all += d * (float)block_sum - dmin * (float)sumi;
    }
    return sum_all;
}

/* vec_dot_impl.h:783-828 */
float mo_vec_dot_q6_k_q8_k(const void *w, const void *a, size_t nblocks) {
    const blk_q6_k *wb = (const blk_q6_k *)w;
    const blk_q8_k *ab = (const blk_q8_k *)a;
    float sum_all = 0.0f;
    for (size_t b = 0; b < nblocks; ++b) {
        const int8_t *q8 = ab[b].qs;
        int32_t block_sum = 0;
        for (size_t sg = 0; sg < QK_K / 16; ++sg) {
            const size_t group32 = sg / 2;
            const size_t half = group32 / 4;
            const size_t gih = group32 & 3;
            const size_t part = sg & 1;
            const uint8_t *ql = wb[b].ql + half * 64 + ((gih & 1) ? 32 : 0) + part * 16;
            const uint8_t *qh = wb[b].qh + half * 32 + part * 16;
            const int shift = (int)(gih * 2);
            const int high_nibble = gih >= 2;
            int32_t dot = 0;
            for (int l = 0; l < 16; ++l) {
                const uint8_t ql_val = high_nibble ? (ql[l] >> 4) : (ql[l] & 0x0F);
                const uint8_t qh_val = (qh[l] >> shift) & 0x03;
                const int8_t q = (int8_t)((ql_val | (qh_val << 4)) - 32);
                dot += (int32_t)q * (int32_t)q8[l];
            }
            block_sum += (int32_t)wb[b].scales[sg] * dot;
            q8 += 16;
        }
        const float d = ab[b].d * mo_f16_to_f32(wb[b].d);
        sum_all += d * (float)block_sum;
    }
    return sum_all;
}

/* fp16 direct dots: vec_dot_impl.h:220-250 (Q4_0), 419-450 (Q8_0), 973-1023 (Q4_K).
 * Q6_K: the reference's cpu_vec_dot_q6_k_f16 (vec_dot_impl.h:1082-1128) decodes with an index
 * pattern that differs from its own dequantizer; the oracle restates that function as written,
 * so parity with "what the reference computes" holds, but no product kernel mirrors it. */
float mo_vec_dot_f16(int kind, const void *w, const uint16_t *a, size_t nblocks, size_t k) {
    float total = 0.0f;
    if (kind == MO_KIND_Q8_0) {
        const blk_q8_0 *wb = (const blk_q8_0 *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            const float scale_w = mo_f16_to_f32(wb[b].scale);
            const size_t start = b * QK;
            const size_t len = (start + QK <= k) ? QK : (k - start);
            for (size_t i = 0; i < len; ++i) {
                const float av = mo_f16_to_f32(a[start + i]);
                total += ((float)wb[b].qs[i]) * scale_w * av;
            }
        }
    } else if (kind == MO_KIND_Q8_1) { /* vec_dot_impl.h:512-539 */
        const blk_q8_1 *wb = (const blk_q8_1 *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            const float scale_w = mo_f16_to_f32(wb[b].scale);
            const size_t start = b * QK;
            const size_t len = (start + QK <= k) ? QK : (k - start);
            for (size_t i = 0; i < len; ++i) {
                const float av = mo_f16_to_f32(a[start + i]);
                total += ((float)wb[b].qs[i]) * scale_w * av;
            }
        }
    } else if (kind == MO_KIND_Q4_0) {
        const blk_q4_0 *wb = (const blk_q4_0 *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            int16_t w16[QK];
            for (int i = 0; i < QK / 2; ++i) {
                w16[i] = (int16_t)((wb[b].qs[i] & 0x0f) - 8);
                w16[i + QK / 2] = (int16_t)((wb[b].qs[i] >> 4) - 8);
            }
            const float scale_w = mo_f16_to_f32(wb[b].scale);
            const size_t start = b * QK;
            const size_t len = (start + QK <= k) ? QK : (k - start);
            for (size_t i = 0; i < len; ++i) {
                const float av = mo_f16_to_f32(a[start + i]);
                total += ((float)w16[i]) * scale_w * av;
            }
        }
    } else if (kind == MO_KIND_Q4_1 || kind == MO_KIND_Q5_0 || kind == MO_KIND_Q5_1) {
        /* vec_dot_impl.h:253-286, 351-416: ((q - 16) * scale) * a for Q5_0, (scale * q + min) * a for the *_1 formats */
        for (size_t b = 0; b < nblocks; ++b) {
            uint8_t qv[QK];
            float scale_w, min_w = 0.0f;
            if (kind == MO_KIND_Q4_1) {
                const blk_q4_1 *wb = (const blk_q4_1 *)w + b;
                for (int i = 0; i < QK / 2; ++i) {
                    qv[i] = wb->qs[i] & 0x0f;
                    qv[i + QK / 2] = wb->qs[i] >> 4;
                }
                scale_w = mo_f16_to_f32(wb->scale);
                min_w = mo_f16_to_f32(wb->min);
            } else if (kind == MO_KIND_Q5_0) {
                const blk_q5_0 *wb = (const blk_q5_0 *)w + b;
                q5_unpack(wb->qh, wb->qs, qv);
                scale_w = mo_f16_to_f32(wb->scale);
            } else {
                const blk_q5_1 *wb = (const blk_q5_1 *)w + b;
                q5_unpack(wb->qh, wb->qs, qv);
                scale_w = mo_f16_to_f32(wb->scale);
                min_w = mo_f16_to_f32(wb->min);
            }
            const size_t start = b * QK;
            const size_t len = (start + QK <= k) ? QK : (k - start);
            for (size_t i = 0; i < len; ++i) {
                const float av = mo_f16_to_f32(a[start + i]);
                if (kind == MO_KIND_Q5_0) {
                    total += ((float)((int32_t)qv[i] - 16)) * scale_w * av;
                } else {
                    const float wv = scale_w * (float)qv[i] + min_w;
                    total += wv * av;
                }
            }
        }
    } else if (kind == MO_KIND_Q4_K) {
        const blk_q4_k *wb = (const blk_q4_k *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            const uint8_t *q = wb[b].qs;
            const float d = mo_f16_to_f32(wb[b].d);
            const float dmin = mo_f16_to_f32(wb[b].dmin);
            const size_t start = b * QK_K;
            const size_t len = (start + QK_K <= k) ? QK_K : (k - start);
            size_t written = 0;
            int is = 0;
            for (size_t j = 0; j < QK_K && written < len; j += 64) {
                uint8_t sc, m;
                get_scale_min_k4(is + 0, wb[b].scales, &sc, &m);
                const float d1 = d * (float)sc;
                const float m1 = dmin * (float)m;
                get_scale_min_k4(is + 1, wb[b].scales, &sc, &m);
                const float d2 = d * (float)sc;
                const float m2 = dmin * (float)m;
                for (int l = 0; l < 32 && written < len; ++l, ++written) {
                    const float av = mo_f16_to_f32(a[start + written]);
                    const float wv = d1 * (float)(q[l] & 0xF) - m1;
                    total += wv * av;
                }
                for (int l = 0; l < 32 && written < len; ++l, ++written) {
                    const float av = mo_f16_to_f32(a[start + written]);
                    const float wv = d2 * (float)(q[l] >> 4) - m2;
                    total += wv * av;
                }
                q += 32;
                is += 2;
            }
        }
    } else if (kind == MO_KIND_Q2_K) {
        /* vec_dot_impl.h:866-908 as written: one scale / min pair per 128 values (scales[0], scales[1]) and the
         * 2-bit values taken in sequential order (value i from bits 2 (i % 4) of qs[i / 4]); both differ from the
         * Q2_K dequantizer. Restated so that the reference's snapshot of this function is reproduced; no product
         * kernel mirrors it. */
        const blk_q2_k *wb = (const blk_q2_k *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            const float d = mo_f16_to_f32(wb[b].d);
            const float dmin = mo_f16_to_f32(wb[b].dmin);
            const uint8_t *q = wb[b].qs;
            const size_t start = b * QK_K;
            const size_t len = (start + QK_K <= k) ? QK_K : (k - start);
            size_t written = 0;
            for (size_t j = 0; j < QK_K && written < len; j += 128) {
                const size_t index = j / 128;
                const float dl = d * (float)(wb[b].scales[index] & 0xF);
                const float ml = dmin * (float)(wb[b].scales[index] >> 4);
                for (size_t i = 0; i < 128 && written < len; ++i, ++written) {
                    const uint8_t qv = (uint8_t)((q[(j + i) / 4] >> (((j + i) % 4) * 2)) & 0x3);
                    const float av = mo_f16_to_f32(a[start + written]);
                    const float wv = dl * (float)qv - ml;
                    total += wv * av;
                }
            }
        }
    } else if (kind == MO_KIND_Q3_K) {
        /* vec_dot_impl.h:910-971 as written: the high-bit mask advances once per 128 values instead of once per
         * 32, which differs from the Q3_K dequantizer. Restated for the same reason as Q2_K. */
        const blk_q3_k *wb = (const blk_q3_k *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            const float d_all = mo_f16_to_f32(wb[b].d);
            const uint8_t *q = wb[b].qs;
            const uint8_t *hm = wb[b].hmask;
            const size_t start = b * QK_K;
            const size_t len = (start + QK_K <= k) ? QK_K : (k - start);
            int8_t scales[16];
            q3_k_unpack_scales(wb[b].scales, scales);
            size_t written = 0;
            int is = 0;
            uint8_t m = 1;
            for (size_t n = 0; n < QK_K && written < len; n += 128) {
                int shift = 0;
                for (int j = 0; j < 4; ++j) {
                    for (int half = 0; half < 2; ++half) {
                        const float dl = d_all * (float)(scales[is++] - 32);
                        for (int l = 0; l < 16 && written < len; ++l, ++written) {
                            const int li = l + 16 * half;
                            const float av = mo_f16_to_f32(a[start + written]);
                            const int8_t qv = (int8_t)((int8_t)((q[li] >> shift) & 3) - ((hm[li] & m) ? 0 : 4));
                            total += dl * (float)qv * av;
                        }
                    }
                    shift += 2;
                }
                q += 32;
                m = (uint8_t)(m << 1);
            }
        }
    } else if (kind == MO_KIND_Q5_K) {
        /* vec_dot_impl.h:1025-1080 as written: the fifth bit is taken from byte j/8 + l (+ 32 for the high nibbles)
         * counted from the start of qh, bit j % 8 = 0, i.e. for j >= 64 and for every high nibble from bytes that
         * belong to other elements or to qs; it differs from the Q5_K dequantizer. Restated so that the reference's
         * snapshot of this function (golden_matmul_llama.h:1355) is reproduced; no product kernel mirrors it. */
        const blk_q5_k *wb = (const blk_q5_k *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            const uint8_t *ql = wb[b].qs;
            const uint8_t *qh = (const uint8_t *)&wb[b] + offsetof(blk_q5_k, qh); /* indexed past qh into qs */
            const float d = mo_f16_to_f32(wb[b].d);
            const float dmin = mo_f16_to_f32(wb[b].dmin);
            const size_t start = b * QK_K;
            const size_t len = (start + QK_K <= k) ? QK_K : (k - start);
            size_t written = 0;
            int is = 0;
            for (size_t j = 0; j < QK_K && written < len; j += 64) {
                uint8_t sc, m;
                get_scale_min_k4(is + 0, wb[b].scales, &sc, &m);
                const float d1 = d * (float)sc;
                const float m1 = dmin * (float)m;
                get_scale_min_k4(is + 1, wb[b].scales, &sc, &m);
                const float d2 = d * (float)sc;
                const float m2 = dmin * (float)m;
                for (int l = 0; l < 32 && written < len; ++l, ++written) {
                    const uint8_t h = (uint8_t)(qh[j / 8 + l] >> (j % 8) & 1);
                    const uint8_t q = (uint8_t)((ql[l] & 0xF) | (h << 4));
                    const float av = mo_f16_to_f32(a[start + written]);
                    const float wv = d1 * (float)q - m1;
                    total += wv * av;
                }
                for (int l = 0; l < 32 && written < len; ++l, ++written) {
                    const uint8_t h = (uint8_t)(qh[j / 8 + l + 32] >> (j % 8) & 1);
                    const uint8_t q = (uint8_t)((ql[l] >> 4) | (h << 4));
                    const float av = mo_f16_to_f32(a[start + written]);
                    const float wv = d2 * (float)q - m2;
                    total += wv * av;
                }
                ql += 32;
                is += 2;
            }
        }
    } else if (kind == MO_KIND_Q6_K) {
        const blk_q6_k *wb = (const blk_q6_k *)w;
        for (size_t b = 0; b < nblocks; ++b) {
            const uint8_t *ql = wb[b].ql;
            const uint8_t *qh = wb[b].qh;
            const float d = mo_f16_to_f32(wb[b].d);
            const size_t start = b * QK_K;
            const size_t len = (start + QK_K <= k) ? QK_K : (k - start);
            size_t written = 0;
            for (size_t j = 0; j < QK_K && written < len; j += 128) {
                const float scale = d * (float)wb[b].scales[j / 128];
                for (size_t i = 0; i < 128 && written < len; ++i, ++written) {
                    const size_t idx = j + i;
                    const uint8_t ql_val = (i % 2 == 0) ? (ql[idx / 2] & 0xF) : (ql[idx / 2] >> 4);
                    const uint8_t qh_val = (qh[idx / 4] >> ((idx % 4) * 2)) & 0x3;
                    const int8_t sq = (int8_t)((int8_t)(ql_val | (qh_val << 4)) - 32);
                    const float av = mo_f16_to_f32(a[start + written]);
                    total += (scale * (float)sq) * av;
                }
            }
        }
    }
    return total;
}

/* ======================= matmul driver ======================= */

typedef float (*dot_fn)(const void *w, const void *a, size_t nblocks);

static dot_fn pick_dot(int kind) {
    switch (kind) {
    case MO_KIND_Q8_0:
        return mo_vec_dot_q8_0_q8_0;
    case MO_KIND_Q4_0:
        return mo_vec_dot_q4_0_q8_0;
    case MO_KIND_Q8_1:
        return mo_vec_dot_q8_1_q8_0;
    case MO_KIND_Q4_1:
        return mo_vec_dot_q4_1_q8_0;
    case MO_KIND_Q5_0:
        return mo_vec_dot_q5_0_q8_0;
    case MO_KIND_Q5_1:
        return mo_vec_dot_q5_1_q8_0;
    case MO_KIND_Q4_K:
        return mo_vec_dot_q4_k_q8_k;
    case MO_KIND_Q5_K:
        return mo_vec_dot_q5_k_q8_k;
    case MO_KIND_Q2_K:
        return mo_vec_dot_q2_k_q8_k;
    case MO_KIND_Q3_K:
        return mo_vec_dot_q3_k_q8_k;
    case MO_KIND_Q6_K:
        return mo_vec_dot_q6_k_q8_k;
    default:
        return NULL;
    }
}

/* matmul_quant_compute.c:1222-1240 */
size_t mo_row_grain(size_t row_count, size_t cols_in_tile, size_t thread_cap) {
    size_t grain = BLOCK_ROWS;
    if (thread_cap == 0) {
        thread_cap = 1;
    }
    if (cols_in_tile <= 4 && row_count > grain * thread_cap) {
        const size_t target_tasks = thread_cap * (cols_in_tile <= 1 ? 8u : 12u);
        size_t dynamic = (row_count + target_tasks - 1) / target_tasks;
        dynamic = ((dynamic + MR - 1) / MR) * MR;
        if (dynamic > grain) {
            grain = dynamic;
        }
    }
    if (grain > 4096) {
        grain = 4096;
    }
    return grain;
}

typedef struct {
    int kind;
    int direct_f16;
    const uint8_t *weight;
    size_t row_bytes;
    size_t block_bytes;
    size_t blocks_per_row;
    size_t act_block_bytes;
    const uint8_t *act_tile;  /* packed path: cols_in_tile * blocks_per_row activation blocks */
    const uint16_t *act_f16;  /* direct path: input base */
    size_t K;
    size_t M;
    size_t n0;
    size_t cols_in_tile;
    float *out_f32;
    uint16_t *out_f16;
    dot_fn dot;
    /* work queue */
    size_t grain;
    size_t next_row;
    pthread_mutex_t lock;
} tile_job;

/* matmul_quant_compute.c:1032-1112 (generic) and :412-466 (Q8_0, >=2 columns): per (row, col) the
 * K blocks are consumed in chunks of 64, each chunk reduced inside the block dot, chunk sums added in order. */
static void tile_compute_rows(const tile_job *job, size_t row_start, size_t row_end) {
    for (size_t m = row_start; m < row_end; ++m) {
        const uint8_t *row_ptr = job->weight + m * job->row_bytes;
        for (size_t c = 0; c < job->cols_in_tile; ++c) {
            float dot = 0.0f;
            if (job->direct_f16) {
                /* matmul_quant_compute.c:1860-1890 */
                dot = mo_vec_dot_f16(job->kind, row_ptr, job->act_f16 + (job->n0 + c) * job->K, job->blocks_per_row,
                                     job->K);
            } else {
                const uint8_t *col = job->act_tile + c * job->blocks_per_row * job->act_block_bytes;
                for (size_t kb = 0; kb < job->blocks_per_row; kb += KC_BLOCKS) {
                    const size_t chunk =
                        (kb + KC_BLOCKS <= job->blocks_per_row) ? KC_BLOCKS : (job->blocks_per_row - kb);
                    dot += job->dot(row_ptr + kb * job->block_bytes, col + kb * job->act_block_bytes, chunk);
                }
            }
            if (job->out_f32 != NULL) {
                job->out_f32[(job->n0 + c) * job->M + m] = dot;
            }
            if (job->out_f16 != NULL) {
                job->out_f16[(job->n0 + c) * job->M + m] = mo_f32_to_f16(dot);
            }
        }
    }
}

static void *tile_worker(void *arg) {
    tile_job *job = (tile_job *)arg;
    for (;;) {
        pthread_mutex_lock(&job->lock);
        const size_t start = job->next_row;
        job->next_row = start + job->grain;
        pthread_mutex_unlock(&job->lock);
        if (start >= job->M) {
            break;
        }
        size_t end = start + job->grain;
        if (end > job->M) {
            end = job->M;
        }
        tile_compute_rows(job, start, end);
    }
    return NULL;
}

static void run_tile(tile_job *job, int threads) {
    job->next_row = 0;
    size_t tasks = (job->M + job->grain - 1) / job->grain;
    int nthreads = threads;
    if ((size_t)nthreads > tasks) {
        nthreads = (int)tasks;
    }
    if (nthreads <= 1) {
        tile_compute_rows(job, 0, job->M);
        return;
    }
    pthread_mutex_init(&job->lock, NULL);
    pthread_t *tids = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nthreads);
    int started = 0;
    for (int t = 0; t < nthreads - 1; ++t) {
        if (pthread_create(&tids[started], NULL, tile_worker, job) == 0) {
            started++;
        }
    }
    tile_worker(job);
    for (int t = 0; t < started; ++t) {
        pthread_join(tids[t], NULL);
    }
    free(tids);
    pthread_mutex_destroy(&job->lock);
}

/* matmul_quant_dispatch.c:373-591 + core/helpers/matmul.c:68-136 + matmul_epilogue.c */
int mo_matmul_quantized(
    int kind, const void *weight, const void *input, int in_dtype, size_t N, size_t K, size_t M, const float *bias,
    void *out, int out_dtype, int force_pack, int threads
) {
    if (weight == NULL || input == NULL || out == NULL) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    dot_fn dot = pick_dot(kind);
    if (dot == NULL) {
        return MO_ERR_UNSUPPORTED_DTYPE;
    }
    const int in_f32 = in_dtype == MO_DTYPE_F32;
    const int in_f16 = in_dtype == MO_DTYPE_F16;
    const int out_f32 = out_dtype == MO_DTYPE_F32;
    const int out_f16 = out_dtype == MO_DTYPE_F16;
    if (!((in_f32 && out_f32) || (in_f16 && (out_f32 || out_f16)))) {
        return MO_ERR_UNSUPPORTED_DTYPE;
    }
    if (threads < 1) {
        threads = 1;
    }
    const size_t bv = mo_block_values(kind);
    const size_t bb = mo_block_bytes(kind);
    const size_t blocks_per_row = (K + bv - 1) / bv;
    const int use_q8_k = (bv == QK_K);
    const size_t act_bb = use_q8_k ? sizeof(blk_q8_k) : sizeof(blk_q8_0);
    const int direct = in_f16 && !force_pack;

    tile_job job;
    memset(&job, 0, sizeof(job));
    job.kind = kind;
    job.direct_f16 = direct;
    job.weight = (const uint8_t *)weight;
    job.row_bytes = bb * blocks_per_row;
    job.block_bytes = bb;
    job.blocks_per_row = blocks_per_row;
    job.act_block_bytes = act_bb;
    job.K = K;
    job.M = M;
    job.out_f32 = out_f32 ? (float *)out : NULL;
    job.out_f16 = out_f16 ? (uint16_t *)out : NULL;
    job.dot = dot;
    job.act_f16 = (const uint16_t *)input;

    uint8_t *act_tile = NULL;
    if (!direct) {
        act_tile = (uint8_t *)malloc(TILE_COLS * blocks_per_row * act_bb + 1);
        if (act_tile == NULL) {
            return MO_ERR_OUT_OF_MEMORY;
        }
    }
    job.act_tile = act_tile;
    const size_t in_elt = in_f16 ? 2 : 4;

    for (size_t n0 = 0; n0 < N; n0 += TILE_COLS) {
        const size_t cols = (n0 + TILE_COLS <= N) ? TILE_COLS : (N - n0);
        job.n0 = n0;
        job.cols_in_tile = cols;
        if (!direct) {
            for (size_t c = 0; c < cols; ++c) {
                const uint8_t *row = (const uint8_t *)input + (n0 + c) * K * in_elt;
                uint8_t *dst = act_tile + c * blocks_per_row * act_bb;
                if (use_q8_k) {
                    mo_pack_q8_k(row, in_dtype, K, dst);
                } else {
                    mo_pack_q8_0(row, in_dtype, K, dst);
                }
            }
            job.grain = mo_row_grain(M, cols, (size_t)threads);
        } else {
            job.grain = 64; /* matmul_quant_compute.c:1936-1938 */
        }
        run_tile(&job, threads);
    }
    free(act_tile);

    if (bias != NULL) {
        if (out_f32) {
            float *o = (float *)out;
            for (size_t n = 0; n < N; ++n) {
                for (size_t m = 0; m < M; ++m) {
                    o[n * M + m] += bias[m];
                }
            }
        } else {
            uint16_t *o = (uint16_t *)out;
            for (size_t n = 0; n < N; ++n) {
                for (size_t m = 0; m < M; ++m) {
                    const float v = mo_f16_to_f32(o[n * M + m]);
                    o[n * M + m] = mo_f32_to_f16(v + bias[m]);
                }
            }
        }
    }
    return MO_OK;
}

/* cpu_matmul_qkv_resolve_head_dim (matmul_qkv_rope.h:14-23) */
size_t mo_rope_resolve_head_dim(size_t dim, uint32_t head_dim) {
    const size_t hd = (size_t)head_dim;
    if (hd == 0 || hd > dim || (dim % hd) != 0 || (hd & 1u) != 0u) {
        return dim;
    }
    return hd;
}

/* src/core/helpers/rope.c:61-110 (rope_scaling_prepare), :112-127 (compute_rope_frequencies), :143-200 */
int mo_rope_frequencies(const mo_rope_params *p, size_t head_dim, float *freqs_out, float *attn_scale_out) {
    if (p == NULL || freqs_out == NULL || attn_scale_out == NULL || (head_dim & 1u) != 0u) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    float freq_scale = p->freq_scale;
    float ext_factor = p->ext_factor;
    float attn_factor = p->attn_factor;
    if (freq_scale <= 0.0f) {
        freq_scale = 1.0f;
    }
    if (attn_factor <= 0.0f) {
        attn_factor = 1.0f;
    }
    if (p->scaling_type == 0 || p->scaling_type == -1) { /* none / unspecified */
        freq_scale = 1.0f;
        ext_factor = 0.0f;
    } else if (p->scaling_type == 1 || p->scaling_type == 3) { /* linear / longrope */
        ext_factor = 0.0f;
    }
    if (!(ext_factor != 0.0f && p->orig_ctx_len > 0 && p->theta > 0.0f && p->beta_fast > 0.0f &&
          p->beta_slow > 0.0f)) {
        ext_factor = 0.0f; /* rope.c:85-93: without the correction range YaRN degenerates to linear scaling */
    }
    float corr_low = 0.0f, corr_high = 0.0f;
    if (ext_factor != 0.0f) { /* rope_yarn_corr_dims (rope.c:46-59) with rope_yarn_corr_factor (:38-44) */
        const float denom = 2.0f * logf(p->theta);
        const float pi = 3.14159265358979323846f;
        float low_raw = 0.0f, high_raw = 0.0f;
        if (denom != 0.0f) {
            low_raw = (float)(int)head_dim * logf((float)(int)p->orig_ctx_len / (p->beta_fast * 2.0f * pi)) / denom;
            high_raw = (float)(int)head_dim * logf((float)(int)p->orig_ctx_len / (p->beta_slow * 2.0f * pi)) / denom;
        }
        corr_low = fmaxf(0.0f, floorf(low_raw));
        corr_high = fminf((float)((int)head_dim - 1), ceilf(high_raw));
    }
    float attn_scale = attn_factor; /* rope.c:95-99 */
    if (ext_factor != 0.0f) {
        const float inv_scale = 1.0f / freq_scale;
        attn_scale *= 1.0f + 0.1f * logf(inv_scale);
    }
    *attn_scale_out = attn_scale;
    const size_t half = head_dim / 2;
    for (size_t i = 0; i < half; ++i) { /* rope.c:112-127 */
        const float freq = powf(p->theta, -((float)(2 * i) / (float)head_dim));
        float scale = freq_scale;
        if (ext_factor != 0.0f) { /* rope_yarn_ramp (rope.c:28-36) */
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
    return MO_OK;
}

/* matmul_qkv_rope.h:50-70 */
static void rope_rotate_head(float *row, size_t dim, float position, const float *freqs, float attn_scale,
                             int rope_type) {
    const size_t pair_count = dim / 2;
    const size_t half_dim = dim / 2;
    const int is_neox = rope_type == 1;
    for (size_t i = 0; i < pair_count; ++i) {
        const float angle = position * freqs[i];
        float sin_theta = sinf(angle); /* cpu_sincosf (cpu_backend_internal.h:48-88) */
        float cos_theta = cosf(angle);
        cos_theta *= attn_scale;
        sin_theta *= attn_scale;
        const size_t even_index = is_neox ? i : 2 * i;
        const size_t odd_index = is_neox ? (i + half_dim) : (2 * i + 1);
        const float even = row[even_index];
        const float odd = row[odd_index];
        row[even_index] = even * cos_theta - odd * sin_theta;
        row[odd_index] = even * sin_theta + odd * cos_theta;
    }
}

/* matmul_qkv_rope.h:123-138 */
void mo_rope_rotate_row(float *row, size_t dim, size_t head_dim, float position, const float *freqs, float attn_scale,
                        int rope_type) {
    if (row == NULL || freqs == NULL) {
        return;
    }
    if (head_dim >= dim) {
        rope_rotate_head(row, dim, position, freqs, attn_scale, rope_type);
        return;
    }
    const size_t head_count = dim / head_dim;
    for (size_t h = 0; h < head_count; ++h) {
        rope_rotate_head(row + h * head_dim, head_dim, position, freqs, attn_scale, rope_type);
    }
}

/* cpu_rope, scalar path (src/backends/cpu/ops/rope/rope_dispatch.c:145-196, 287-372): rows of `dim` values, one
 * position per row, values loaded as fp32, rotated in fp32 and rounded once by the store */
int mo_rope(
    const void *x, int dtype, size_t rows, size_t dim, size_t x_row_stride, size_t out_row_stride,
    const mo_rope_params *rope, const void *positions, int pos_dtype, void *out
) {
    if (x == NULL || out == NULL || rope == NULL || positions == NULL) {
        return MO_ERR_INVALID_ARGUMENT; /* :147-155, 22-25 */
    }
    if (dtype != MO_DTYPE_F32 && dtype != MO_DTYPE_F16) {
        return MO_ERR_UNSUPPORTED_DTYPE;
    }
    if (dim % 2 != 0) {
        return MO_ERR_DIMENSION_MISMATCH; /* :45-49 */
    }
    if (rows == 0 || dim == 0) {
        return MO_ERR_INVALID_ARGUMENT; /* :51-56 */
    }
    if (pos_dtype != MO_DTYPE_F32 && pos_dtype != MO_DTYPE_I32 && pos_dtype != MO_DTYPE_I64) {
        return MO_ERR_UNSUPPORTED_DTYPE; /* :164-168 */
    }
    if (x_row_stride < dim || out_row_stride < dim) {
        return MO_ERR_DIMENSION_MISMATCH; /* :183-186 */
    }
    const size_t half = dim / 2;
    float *freqs = (float *)malloc(half * sizeof(float));
    if (freqs == NULL) {
        return MO_ERR_OUT_OF_MEMORY;
    }
    float attn_scale = 1.0f;
    const int st = mo_rope_frequencies(rope, dim, freqs, &attn_scale); /* cpu_rope_prepare_freqs (:123-143) */
    if (st != MO_OK) {
        free(freqs);
        return st;
    }
    const int is_neox = rope->rope_type == 1;
    for (size_t token = 0; token < rows; ++token) {
        float pos; /* cpu_rope_position_as_f32 (cpu_backend_internal.h:567-578) */
        if (pos_dtype == MO_DTYPE_F32) {
            pos = ((const float *)positions)[token];
        } else if (pos_dtype == MO_DTYPE_I32) {
            pos = (float)((const int32_t *)positions)[token];
        } else {
            pos = (float)((const int64_t *)positions)[token];
        }
        const size_t base_in = token * x_row_stride, base_out = token * out_row_stride;
        for (size_t i = 0; i < half; ++i) { /* :343-367 */
            const float angle = pos * freqs[i];
            float sin_theta = sinf(angle);
            float cos_theta = cosf(angle);
            cos_theta *= attn_scale;
            sin_theta *= attn_scale;
            const size_t even_offset = is_neox ? i : 2 * i;
            const size_t odd_offset = is_neox ? (i + half) : (2 * i + 1);
            float x_even, x_odd;
            if (dtype == MO_DTYPE_F16) {
                x_even = mo_f16_to_f32(((const uint16_t *)x)[base_in + even_offset]);
                x_odd = mo_f16_to_f32(((const uint16_t *)x)[base_in + odd_offset]);
            } else {
                x_even = ((const float *)x)[base_in + even_offset];
                x_odd = ((const float *)x)[base_in + odd_offset];
            }
            const float rotated_even = x_even * cos_theta - x_odd * sin_theta;
            const float rotated_odd = x_even * sin_theta + x_odd * cos_theta;
            if (dtype == MO_DTYPE_F16) {
                ((uint16_t *)out)[base_out + even_offset] = mo_f32_to_f16(rotated_even);
                ((uint16_t *)out)[base_out + odd_offset] = mo_f32_to_f16(rotated_odd);
            } else {
                ((float *)out)[base_out + even_offset] = rotated_even;
                ((float *)out)[base_out + odd_offset] = rotated_odd;
            }
        }
    }
    free(freqs);
    return MO_OK;
}

/* matmul_qkv.c:749-947 (cpu_matmul_qkv_run_separate_quantized_impl), value load/store helpers :89-116 */
int mo_matmul_qkv_separate_rope(
    int kind, const void *const weights[3], const void *input, int in_dtype, size_t N, size_t K, size_t M,
    const void *const bias[3], int bias_dtype, void *const out[3], const mo_rope_params *rope, const void *positions,
    int pos_dtype
) {
    if (weights == NULL || input == NULL || out == NULL) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    for (int i = 0; i < 3; ++i) {
        if (weights[i] == NULL || out[i] == NULL) {
            return MO_ERR_INVALID_ARGUMENT;
        }
    }
    if (in_dtype != MO_DTYPE_F32 && in_dtype != MO_DTYPE_F16) {
        return MO_ERR_NOT_IMPLEMENTED; /* :761-763 */
    }
    dot_fn dot = pick_dot(kind);
    if (dot == NULL) {
        return MO_ERR_NOT_IMPLEMENTED;
    }
    /* :809-822: the rotary state exists only when q or k is rotated */
    const int rope_q = rope != NULL && rope->apply_to_q;
    const int rope_k = rope != NULL && rope->apply_to_k;
    size_t head_dim = 0;
    float *freqs = NULL;
    float attn_scale = 1.0f;
    if (rope_q || rope_k) {
        if (positions == NULL ||
            (pos_dtype != MO_DTYPE_F32 && pos_dtype != MO_DTYPE_I32 && pos_dtype != MO_DTYPE_I64)) {
            return MO_ERR_INVALID_ARGUMENT;
        }
        head_dim = mo_rope_resolve_head_dim(M, rope->head_dim);
        if ((head_dim & 1u) != 0u) {
            return MO_ERR_INVALID_ARGUMENT; /* rope.c:159-162 */
        }
        freqs = (float *)malloc((head_dim / 2 + 1) * sizeof(float));
        if (freqs == NULL) {
            return MO_ERR_OUT_OF_MEMORY;
        }
        const int st = mo_rope_frequencies(rope, head_dim, freqs, &attn_scale);
        if (st != MO_OK) {
            free(freqs);
            return st;
        }
    }
    const size_t bv = mo_block_values(kind);
    const size_t bb = mo_block_bytes(kind);
    const size_t blocks_per_row = (K + bv - 1) / bv; /* :802 */
    const size_t row_bytes = bb * blocks_per_row;
    const int use_q8_k = (bv == QK_K);
    const size_t act_bb = use_q8_k ? sizeof(blk_q8_k) : sizeof(blk_q8_0);
    uint8_t *act = (uint8_t *)malloc(blocks_per_row * act_bb + 1);
    float *rows = (float *)malloc(3 * M * sizeof(float) + 1); /* the fp32 row buffers (:824-846, 883-886) */
    if (act == NULL || rows == NULL) {
        free(act);
        free(rows);
        free(freqs);
        return MO_ERR_OUT_OF_MEMORY;
    }
    const size_t in_elt = in_dtype == MO_DTYPE_F16 ? 2 : 4;
    for (size_t n = 0; n < N; ++n) { /* :876 */
        const uint8_t *row = (const uint8_t *)input + n * K * in_elt;
        if (use_q8_k) {
            mo_pack_q8_k(row, in_dtype, K, act);
        } else {
            mo_pack_q8_0(row, in_dtype, K, act);
        }
        for (size_t m = 0; m < M; ++m) { /* :888 */
            for (int i = 0; i < 3; ++i) {
                float acc = 0.0f; /* :889-891: the accumulator starts from the bias */
                if (bias != NULL && bias[i] != NULL) {
                    acc = bias_dtype == MO_DTYPE_F16 ? mo_f16_to_f32(((const uint16_t *)bias[i])[m])
                                                     : ((const float *)bias[i])[m];
                }
                acc += dot((const uint8_t *)weights[i] + m * row_bytes, act, blocks_per_row); /* :902-914 */
                rows[(size_t)i * M + m] = acc;
            }
        }
        if (rope_q || rope_k) { /* :917-924 -> cpu_matmul_qkv_apply_rope_row (:700-730) */
            float pos;
            if (pos_dtype == MO_DTYPE_F32) {
                pos = ((const float *)positions)[n];
            } else if (pos_dtype == MO_DTYPE_I32) {
                pos = (float)((const int32_t *)positions)[n];
            } else {
                pos = (float)((const int64_t *)positions)[n];
            }
            if (rope_q) {
                mo_rope_rotate_row(rows, M, head_dim, pos, freqs, attn_scale, rope->rope_type);
            }
            if (rope_k) {
                mo_rope_rotate_row(rows + M, M, head_dim, pos, freqs, attn_scale, rope->rope_type);
            }
        }
        for (int i = 0; i < 3; ++i) { /* the store rounds once (:107-109, 687-698) */
            for (size_t m = 0; m < M; ++m) {
                const float v = rows[(size_t)i * M + m];
                if (in_dtype == MO_DTYPE_F16) {
                    ((uint16_t *)out[i])[n * M + m] = mo_f32_to_f16(v);
                } else {
                    ((float *)out[i])[n * M + m] = v;
                }
            }
        }
    }
    free(act);
    free(rows);
    free(freqs);
    return MO_OK;
}

int mo_matmul_qkv_separate(
    int kind, const void *const weights[3], const void *input, int in_dtype, size_t N, size_t K, size_t M,
    const void *const bias[3], int bias_dtype, void *const out[3]
) {
    return mo_matmul_qkv_separate_rope(kind, weights, input, in_dtype, N, K, M, bias, bias_dtype, out, NULL, NULL, 0);
}

/* ======================= embedding gather ======================= */

/* embedding_scalar.c:381-447 (worker), :241-303 (quantized row), :167-185 (zero row), :187-209 (stores) */
int mo_embedding_gather_quantized(
    int kind, const void *weights, size_t vocab, size_t dim, const void *ids, int ids_dtype, size_t n, void *out,
    int out_dtype, float scale, int32_t padding_id, int bounds_check, size_t *error_index
) {
    const size_t bv = mo_block_values(kind);
    const size_t bb = mo_block_bytes(kind);
    if (bv == 0 || weights == NULL || ids == NULL || out == NULL) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    if (ids_dtype != MO_DTYPE_I32 && ids_dtype != MO_DTYPE_I64) {
        return MO_ERR_UNSUPPORTED_DTYPE;
    }
    if (out_dtype != MO_DTYPE_F32 && out_dtype != MO_DTYPE_F16) {
        return MO_ERR_UNSUPPORTED_DTYPE;
    }
    const size_t blocks_per_row = (dim + bv - 1) / bv;
    const size_t row_bytes = blocks_per_row * bb;
    float decoded[QK_K];
    for (size_t idx = 0; idx < n; ++idx) {
        const int64_t token = ids_dtype == MO_DTYPE_I32 ? (int64_t)((const int32_t *)ids)[idx]
                                                        : ((const int64_t *)ids)[idx];
        int zero = 0;
        if (padding_id >= 0 && token == (int64_t)padding_id) {
            zero = 1; /* :411-414 */
        } else if (token < 0 || (uint64_t)token >= (uint64_t)vocab) {
            if (bounds_check) { /* :416-423 */
                if (error_index != NULL) {
                    *error_index = idx;
                }
                return MO_ERR_INVALID_ARGUMENT;
            }
            zero = 1;
        }
        if (zero) { /* :167-177: memset of the row */
            if (out_dtype == MO_DTYPE_F32) {
                memset((float *)out + idx * dim, 0, dim * sizeof(float));
            } else {
                memset((uint16_t *)out + idx * dim, 0, dim * sizeof(uint16_t));
            }
            continue;
        }
        const uint8_t *row = (const uint8_t *)weights + (size_t)token * row_bytes;
        for (size_t b = 0; b < blocks_per_row; ++b) { /* :255-300 */
            const size_t base_col = b * bv;
            if (base_col >= dim) {
                break;
            }
            const size_t remaining = dim - base_col;
            const size_t count = remaining < bv ? remaining : bv;
            const uint8_t *blk = row + b * bb;
            switch (kind) {
            case MO_KIND_Q4_0: { /* cpu_embedding_decode_q4_0_interleaved, :221-229 */
                const blk_q4_0 *q = (const blk_q4_0 *)blk;
                const float sc = mo_f16_to_f32(q->scale);
                for (size_t i = 0; i < count; ++i) {
                    const uint8_t packed = q->qs[i >> 1];
                    int32_t v = (i & 1) ? ((packed >> 4) & 0x0f) : (packed & 0x0f);
                    v -= 8;
                    decoded[i] = sc * (float)v;
                }
                break;
            }
            case MO_KIND_Q8_0:
                q8_0_dequantize_block((const blk_q8_0 *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q4_1: { /* cpu_embedding_decode_q4_1_interleaved, :231-240. The reference holds no golden for
                                  * this case: the tests pin it as the Q4_1 dequantizer's values (golden) in the
                                  * Q4_0 case's nibble order (golden). */
                const blk_q4_1 *q = (const blk_q4_1 *)blk;
                const float sc = mo_f16_to_f32(q->scale);
                const float mn = mo_f16_to_f32(q->min);
                for (size_t i = 0; i < count; ++i) {
                    const uint8_t packed = q->qs[i >> 1];
                    const uint8_t v = (uint8_t)((i & 1) ? ((packed >> 4) & 0x0f) : (packed & 0x0f));
                    decoded[i] = sc * (float)v + mn;
                }
                break;
            }
            /* Q5_0 / Q5_1 use their dequantizers. */
            case MO_KIND_Q8_1:
                q8_1_dequantize_block((const blk_q8_1 *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q5_0:
                q5_0_dequantize_block((const blk_q5_0 *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q5_1:
                q5_1_dequantize_block((const blk_q5_1 *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q4_K:
                q4_k_dequantize_block((const blk_q4_k *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q5_K:
                q5_k_dequantize_block((const blk_q5_k *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q2_K:
                q2_k_dequantize_block((const blk_q2_k *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q3_K:
                q3_k_dequantize_block((const blk_q3_k *)blk, (uint32_t)count, decoded);
                break;
            case MO_KIND_Q6_K:
                q6_k_dequantize_block((const blk_q6_k *)blk, (uint32_t)count, decoded);
                break;
            default:
                return MO_ERR_NOT_IMPLEMENTED;
            }
            if (out_dtype == MO_DTYPE_F32) { /* :187-199 */
                float *o = (float *)out + idx * dim + base_col;
                for (size_t i = 0; i < count; ++i) {
                    o[i] = scale == 1.0f ? decoded[i] : decoded[i] * scale;
                }
            } else { /* :201-209 */
                uint16_t *o = (uint16_t *)out + idx * dim + base_col;
                for (size_t i = 0; i < count; ++i) {
                    o[i] = mo_f32_to_f16(decoded[i] * scale);
                }
            }
        }
    }
    return MO_OK;
}

/* ======================= top-k / router / MoE ======================= */

/* moe_ops.c:789-889 */
int mo_topk(const float *x, size_t rows, size_t cols, size_t k, float *values_out, int32_t *indices_out) {
    if (x == NULL || values_out == NULL || indices_out == NULL || k == 0 || k > cols) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    for (size_t row = 0; row < rows; ++row) {
        float *bvals = values_out + row * k;
        int32_t *bidx = indices_out + row * k;
        for (size_t i = 0; i < k; ++i) {
            bvals[i] = -FLT_MAX;
            bidx[i] = -1;
        }
        for (size_t col = 0; col < cols; ++col) {
            const float value = x[row * cols + col];
            size_t insert_pos = k;
            for (size_t i = 0; i < k; ++i) {
                const int better = value > bvals[i];
                const int same = value == bvals[i] && (int32_t)col < bidx[i];
                if (better || same) {
                    insert_pos = i;
                    break;
                }
            }
            if (insert_pos == k) {
                continue;
            }
            for (size_t i = k - 1; i > insert_pos; --i) {
                bvals[i] = bvals[i - 1];
                bidx[i] = bidx[i - 1];
            }
            bvals[insert_pos] = value;
            bidx[insert_pos] = (int32_t)col;
        }
    }
    return MO_OK;
}

/* Numerically-stable softmax over the selected logits; the graph applies marmot's generic softmax op
 * to the [T,k] top-k values (graph_builder.cpp:2276-2316): max-subtract, expf, sum in order, divide. */
void mo_softmax_rows(const float *x, size_t rows, size_t k, float *out) {
    for (size_t r = 0; r < rows; ++r) {
        const float *in = x + r * k;
        float *o = out + r * k;
        float mx = in[0];
        for (size_t i = 1; i < k; ++i) {
            if (in[i] > mx) {
                mx = in[i];
            }
        }
        float sum = 0.0f;
        for (size_t i = 0; i < k; ++i) {
            o[i] = expf(in[i] - mx);
            sum += o[i];
        }
        for (size_t i = 0; i < k; ++i) {
            o[i] = o[i] / sum;
        }
    }
}

/* moe_ops.c:318-324 */
static inline float moe_silu(float x) {
    return x / (1.0f + expf(-x));
}
static inline float moe_gelu(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}

/* ---- the fp32 ops between the linears
 * RMS normalization, scalar float32 path: compute_mean_square_scalar + normalize_rms_scalar
 * (src/backends/cpu/ops/normalization/scalar/normalization_scalar.c:469-510, 780-791), 1 / sqrtf
 * (normalization_internal.h:8-10); weight_offset 0 is cpu_rmsnorm_impl, 1 cpu_rmsnorm_gemma_impl
 * (normalization_dispatch.c:240-246). residual and weight may be NULL. */
int mo_rms_norm(const float *x, const float *residual, const float *weight, float weight_offset, float eps,
                size_t rows, size_t cols, float *out) {
    if (rows == 0 || cols == 0) {
        return MO_OK;
    }
    for (size_t r = 0; r < rows; ++r) {
        const float *xr = x + r * cols;
        const float *rr = residual != NULL ? residual + r * cols : NULL;
        float *or_ = out + r * cols;
        float sum = 0.0f;
        for (size_t i = 0; i < cols; ++i) {
            float v = xr[i];
            if (rr != NULL) {
                v += rr[i];
            }
            sum += v * v;
        }
        const float mean_sq = sum / (float)cols;
        const float inv_rms = 1.0f / sqrtf(mean_sq + eps);
        for (size_t i = 0; i < cols; ++i) {
            float v = xr[i];
            if (rr != NULL) {
                v = xr[i] + rr[i];
            }
            or_[i] = weight != NULL ? v * inv_rms * (weight[i] + weight_offset) : v * inv_rms;
        }
    }
    return MO_OK;
}

/* cpu_swiglu_f32_scalar / cpu_geglu_f32_scalar (src/backends/cpu/ops/elementwise/scalar/elementwise_f32_scalar.c:
 * 11-20, 147-214): out = silu(gate) * up, or gelu_tanh(gate) * up (geglu != 0). */
int mo_glu(const float *gate, const float *up, size_t n, int geglu, float *out) {
    for (size_t i = 0; i < n; ++i) {
        const float g = gate[i];
        float a;
        if (geglu) {
            const float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
            a = 0.5f * g * (1.0f + tanhf(inner));
        } else {
            a = g / (1.0f + expf(-g));
        }
        out[i] = a * up[i];
    }
    return MO_OK;
}

/* The gated product of moe_ops.c:548-559 on its own: out[i] = act(gate[i]) * up[i]. */
int mo_moe_glu(const float *gate, const float *up, size_t n, int ffn_type, float *out) {
    if (ffn_type != MO_FFN_SWIGLU && ffn_type != MO_FFN_GEGLU) {
        return MO_ERR_NOT_IMPLEMENTED;
    }
    for (size_t i = 0; i < n; ++i) {
        const float g = gate[i];
        out[i] = (ffn_type == MO_FFN_GEGLU ? moe_gelu(g) : moe_silu(g)) * up[i];
    }
    return MO_OK;
}

/* moe_ops.c:506-568: gate/up (shared activation quantization) -> act(gate)*up -> down */
static int moe_expert_body(
    const float *rows_in, size_t count, size_t H, size_t F, int kind_gu, int kind_down, const uint8_t *gate_w,
    const uint8_t *up_w, const uint8_t *down_w, int ffn_type, int threads, float *gate_buf, float *up_buf,
    float *down_out
) {
    int st = mo_matmul_quantized(kind_gu, gate_w, rows_in, MO_DTYPE_F32, count, H, F, NULL, gate_buf, MO_DTYPE_F32, 0,
                                 threads);
    if (st != MO_OK) {
        return st;
    }
    st = mo_matmul_quantized(kind_gu, up_w, rows_in, MO_DTYPE_F32, count, H, F, NULL, up_buf, MO_DTYPE_F32, 0,
                             threads);
    if (st != MO_OK) {
        return st;
    }
    st = mo_moe_glu(gate_buf, up_buf, count * F, ffn_type, gate_buf);
    if (st != MO_OK) {
        return st;
    }
    return mo_matmul_quantized(kind_down, down_w, gate_buf, MO_DTYPE_F32, count, F, H, NULL, down_out, MO_DTYPE_F32,
                               0, threads);
}

/* moe_ops.c:475-504: active experts by descending route count, ties by ascending id */
static size_t moe_build_expert_order(size_t *order, const size_t *counts, size_t E) {
    size_t active = 0;
    for (size_t e = 0; e < E; ++e) {
        if (counts[e] != 0) {
            order[active++] = e;
        }
    }
    for (size_t i = 1; i < active; ++i) {
        const size_t e = order[i];
        const size_t c = counts[e];
        size_t j = i;
        while (j > 0) {
            const size_t pe = order[j - 1];
            const size_t pc = counts[pe];
            if (pc > c || (pc == c && pe < e)) {
                break;
            }
            order[j] = pe;
            --j;
        }
        order[j] = e;
    }
    return active;
}

typedef struct {
    size_t H, F;
    int kind_gu, kind_down;
    const uint8_t *gate, *up, *down;
    size_t gu_slice, down_slice;
    int ffn_type;
    const size_t *counts;
    const size_t *offsets;
    size_t *order;
    size_t active;
    const float *route_hidden;
    float *route_down;
    float *gate_buf;
    float *up_buf;
    int inner_threads;
    size_t next;
    int first_error;
    pthread_mutex_t lock;
} moe_group_ctx;

static void *moe_group_worker(void *arg) {
    moe_group_ctx *g = (moe_group_ctx *)arg;
    for (;;) {
        pthread_mutex_lock(&g->lock);
        const size_t idx = g->next++;
        const int err = g->first_error;
        pthread_mutex_unlock(&g->lock);
        if (err != MO_OK || idx >= g->active) {
            break;
        }
        const size_t e = g->order[idx];
        const size_t off = g->offsets[e];
        const int st = moe_expert_body(
            g->route_hidden + off * g->H, g->counts[e], g->H, g->F, g->kind_gu, g->kind_down,
            g->gate + e * g->gu_slice, g->up + e * g->gu_slice, g->down + e * g->down_slice, g->ffn_type,
            g->inner_threads, g->gate_buf + off * g->F, g->up_buf + off * g->F, g->route_down + off * g->H
        );
        if (st != MO_OK) {
            pthread_mutex_lock(&g->lock);
            if (g->first_error == MO_OK) {
                g->first_error = st;
            }
            pthread_mutex_unlock(&g->lock);
            break;
        }
    }
    return NULL;
}

static int moe_run_group(moe_group_ctx *g, int workers) {
    g->next = 0;
    g->first_error = MO_OK;
    pthread_mutex_init(&g->lock, NULL);
    if ((size_t)workers > g->active) {
        workers = (int)g->active;
    }
    if (workers <= 1) {
        moe_group_worker(g);
    } else {
        pthread_t *tids = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)workers);
        int started = 0;
        for (int t = 0; t < workers - 1; ++t) {
            if (pthread_create(&tids[started], NULL, moe_group_worker, g) == 0) {
                started++;
            }
        }
        moe_group_worker(g);
        for (int t = 0; t < started; ++t) {
            pthread_join(tids[t], NULL);
        }
        free(tids);
    }
    pthread_mutex_destroy(&g->lock);
    return g->first_error;
}

int mo_moe_experts(
    const float *hidden, size_t T, size_t H, size_t F, size_t E, size_t kpt, int kind_gu, int kind_down,
    const void *gate, const void *up, const void *down, const int32_t *topk_ids, const float *topk_weights,
    float weights_scale, int policy, int ffn_type, int force_grouped, int threads, float *out
) {
    if (hidden == NULL || gate == NULL || up == NULL || down == NULL || topk_ids == NULL || topk_weights == NULL ||
        out == NULL) {
        return MO_ERR_INVALID_ARGUMENT;
    }
    if (ffn_type != MO_FFN_SWIGLU && ffn_type != MO_FFN_GEGLU) {
        return MO_ERR_NOT_IMPLEMENTED;
    }
    const size_t routes = T * kpt;
    const size_t gu_slice = F * mo_row_bytes(kind_gu, H);  /* moe_ops.c:326-345 */
    const size_t down_slice = H * mo_row_bytes(kind_down, F);
    if (gu_slice == 0 || down_slice == 0) {
        return MO_ERR_UNSUPPORTED_DTYPE;
    }

    uint32_t *sorted_tokens = (uint32_t *)malloc((routes + 1) * sizeof(uint32_t));
    float *sorted_weights = (float *)malloc((routes + 1) * sizeof(float));
    size_t *counts = (size_t *)calloc(E + 1, sizeof(size_t));
    size_t *offsets = (size_t *)calloc(E + 1, sizeof(size_t));
    size_t *cursor = (size_t *)calloc(E + 1, sizeof(size_t));
    float *route_hidden = (float *)malloc((routes * H + 1) * sizeof(float));
    float *route_down = (float *)malloc((routes * H + 1) * sizeof(float));
    float *gate_buf = (float *)malloc((routes * F + 1) * sizeof(float));
    float *up_buf = (float *)malloc((routes * F + 1) * sizeof(float));
    int status = MO_OK;
    if (!sorted_tokens || !sorted_weights || !counts || !offsets || !cursor || !route_hidden || !route_down ||
        !gate_buf || !up_buf) {
        status = MO_ERR_OUT_OF_MEMORY;
        goto done;
    }

    const int decode = !force_grouped && T <= 4 && routes <= 64; /* moe_ops.c:417-424 */

    if (decode) {
        /* moe_ops.c:622-787: experts in first-appearance order */
        uint32_t active[64];
        size_t acount[64], aoff[64], acur[64];
        size_t nactive = 0;
        for (size_t t = 0; t < T; ++t) {
            memset(out + t * H, 0, H * sizeof(float));
            for (size_t s = 0; s < kpt; ++s) {
                const int32_t e = topk_ids[t * kpt + s];
                if (e < 0) {
                    status = MO_ERR_INVALID_ARGUMENT;
                    goto done;
                }
                size_t slot = 0;
                for (; slot < nactive; ++slot) {
                    if (active[slot] == (uint32_t)e) {
                        break;
                    }
                }
                if (slot == nactive) {
                    active[nactive] = (uint32_t)e;
                    acount[nactive] = 0;
                    nactive++;
                }
                acount[slot]++;
            }
        }
        size_t prefix = 0;
        for (size_t slot = 0; slot < nactive; ++slot) {
            aoff[slot] = prefix;
            acur[slot] = prefix;
            prefix += acount[slot];
        }
        for (size_t t = 0; t < T; ++t) {
            float norm = weights_scale;
            if (policy == MO_ROUTER_RENORMALIZE_SELECTED) {
                float ws = 0.0f;
                for (size_t s = 0; s < kpt; ++s) {
                    ws += topk_weights[t * kpt + s];
                }
                norm = ws > FLT_MIN ? weights_scale / ws : 0.0f;
            }
            for (size_t s = 0; s < kpt; ++s) {
                const uint32_t e = (uint32_t)topk_ids[t * kpt + s];
                size_t slot = 0;
                for (; slot < nactive; ++slot) {
                    if (active[slot] == e) {
                        break;
                    }
                }
                const size_t pos = acur[slot]++;
                sorted_tokens[pos] = (uint32_t)t;
                sorted_weights[pos] = topk_weights[t * kpt + s] * norm;
            }
        }
        for (size_t slot = 0; slot < nactive; ++slot) {
            const size_t count = acount[slot];
            const size_t off = aoff[slot];
            const size_t e = active[slot];
            if (e >= E) {
                status = MO_ERR_INVALID_ARGUMENT;
                goto done;
            }
            for (size_t r = 0; r < count; ++r) {
                memcpy(route_hidden + r * H, hidden + (size_t)sorted_tokens[off + r] * H, H * sizeof(float));
            }
            status = moe_expert_body(route_hidden, count, H, F, kind_gu, kind_down,
                                     (const uint8_t *)gate + e * gu_slice, (const uint8_t *)up + e * gu_slice,
                                     (const uint8_t *)down + e * down_slice, ffn_type, threads, gate_buf, up_buf,
                                     route_down);
            if (status != MO_OK) {
                goto done;
            }
            for (size_t r = 0; r < count; ++r) {
                const size_t t = sorted_tokens[off + r];
                const float w = sorted_weights[off + r];
                for (size_t c = 0; c < H; ++c) {
                    out[t * H + c] += w * route_down[r * H + c];
                }
            }
        }
        goto done;
    }

    /* grouped path: moe_ops.c:891-1049 */
    for (size_t t = 0; t < T; ++t) {
        for (size_t s = 0; s < kpt; ++s) {
            const int32_t e = topk_ids[t * kpt + s];
            if (e < 0 || (size_t)e >= E) {
                status = MO_ERR_INVALID_ARGUMENT;
                goto done;
            }
            counts[e]++;
        }
    }
    size_t prefix = 0;
    for (size_t e = 0; e < E; ++e) {
        offsets[e] = prefix;
        cursor[e] = prefix;
        prefix += counts[e];
    }
    for (size_t t = 0; t < T; ++t) {
        float norm = weights_scale;
        if (policy == MO_ROUTER_RENORMALIZE_SELECTED) {
            float ws = 0.0f;
            for (size_t s = 0; s < kpt; ++s) {
                ws += topk_weights[t * kpt + s];
            }
            norm = ws > FLT_MIN ? weights_scale / ws : 0.0f;
        }
        for (size_t s = 0; s < kpt; ++s) {
            const size_t e = (size_t)topk_ids[t * kpt + s];
            const size_t pos = cursor[e]++;
            sorted_tokens[pos] = (uint32_t)t;
            sorted_weights[pos] = topk_weights[t * kpt + s] * norm;
        }
    }
    for (size_t r = 0; r < routes; ++r) {
        memcpy(route_hidden + r * H, hidden + (size_t)sorted_tokens[r] * H, H * sizeof(float));
    }
    for (size_t t = 0; t < T; ++t) {
        memset(out + t * H, 0, H * sizeof(float));
    }
    /* moe_ops.c:475-504, 586-620, 1004-1031: experts are visited in descending-count order, in parallel over
     * experts (inner matmul single-threaded) when there are >= 32 routes and more than one thread. Each expert
     * writes disjoint slices of the route buffers, so the visiting order does not change any value. */
    {
        moe_group_ctx g;
        memset(&g, 0, sizeof(g));
        g.H = H;
        g.F = F;
        g.kind_gu = kind_gu;
        g.kind_down = kind_down;
        g.gate = (const uint8_t *)gate;
        g.up = (const uint8_t *)up;
        g.down = (const uint8_t *)down;
        g.gu_slice = gu_slice;
        g.down_slice = down_slice;
        g.ffn_type = ffn_type;
        g.counts = counts;
        g.offsets = offsets;
        g.route_hidden = route_hidden;
        g.route_down = route_down;
        g.gate_buf = gate_buf;
        g.up_buf = up_buf;
        g.order = cursor; /* cursor[] is no longer needed: reuse as the visiting order */
        g.active = moe_build_expert_order(g.order, counts, E);
        const int parallel = threads > 1 && routes >= 32;
        g.inner_threads = parallel ? 1 : threads;
        status = moe_run_group(&g, parallel ? threads : 1);
        if (status != MO_OK) {
            goto done;
        }
    }
    /* moe_ops.c:1034-1042: scatter in sorted-route order */
    for (size_t r = 0; r < routes; ++r) {
        const size_t t = sorted_tokens[r];
        const float w = sorted_weights[r];
        for (size_t c = 0; c < H; ++c) {
            out[t * H + c] += w * route_down[r * H + c];
        }
    }

done:
    free(sorted_tokens);
    free(sorted_weights);
    free(counts);
    free(offsets);
    free(cursor);
    free(route_hidden);
    free(route_down);
    free(gate_buf);
    free(up_buf);
    return status;
}

/* ======================= paged attention ======================= */

/* marmot_f32_to_bf16_ref / marmot_bf16_to_f32_ref (src/utils/dtype_ref.c:86-104): round to nearest even on the bits */
static uint16_t pa_f32_to_bf16(float value) {
    uint32_t bits;
    memcpy(&bits, &value, sizeof(bits));
    const uint32_t bias = 0x7FFFu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + bias) >> 16);
}

static float pa_bf16_to_f32(uint16_t h) {
    const uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, sizeof(f));
    return f;
}

/* marmot_fp8_quantize with 4 exponent bits, 3 mantissa bits, bias 7, no infinity, max 240 (dtype_ref.c:118-176) */
uint8_t mo_f32_to_fp8_e4m3(float value) {
    if (isnan(value)) {
        return 0x79; /* exponent field 15, payload 1, sign 0 */
    }
    const uint8_t sign = value < 0 ? 0x80 : 0;
    const float mag = fabsf(value);
    if (isinf(value) || mag > 240.0f) {
        return (uint8_t)(sign | 0x77); /* largest finite: exponent field 14, mantissa 7 */
    }
    if (mag == 0.0f) {
        return sign;
    }
    int e;
    float m = frexpf(mag, &e); /* mag = m * 2^e, m in [0.5, 1) */
    m *= 2.0f;
    e -= 1;
    int field = e + 7;
    if (field > 0 && field < 15) {
        int r = (int)lrintf((m - 1.0f) * 8.0f); /* nearest, ties to even */
        if (r == 8) {
            r = 0;
            field += 1;
            if (field >= 15) {
                return (uint8_t)(sign | 0x77);
            }
        }
        return (uint8_t)(sign | (field << 3) | (r & 7));
    }
    /* below the smallest normal 2^-6: multiples of 2^-9 */
    int r = (int)lrintf(ldexpf(mag, 6 + 3));
    if (r == 0) {
        return sign;
    }
    if (r > 7) {
        r = 7;
    }
    return (uint8_t)(sign | r);
}

/* marmot_fp8_dequantize, same format (dtype_ref.c:178-205) */
float mo_fp8_e4m3_to_f32(uint8_t bits) {
    const int field = (bits >> 3) & 15, mant = bits & 7;
    const float s = (bits & 0x80) ? -1.0f : 1.0f;
    if (field == 15) {
        return nanf("");
    }
    if (field == 0) {
        return mant == 0 ? ((bits & 0x80) ? -0.0f : 0.0f) : s * ldexpf((float)mant / 8.0f, -6);
    }
    return s * ldexpf(1.0f + (float)mant / 8.0f, field - 7);
}

/* cpu_paged_attention_fp8_quant / _dequant / _scale_from_max (paged_attention_ref.c:142-163) */
static uint8_t pa_fp8_quant(float value, float scale) {
    return scale > 0.0f ? mo_f32_to_fp8_e4m3(value / scale) : 0;
}
static float pa_fp8_dequant(uint8_t v, float scale) {
    return scale > 0.0f ? mo_fp8_e4m3_to_f32(v) * scale : 0.0f;
}
static float pa_fp8_scale(float max_abs) {
    return max_abs > 0.0f ? max_abs / 240.0f : 1.0f;
}

/* cpu_load_as_f32 / cpu_store_from_f32 (cpu_backend_internal.h:641-680) for the three float types */
static float pa_load(int dtype, const void *data, size_t index) {
    switch (dtype) {
    case MO_DTYPE_F16:
        return mo_f16_to_f32(((const uint16_t *)data)[index]);
    case MO_DTYPE_BF16:
        return pa_bf16_to_f32(((const uint16_t *)data)[index]);
    default:
        return ((const float *)data)[index];
    }
}

static void pa_store(int dtype, void *data, size_t index, float value) {
    switch (dtype) {
    case MO_DTYPE_F16:
        ((uint16_t *)data)[index] = mo_f32_to_f16(value);
        break;
    case MO_DTYPE_BF16:
        ((uint16_t *)data)[index] = pa_f32_to_bf16(value);
        break;
    default:
        ((float *)data)[index] = value;
        break;
    }
}

static int pa_float_dtype(int dtype) {
    return dtype == MO_DTYPE_F32 || dtype == MO_DTYPE_F16 || dtype == MO_DTYPE_BF16;
}

/* cpu_paged_attention_choose_block_n, paged_attention_ref.c:31-50 */
static size_t pa_block_n(size_t head_dim) {
    size_t rows = (64u * 1024u) / (2 * head_dim * sizeof(float));
    if (rows < 32) {
        rows = 32;
    }
    if (rows > 256) {
        rows = 256;
    }
    return rows;
}

int mo_paged_attention(const mo_paged_attention_args *a) {
    if (a == NULL || a->token_meta == NULL || a->q == NULL || a->k_new == NULL || a->v_new == NULL || a->kv_k == NULL ||
        a->kv_v == NULL || a->block_table == NULL || a->out == NULL) {
        return MO_ERR_INVALID_ARGUMENT; /* :574-577, :799-803 */
    }
    if (a->token_count == 0) {
        return 0;
    }
    if (a->num_q_heads == 0 || a->num_kv_heads == 0 || a->head_dim == 0 || a->block_size == 0 ||
        (a->block_size & (a->block_size - 1u)) != 0 || a->num_q_heads % a->num_kv_heads != 0) {
        return MO_ERR_INVALID_ARGUMENT; /* :581-596 */
    }
    const int fp8 = a->kv_dtype == MO_DTYPE_F8_E4M3;
    if (!pa_float_dtype(a->act_dtype) || (!fp8 && !pa_float_dtype(a->kv_dtype))) {
        return MO_ERR_UNSUPPORTED_DTYPE; /* :622-630 */
    }
    if (fp8 && (a->kv_k_scale == NULL || a->kv_v_scale == NULL)) {
        return MO_ERR_INVALID_ARGUMENT; /* :695-698 */
    }
    if (a->kv_layers <= a->layer_idx) {
        return MO_ERR_DIMENSION_MISMATCH; /* :673-676 */
    }
    uint32_t shift = 0;
    while ((1u << shift) < a->block_size) {
        ++shift;
    }
    const uint32_t mask = a->block_size - 1u;
    const size_t hd = a->head_dim;
    for (size_t t = 0; t < a->token_count; ++t) { /* :809-823 */
        const uint32_t seq_slot = a->token_meta[t * a->meta_stride[0]];
        const uint32_t kv_slot = a->token_meta[t * a->meta_stride[0] + 2 * a->meta_stride[1]];
        if (seq_slot >= a->max_seqs || (kv_slot >> shift) >= a->kv_blocks) {
            return MO_ERR_DIMENSION_MISMATCH;
        }
    }
    if (fp8) { /* :825-989 */
        const size_t nb = a->kv_blocks, nh = a->num_kv_heads;
        uint32_t *min_off = (uint32_t *)malloc(nb * sizeof(uint32_t));
        float *new_k = (float *)calloc(nb * nh, sizeof(float)), *new_v = (float *)calloc(nb * nh, sizeof(float));
        if (min_off == NULL || new_k == NULL || new_v == NULL) {
            free(min_off), free(new_k), free(new_v);
            return MO_ERR_INVALID_ARGUMENT;
        }
        for (size_t b = 0; b < nb; ++b) {
            min_off[b] = a->block_size; /* "untouched" */
        }
        for (size_t t = 0; t < a->token_count; ++t) { /* largest magnitudes of the new rows, first offset written */
            const uint32_t kv_slot = a->token_meta[t * a->meta_stride[0] + 2 * a->meta_stride[1]];
            const uint32_t b = kv_slot >> shift, off = kv_slot & mask;
            if (off < min_off[b]) {
                min_off[b] = off;
            }
            for (size_t h = 0; h < nh; ++h) {
                for (size_t d = 0; d < hd; ++d) {
                    const float kx = fabsf(pa_load(a->act_dtype, a->k_new, t * a->k_stride[0] + h * a->k_stride[1] + d * a->k_stride[2]));
                    const float vx = fabsf(pa_load(a->act_dtype, a->v_new, t * a->v_stride[0] + h * a->v_stride[1] + d * a->v_stride[2]));
                    if (kx > new_k[b * nh + h]) {
                        new_k[b * nh + h] = kx;
                    }
                    if (vx > new_v[b * nh + h]) {
                        new_v[b * nh + h] = vx;
                    }
                }
            }
        }
        uint8_t *caches[2] = {(uint8_t *)a->kv_k, (uint8_t *)a->kv_v};
        float *scales[2] = {a->kv_k_scale, a->kv_v_scale};
        float *news[2] = {new_k, new_v};
        for (size_t b = 0; b < nb; ++b) {
            if (min_off[b] == a->block_size) {
                continue;
            }
            const uint32_t existing = min_off[b];
            for (size_t h = 0; h < nh; ++h) {
                const size_t si = b * a->scale_stride[0] + (size_t)a->layer_idx * a->scale_stride[1] + h * a->scale_stride[2];
                for (int which = 0; which < 2; ++which) {
                    const float old_scale = scales[which][si];
                    float big = 0.0f;
                    if (existing > 0 && old_scale > 0.0f) {
                        for (uint32_t p = 0; p < existing; ++p) {
                            const size_t base = b * a->kv_stride[0] + (size_t)a->layer_idx * a->kv_stride[1] +
                                                h * a->kv_stride[2] + (size_t)p * a->kv_stride[3];
                            for (size_t d = 0; d < hd; ++d) {
                                const float x = fabsf(pa_fp8_dequant(caches[which][base + d * a->kv_stride[4]], old_scale));
                                if (x > big) {
                                    big = x;
                                }
                            }
                        }
                    }
                    if (news[which][b * nh + h] > big) {
                        big = news[which][b * nh + h];
                    }
                    const float new_scale = pa_fp8_scale(big);
                    if (existing > 0 && new_scale != old_scale) { /* re-encode what the block already holds */
                        for (uint32_t p = 0; p < existing; ++p) {
                            const size_t base = b * a->kv_stride[0] + (size_t)a->layer_idx * a->kv_stride[1] +
                                                h * a->kv_stride[2] + (size_t)p * a->kv_stride[3];
                            for (size_t d = 0; d < hd; ++d) {
                                uint8_t *c = &caches[which][base + d * a->kv_stride[4]];
                                *c = pa_fp8_quant(pa_fp8_dequant(*c, old_scale), new_scale);
                            }
                        }
                    }
                    scales[which][si] = new_scale;
                }
            }
        }
        for (size_t t = 0; t < a->token_count; ++t) { /* the new rows, encoded with their block's scale */
            const uint32_t kv_slot = a->token_meta[t * a->meta_stride[0] + 2 * a->meta_stride[1]];
            const size_t b = kv_slot >> shift;
            for (size_t h = 0; h < nh; ++h) {
                const size_t si = b * a->scale_stride[0] + (size_t)a->layer_idx * a->scale_stride[1] + h * a->scale_stride[2];
                const size_t base = b * a->kv_stride[0] + (size_t)a->layer_idx * a->kv_stride[1] + h * a->kv_stride[2] +
                                    (size_t)(kv_slot & mask) * a->kv_stride[3];
                for (size_t d = 0; d < hd; ++d) {
                    ((uint8_t *)a->kv_k)[base + d * a->kv_stride[4]] = pa_fp8_quant(
                        pa_load(a->act_dtype, a->k_new, t * a->k_stride[0] + h * a->k_stride[1] + d * a->k_stride[2]),
                        a->kv_k_scale[si]);
                    ((uint8_t *)a->kv_v)[base + d * a->kv_stride[4]] = pa_fp8_quant(
                        pa_load(a->act_dtype, a->v_new, t * a->v_stride[0] + h * a->v_stride[1] + d * a->v_stride[2]),
                        a->kv_v_scale[si]);
                }
            }
        }
        free(min_off), free(new_k), free(new_v);
    }
    /* the new rows go into the cache first (:346-373): same dtype = bit copy, otherwise through fp32 */
    for (size_t t = 0; !fp8 && t < a->token_count; ++t) {
        const uint32_t kv_slot = a->token_meta[t * a->meta_stride[0] + 2 * a->meta_stride[1]];
        const size_t base = (size_t)(kv_slot >> shift) * a->kv_stride[0] + (size_t)a->layer_idx * a->kv_stride[1] +
                            (size_t)(kv_slot & mask) * a->kv_stride[3];
        for (size_t h = 0; h < a->num_kv_heads; ++h) {
            for (size_t d = 0; d < hd; ++d) {
                const size_t dst = base + h * a->kv_stride[2] + d * a->kv_stride[4];
                const size_t ks = t * a->k_stride[0] + h * a->k_stride[1] + d * a->k_stride[2];
                const size_t vs = t * a->v_stride[0] + h * a->v_stride[1] + d * a->v_stride[2];
                if (a->act_dtype == a->kv_dtype && a->act_dtype != MO_DTYPE_F32) {
                    ((uint16_t *)a->kv_k)[dst] = ((const uint16_t *)a->k_new)[ks];
                    ((uint16_t *)a->kv_v)[dst] = ((const uint16_t *)a->v_new)[vs];
                } else {
                    pa_store(a->kv_dtype, a->kv_k, dst, pa_load(a->act_dtype, a->k_new, ks));
                    pa_store(a->kv_dtype, a->kv_v, dst, pa_load(a->act_dtype, a->v_new, vs));
                }
            }
        }
    }
    const size_t block_n = pa_block_n(hd);
    float *q_vec = (float *)malloc(hd * sizeof(float));
    float *out_vec = (float *)malloc(hd * sizeof(float));
    float *k_block = (float *)malloc(block_n * hd * sizeof(float));
    float *v_block = (float *)malloc(block_n * hd * sizeof(float));
    float *scores = (float *)malloc(block_n * sizeof(float));
    if (q_vec == NULL || out_vec == NULL || k_block == NULL || v_block == NULL || scores == NULL) {
        free(q_vec), free(out_vec), free(k_block), free(v_block), free(scores);
        return MO_ERR_INVALID_ARGUMENT;
    }
    const size_t group = a->num_q_heads / a->num_kv_heads;
    for (size_t t = 0; t < a->token_count; ++t) { /* cpu_paged_attention_attention_range, :398-569 */
        const uint32_t seq_slot = a->token_meta[t * a->meta_stride[0]];
        const uint32_t pos = a->token_meta[t * a->meta_stride[0] + a->meta_stride[1]];
        const uint32_t kv_len = pos + 1u;
        for (size_t qh = 0; qh < a->num_q_heads; ++qh) {
            const size_t kvh = qh / group;
            const size_t q_base = t * a->q_stride[0] + qh * a->q_stride[1];
            const size_t out_base = t * a->out_stride[0] + qh * a->out_stride[1];
            for (size_t d = 0; d < hd; ++d) {
                q_vec[d] = pa_load(a->act_dtype, a->q, q_base + d * a->q_stride[2]);
            }
            if (a->scale != 1.0f) {
                for (size_t d = 0; d < hd; ++d) {
                    q_vec[d] *= a->scale;
                }
            }
            memset(out_vec, 0, hd * sizeof(float));
            float max_score = -INFINITY, sum = 0.0f;
            int has_any = 0;
            for (uint32_t k_start = 0; k_start < kv_len; k_start += (uint32_t)block_n) {
                uint32_t k_limit = k_start + (uint32_t)block_n;
                if (k_limit > kv_len || k_limit < k_start) {
                    k_limit = kv_len;
                }
                size_t k_count = 0;
                for (uint32_t p = k_start; p < k_limit; ++p) {
                    const uint32_t logical = p >> shift;
                    if (logical >= a->max_blocks_per_seq) {
                        break;
                    }
                    const uint32_t tb = a->block_table[(size_t)seq_slot * a->table_stride[0] +
                                                       (size_t)logical * a->table_stride[1]];
                    if (tb == 0xFFFFFFFFu) {
                        continue;
                    }
                    const size_t base = (size_t)tb * a->kv_stride[0] + (size_t)a->layer_idx * a->kv_stride[1] +
                                        kvh * a->kv_stride[2] + (size_t)(p & mask) * a->kv_stride[3];
                    if (fp8) { /* :474-498: the block's scales */
                        const size_t si = (size_t)tb * a->scale_stride[0] + (size_t)a->layer_idx * a->scale_stride[1] +
                                          kvh * a->scale_stride[2];
                        for (size_t d = 0; d < hd; ++d) {
                            k_block[k_count * hd + d] =
                                pa_fp8_dequant(((const uint8_t *)a->kv_k)[base + d * a->kv_stride[4]], a->kv_k_scale[si]);
                            v_block[k_count * hd + d] =
                                pa_fp8_dequant(((const uint8_t *)a->kv_v)[base + d * a->kv_stride[4]], a->kv_v_scale[si]);
                        }
                        ++k_count;
                        continue;
                    }
                    for (size_t d = 0; d < hd; ++d) {
                        k_block[k_count * hd + d] = pa_load(a->kv_dtype, a->kv_k, base + d * a->kv_stride[4]);
                        v_block[k_count * hd + d] = pa_load(a->kv_dtype, a->kv_v, base + d * a->kv_stride[4]);
                    }
                    ++k_count;
                }
                if (k_count == 0) {
                    continue;
                }
                float row_max = -INFINITY;
                for (size_t kj = 0; kj < k_count; ++kj) { /* cpu_paged_attention_dot_f32_scalar */
                    float dot = 0.0f;
                    for (size_t d = 0; d < hd; ++d) {
                        dot += q_vec[d] * k_block[kj * hd + d];
                    }
                    scores[kj] = dot;
                    if (dot > row_max) {
                        row_max = dot;
                    }
                }
                const float next_max = max_score > row_max ? max_score : row_max;
                const float exp_prev = max_score == -INFINITY ? 0.0f : expf(max_score - next_max);
                if (exp_prev != 1.0f) {
                    for (size_t d = 0; d < hd; ++d) {
                        out_vec[d] *= exp_prev;
                    }
                }
                float block_sum = 0.0f; /* cpu_paged_attention_block_sum_f32_scalar */
                for (size_t kj = 0; kj < k_count; ++kj) {
                    const float weight = expf(scores[kj] - next_max);
                    block_sum += weight;
                    for (size_t d = 0; d < hd; ++d) {
                        out_vec[d] += weight * v_block[kj * hd + d];
                    }
                }
                sum = sum * exp_prev + block_sum;
                max_score = next_max;
                has_any = 1;
            }
            if (!has_any) {
                for (size_t d = 0; d < hd; ++d) {
                    pa_store(a->act_dtype, a->out, out_base + d * a->out_stride[2], 0.0f);
                }
                continue;
            }
            const float inv_sum = sum > 0.0f ? 1.0f / sum : 0.0f;
            for (size_t d = 0; d < hd; ++d) {
                pa_store(a->act_dtype, a->out, out_base + d * a->out_stride[2],
                         inv_sum != 1.0f ? out_vec[d] * inv_sum : out_vec[d]);
            }
        }
    }
    free(q_vec), free(out_vec), free(k_block), free(v_block), free(scores);
    return 0;
}

/* ------------------------------------------------------------------ tensor operations around the linears */

/* gelu_scalar, gelu_tanh_scalar, silu_scalar_fn (src/backends/cpu/ops/unary/scalar/unary_scalar.c:201-218); FLOAT16
 * values are widened, computed in fp32 and rounded back (CPU_UNARY_DEFINE_FLOAT_ACTIVATION, unary_scalar.c:360-385) */
static float unary_value(int op, float x) {
    switch (op) {
    case 0: {
        const float inv_sqrt2 = 0.7071067811865475f;
        return x * 0.5f * (1.0f + erff(x * inv_sqrt2));
    }
    case 1: {
        const float sqrt_2_over_pi = 0.7978845608028654f;
        const float coeff = 0.044715f;
        const float inner = sqrt_2_over_pi * (x + coeff * x * x * x);
        return 0.5f * x * (1.0f + tanhf(inner));
    }
    default:
        return x / (1.0f + expf(-x));
    }
}

int mo_unary(int op, const void *x, int dtype, size_t n, void *out) {
    if (op < 0 || op > 2 || (dtype != MO_DTYPE_F32 && dtype != MO_DTYPE_F16)) {
        return -1;
    }
    for (size_t i = 0; i < n; ++i) {
        if (dtype == MO_DTYPE_F32) {
            ((float *)out)[i] = unary_value(op, ((const float *)x)[i]);
        } else {
            ((uint16_t *)out)[i] = mo_f32_to_f16(unary_value(op, mo_f16_to_f32(((const uint16_t *)x)[i])));
        }
    }
    return 0;
}

/* softmax_f32_scalar (src/backends/cpu/ops/softmax/scalar/softmax_f32_scalar.c:30-83) over a contiguous tensor seen as
 * [outer, axis, inner] (marmot_softmax_prepare, src/core/helpers/norm.c:123-179); softmax_safe_expf flushes
 * differences at or below -88 to zero (softmax_internal.h:14-26) */
int mo_softmax(const float *x, size_t outer, size_t axis, size_t inner, float *out) {
    if (axis == 0) {
        return -1;
    }
    for (size_t row = 0; row < outer * inner; ++row) {
        const size_t o = row / inner, j = row % inner;
        const size_t base = o * axis * inner + j;
        float max_val = inner == 1 ? x[base] : -FLT_MAX;
        for (size_t a = 0; a < axis; ++a) {
            const float v = x[base + a * inner];
            if (v > max_val) {
                max_val = v;
            }
        }
        float sum = 0.0f;
        for (size_t a = 0; a < axis; ++a) {
            const float diff = x[base + a * inner] - max_val;
            const float e = diff <= -88.0f ? 0.0f : expf(diff);
            out[base + a * inner] = e;
            sum += e;
        }
        const float inv_sum = 1.0f / sum;
        for (size_t a = 0; a < axis; ++a) {
            out[base + a * inner] *= inv_sum;
        }
    }
    return 0;
}

/* cpu_convert_* between FLOAT32, FLOAT16 and BFLOAT16 (src/backends/cpu/ops/convert/dtype_convert.c:17-130): the vector
 * body's rounding (to nearest even) for every element; the 16-bit types convert to each other through FLOAT32
 * (src/utils/dtype_ref.c:86-114) */
static float conv_load(int dtype, const void *p, size_t i) {
    if (dtype == MO_DTYPE_F32) {
        return ((const float *)p)[i];
    }
    if (dtype == MO_DTYPE_F16) {
        return mo_f16_to_f32(((const uint16_t *)p)[i]);
    }
    uint32_t bits = (uint32_t)((const uint16_t *)p)[i] << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static void conv_store(int dtype, void *p, size_t i, float v) {
    if (dtype == MO_DTYPE_F32) {
        ((float *)p)[i] = v;
    } else if (dtype == MO_DTYPE_F16) {
        ((uint16_t *)p)[i] = mo_f32_to_f16(v);
    } else {
        uint32_t bits;
        memcpy(&bits, &v, 4);
        const uint32_t rounding_bias = 0x7FFFu + ((bits >> 16) & 1u);
        ((uint16_t *)p)[i] = (uint16_t)((bits + rounding_bias) >> 16);
    }
}

/* softmax_f16_scalar / softmax_bf16_scalar (src/backends/cpu/ops/softmax/scalar/softmax_misc_scalar.c:4-62, 64-122;
 * softmax_find_max_f16 and softmax_scale_f16, softmax_internal.h:119-215) over [outer, axis, inner] of a 16-bit type:
 * the maximum (from -FLT_MAX) and the sum of the exponentials are FLOAT32; every exponential is rounded to the tensor's
 * type when it is stored, and the stored value, widened again, is multiplied by 1 / sum and rounded a second time.
 * dtype FLOAT32 is mo_softmax. */
int mo_softmax_typed(int dtype, const void *x, size_t outer, size_t axis, size_t inner, void *out) {
    if (dtype == MO_DTYPE_F32) {
        return mo_softmax((const float *)x, outer, axis, inner, (float *)out);
    }
    if ((dtype != MO_DTYPE_F16 && dtype != MO_DTYPE_BF16) || axis == 0) {
        return -1;
    }
    for (size_t row = 0; row < outer * inner; ++row) {
        const size_t o = row / inner, j = row % inner;
        const size_t base = o * axis * inner + j;
        float max_val = -FLT_MAX;
        for (size_t a = 0; a < axis; ++a) {
            const float v = conv_load(dtype, x, base + a * inner);
            if (v > max_val) {
                max_val = v;
            }
        }
        float sum = 0.0f;
        for (size_t a = 0; a < axis; ++a) {
            const float diff = conv_load(dtype, x, base + a * inner) - max_val;
            const float e = diff <= -88.0f ? 0.0f : expf(diff);
            sum += e;
            conv_store(dtype, out, base + a * inner, e);
        }
        const float inv_sum = 1.0f / sum;
        for (size_t a = 0; a < axis; ++a) {
            conv_store(dtype, out, base + a * inner, conv_load(dtype, out, base + a * inner) * inv_sum);
        }
    }
    return 0;
}

int mo_convert(void *dst, int dst_dtype, const void *src, int src_dtype, size_t n) {
    const int ok_s = src_dtype == MO_DTYPE_F32 || src_dtype == MO_DTYPE_F16 || src_dtype == MO_DTYPE_BF16;
    const int ok_d = dst_dtype == MO_DTYPE_F32 || dst_dtype == MO_DTYPE_F16 || dst_dtype == MO_DTYPE_BF16;
    if (!ok_s || !ok_d) {
        return -1;
    }
    if (src_dtype == dst_dtype) { /* equal types: a copy */
        memcpy(dst, src, n * (src_dtype == MO_DTYPE_F32 ? 4 : 2));
        return 0;
    }
    for (size_t i = 0; i < n; ++i) {
        conv_store(dst_dtype, dst, i, conv_load(src_dtype, src, i));
    }
    return 0;
}

/* cpu_gather_rows (src/backends/cpu/ops/tensor_ops/tensor_ops.c:464-547), rows with unit column stride: strides in
 * elements; returns -1 and the offending output row for an index outside [0, rows_in) */
int mo_gather_rows(const void *x, size_t rows_in, size_t cols, size_t elem_size, size_t in_stride0, const void *idx,
                   int idx_is_signed, size_t idx_stride, size_t rows_out, void *out, size_t out_stride0,
                   size_t *bad_row) {
    for (size_t r = 0; r < rows_out; ++r) {
        int64_t row_idx;
        if (idx_is_signed) {
            row_idx = ((const int32_t *)idx)[r * idx_stride];
        } else {
            row_idx = (int64_t)((const uint32_t *)idx)[r * idx_stride];
        }
        if (row_idx < 0 || (size_t)row_idx >= rows_in) {
            if (bad_row != NULL) {
                *bad_row = r;
            }
            return -1;
        }
        memcpy((uint8_t *)out + r * out_stride0 * elem_size, (const uint8_t *)x + (size_t)row_idx * in_stride0 * elem_size,
               cols * elem_size);
    }
    return 0;
}

/* cpu_slice (tensor_ops.c:401-462): contiguous input of shape in_shape, contiguous output of shape out_shape, a run of
 * sizes[ndim - 1] elements copied per position of the leading dimensions */
int mo_slice(const void *x, void *out, size_t elem_size, size_t ndim, const size_t *in_shape, const size_t *out_shape,
             const size_t *starts, const size_t *sizes) {
    if (ndim == 0) {
        return 0;
    }
    if (ndim > 8) {
        return -1;
    }
    size_t src_strides[8], dst_strides[8], counters[8] = {0};
    src_strides[ndim - 1] = 1;
    dst_strides[ndim - 1] = 1;
    for (int i = (int)ndim - 2; i >= 0; --i) {
        src_strides[i] = src_strides[i + 1] * in_shape[i + 1];
        dst_strides[i] = dst_strides[i + 1] * out_shape[i + 1];
    }
    const size_t copy_block = sizes[ndim - 1] * elem_size;
    const size_t loops = ndim > 1 ? ndim - 1 : 0;
    for (size_t d = 0; d < ndim; ++d) {
        if (sizes[d] == 0) {
            return 0;
        }
    }
    for (;;) {
        size_t src_index = starts[ndim - 1] * src_strides[ndim - 1];
        size_t dst_index = 0;
        for (size_t d = 0; d < loops; ++d) {
            src_index += (starts[d] + counters[d]) * src_strides[d];
            dst_index += counters[d] * dst_strides[d];
        }
        memcpy((uint8_t *)out + dst_index * elem_size, (const uint8_t *)x + src_index * elem_size, copy_block);
        if (loops == 0) {
            break;
        }
        int dim = (int)loops - 1;
        while (dim >= 0) {
            counters[dim]++;
            if (counters[dim] < sizes[dim]) {
                break;
            }
            counters[dim] = 0;
            dim--;
        }
        if (dim < 0) {
            break;
        }
    }
    return 0;
}

// Paged attention (marmot_paged_attention; CPU counterpart cpu_paged_attention_impl,
// src/backends/cpu/ops/paged_attention/paged_attention_ref.c:573-1082): every token's new key / value rows are written
// into the paged cache at the token's kv_slot, then every (token, query head) attends over positions 0 .. pos of its
// sequence through the block table.
//
// Attention kernel: one workgroup of 16 groups of 16 lanes per (token, up to four query heads of one key / value
// head). A group walks the positions g, g + 16, g + 32, ...: its 16 lanes split the head dimension (a lane holds EPL consecutive values of the
// query, of the running output and of each key / value row, so a row is read as one contiguous run by the group), the
// dot product is reduced inside the group with data-parallel-primitive moves, and the group keeps its own running
// maximum, sum and output (online softmax). The groups meet in LDS at the end. All arithmetic is fp32 like the
// reference's; only the order of the sums differs (per group instead of per block of positions). Rows are read with
// 16-byte loads when the head dimension is exactly 16 x EPL values with unit stride, element by element otherwise.
// A token whose sequence slot or cache block is out of range is skipped (the host rejects such calls when it may read
// the metadata, like the reference).
#include "mh_common.h"

#include <math.h>

namespace mh {

constexpr uint32_t PA_NO_BLOCK = 0xFFFFFFFFu;

struct PaParams {
    uint32_t token_count, layer_idx, num_q_heads, num_kv_heads, head_dim, block_size;
    float scale;
    int act_dtype, kv_dtype;
    const uint32_t *meta;
    size_t meta_stride[2];
    const void *q, *k_new, *v_new;
    size_t q_stride[3], k_stride[3], v_stride[3];
    void *kv_k, *kv_v;
    size_t kv_stride[5];
    size_t kv_blocks, kv_layers;
    const uint32_t *table;
    size_t table_stride[2];
    size_t max_seqs, max_blocks;
    void *out;
    size_t out_stride[3];
    uint32_t shift, mask, group;
    int q_vec, kv_vec;  // 16-byte loads of the query / of the cache rows
    int *flag;          // metadata check: 1 + index of an offending token (maximum)
    float *k_scale, *v_scale;  // FLOAT8_E4M3 cache: scales [blocks][layers][kv heads] at scale_stride
    size_t scale_stride[3];
    uint32_t *new_kmax, *new_vmax;  // scratch [blocks][kv heads]: largest new magnitudes as float bits
    uint32_t *min_off;              // scratch [blocks]: first offset this call writes (block_size = untouched)
    uint32_t *claim;                // scratch [blocks][kv heads]: the token whose workgroup rescales the block (~0 = none yet)
    uint32_t splits;    // workgroups along the history of one (token, heads) pair
    float *partial;     // splits > 1: [token][query head][split][2 + head_dim]: maximum, sum, unnormalized output
};

// marmot_f32_to_bf16_ref / marmot_bf16_to_f32_ref (src/utils/dtype_ref.c:86-104): round to nearest even on the bits
__device__ __forceinline__ uint16_t pa_f2bf(float v) {
    const uint32_t bits = __float_as_uint(v);
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float pa_bf2f(uint16_t h) {
    return __uint_as_float((uint32_t)h << 16);
}

// The reference's e4m3 (marmot_fp8_dequantize / marmot_fp8_quantize with 4 exponent bits, 3 mantissa bits, bias 7,
// no infinity, largest finite value 240: src/utils/dtype_ref.c:118-212).
__device__ __forceinline__ float pa_fp8_to_f32(uint32_t c) {
    const uint32_t field = (c >> 3) & 15u, mant = c & 7u, sign = (c & 0x80u) << 24;
    if (field == 15u) {
        return __uint_as_float(0x7fc00000u);
    }
    if (field == 0u) {
        return __uint_as_float(__float_as_uint((float)mant * 0.001953125f) | sign);  // mant / 8 * 2^-6
    }
    return __uint_as_float(sign | ((field + 120u) << 23) | (mant << 20));  // (1 + mant / 8) * 2^(field - 7)
}

__device__ __forceinline__ uint32_t pa_f32_to_fp8(float value) {
    if (value != value) {
        return 0x79u;
    }
    const uint32_t sign = value < 0.0f ? 0x80u : 0u;
    const float mag = fabsf(value);
    if (mag > 240.0f) {  // infinity included
        return sign | 0x77u;
    }
    if (mag == 0.0f) {
        return sign;
    }
    int e;
    float m = frexpf(mag, &e);  // mag = m * 2^e, m in [0.5, 1)
    m *= 2.0f;
    e -= 1;
    int field = e + 7;
    if (field > 0 && field < 15) {
        int r = (int)rintf((m - 1.0f) * 8.0f);  // nearest, ties to even
        if (r == 8) {
            r = 0;
            field += 1;
            if (field >= 15) {
                return sign | 0x77u;
            }
        }
        return sign | ((uint32_t)field << 3) | (uint32_t)(r & 7);
    }
    int r = (int)rintf(ldexpf(mag, 9));  // below the smallest normal 2^-6: multiples of 2^-9, never rounded up into
    if (r == 0) {                        // the normal range
        return sign;
    }
    return sign | (uint32_t)(r > 7 ? 7 : r);
}

// cpu_paged_attention_fp8_quant / _dequant / _scale_from_max (paged_attention_ref.c:142-163)
__device__ __forceinline__ uint32_t pa_fp8_quant(float value, float scale) {
    return scale > 0.0f ? pa_f32_to_fp8(value / scale) : 0u;
}
__device__ __forceinline__ float pa_fp8_dequant(uint32_t c, float scale) {
    return scale > 0.0f ? pa_fp8_to_f32(c) * scale : 0.0f;
}

__device__ __forceinline__ float pa_load(const void *data, int dtype, size_t i) {
    if (dtype == MARMOT_HIP_DTYPE_F8_E4M3) {  // the code's value; the caller applies the block's scale
        return pa_fp8_to_f32(((const uint8_t *)data)[i]);
    }
    if (dtype == MARMOT_HIP_DTYPE_F16) {
        return h2f(((const uint16_t *)data)[i]);
    }
    if (dtype == MARMOT_HIP_DTYPE_BF16) {
        return pa_bf2f(((const uint16_t *)data)[i]);
    }
    return ((const float *)data)[i];
}

__device__ __forceinline__ void pa_store(void *data, int dtype, size_t i, float v) {
    if (dtype == MARMOT_HIP_DTYPE_F16) {
        ((uint16_t *)data)[i] = f2h(v);
    } else if (dtype == MARMOT_HIP_DTYPE_BF16) {
        ((uint16_t *)data)[i] = pa_f2bf(v);
    } else {
        ((float *)data)[i] = v;
    }
}

// exp(x) for x <= 0 (softmax weights and rescaling factors): the hardware's base-2 exponential, about 2 units in the
// last place -- far inside the tolerance of the output, and a fraction of the library routine's instructions
__device__ __forceinline__ float pa_exp(float x) {
    return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f);
}

// EPL consecutive values starting at element `first` (unit stride, 16-byte aligned start for the storage type)
template <int EPL>
__device__ __forceinline__ void pa_load_run(const void *data, int dtype, size_t first, float (&v)[EPL]) {
    if (dtype == MARMOT_HIP_DTYPE_F8_E4M3) {
        uint32_t w[EPL / 4];
        if constexpr (EPL == 4) {
            w[0] = *(const uint32_t *)((const uint8_t *)data + first);
        } else if constexpr (EPL == 8) {
            const uint2 u = *(const uint2 *)((const uint8_t *)data + first);
            w[0] = u.x, w[1] = u.y;
        } else {
            const uint4 u = *(const uint4 *)((const uint8_t *)data + first);
            w[0] = u.x, w[1] = u.y, w[2] = u.z, w[3] = u.w;
        }
        // Codes whose exponent field is below 15 mean the same in this format and in the hardware's e4m3 (bias 7,
        // same subnormals), which converts two bytes per instruction; a word that holds a field of 15 (this format's
        // NaN) takes the bit-level decoder.
        typedef float pa_f2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int i = 0; i < EPL / 4; ++i) {
            if (((((w[i] & 0x78787878u) + 0x08080808u) & 0x80808080u)) == 0u) {
                const pa_f2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
                const pa_f2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
                v[4 * i] = lo.x, v[4 * i + 1] = lo.y, v[4 * i + 2] = hi.x, v[4 * i + 3] = hi.y;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[4 * i + e] = pa_fp8_to_f32((w[i] >> (8 * e)) & 0xffu);
                }
            }
        }
    } else if (dtype == MARMOT_HIP_DTYPE_F32) {
#pragma unroll
        for (int e = 0; e < EPL; e += 4) {
            const float4 f = *(const float4 *)((const float *)data + first + e);
            v[e] = f.x, v[e + 1] = f.y, v[e + 2] = f.z, v[e + 3] = f.w;
        }
    } else {
        uint32_t w[EPL / 2];
        if constexpr (EPL == 4) {
            const uint2 u = *(const uint2 *)((const uint16_t *)data + first);
            w[0] = u.x, w[1] = u.y;
        } else {
#pragma unroll
            for (int e = 0; e < EPL / 2; e += 4) {
                const uint4 u = *(const uint4 *)((const uint16_t *)data + first + 2 * e);
                w[e] = u.x, w[e + 1] = u.y, w[e + 2] = u.z, w[e + 3] = u.w;
            }
        }
#pragma unroll
        for (int e = 0; e < EPL / 2; ++e) {
            if (dtype == MARMOT_HIP_DTYPE_F16) {
                v[2 * e] = h2f((uint16_t)(w[e] & 0xffffu));
                v[2 * e + 1] = h2f((uint16_t)(w[e] >> 16));
            } else {
                v[2 * e] = __uint_as_float(w[e] << 16);
                v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
            }
        }
    }
}

// ---- metadata check (paged_attention_ref.c:809-823): sequence slots inside the block table, kv slots inside the cache
__global__ __launch_bounds__(256) void k_pa_check(const PaParams p) {
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= p.token_count) {
        return;
    }
    const uint32_t seq = p.meta[t * p.meta_stride[0]];
    const uint32_t slot = p.meta[t * p.meta_stride[0] + 2 * p.meta_stride[1]];
    if (seq >= p.max_seqs || (slot >> p.shift) >= p.kv_blocks) {
        atomicMax(p.flag, (int)(p.token_count - t));  // the maximum names the first offender
    }
}

// ---- cache write (cpu_paged_attention_kv_write_range, :346-373): one workgroup per (token, kv head)
__global__ __launch_bounds__(128) void k_pa_write(const PaParams p) {
    const uint32_t t = blockIdx.x, h = blockIdx.y;
    const uint32_t slot = p.meta[t * p.meta_stride[0] + 2 * p.meta_stride[1]];
    const uint32_t block = slot >> p.shift;
    if (block >= p.kv_blocks) {
        return;
    }
    const size_t dst0 = (size_t)block * p.kv_stride[0] + (size_t)p.layer_idx * p.kv_stride[1] + (size_t)h * p.kv_stride[2] +
                        (size_t)(slot & p.mask) * p.kv_stride[3];
    const size_t k0 = (size_t)t * p.k_stride[0] + (size_t)h * p.k_stride[1];
    const size_t v0 = (size_t)t * p.v_stride[0] + (size_t)h * p.v_stride[1];
    const bool bits16 = p.act_dtype == p.kv_dtype && p.act_dtype != MARMOT_HIP_DTYPE_F32;
    for (uint32_t d = threadIdx.x; d < p.head_dim; d += blockDim.x) {
        const size_t dst = dst0 + d * p.kv_stride[4];
        if (bits16) {  // same 16-bit storage type: the bits travel unchanged
            ((uint16_t *)p.kv_k)[dst] = ((const uint16_t *)p.k_new)[k0 + d * p.k_stride[2]];
            ((uint16_t *)p.kv_v)[dst] = ((const uint16_t *)p.v_new)[v0 + d * p.v_stride[2]];
        } else {
            pa_store(p.kv_k, p.kv_dtype, dst, pa_load(p.k_new, p.act_dtype, k0 + d * p.k_stride[2]));
            pa_store(p.kv_v, p.kv_dtype, dst, pa_load(p.v_new, p.act_dtype, v0 + d * p.v_stride[2]));
        }
    }
}

// ---- the FLOAT8_E4M3 cache write (paged_attention_ref.c:825-989) in four launches
// 1. scratch: no new magnitudes, no block touched
__global__ __launch_bounds__(256) void k_pa_fp8_init(const PaParams p) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < p.kv_blocks * p.num_kv_heads) {
        p.new_kmax[i] = 0u;
        p.new_vmax[i] = 0u;
        p.claim[i] = 0xffffffffu;
    }
    if (i < p.kv_blocks) {
        p.min_off[i] = p.block_size;
    }
}

__device__ __forceinline__ float pa_block_max(float v, float *red) {  // maximum over a workgroup of 128 threads
    red[threadIdx.x] = v;
    __syncthreads();
    for (int s = 64; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
        }
        __syncthreads();
    }
    const float r = red[0];
    __syncthreads();
    return r;
}

// 2. per (token, kv head): the largest magnitudes of the new key and value rows into their block's entry (non-negative
//    floats order like their bits), and the first offset written in the block
__global__ __launch_bounds__(128) void k_pa_fp8_scan_new(const PaParams p) {
    __shared__ float red[128];
    const uint32_t t = blockIdx.x, h = blockIdx.y;
    const uint32_t slot = p.meta[t * p.meta_stride[0] + 2 * p.meta_stride[1]];
    const uint32_t block = slot >> p.shift;
    if (block >= p.kv_blocks) {
        return;
    }
    float km = 0.0f, vm = 0.0f;
    for (uint32_t d = threadIdx.x; d < p.head_dim; d += 128u) {
        km = fmaxf(km, fabsf(pa_load(p.k_new, p.act_dtype, (size_t)t * p.k_stride[0] + (size_t)h * p.k_stride[1] + d * p.k_stride[2])));
        vm = fmaxf(vm, fabsf(pa_load(p.v_new, p.act_dtype, (size_t)t * p.v_stride[0] + (size_t)h * p.v_stride[1] + d * p.v_stride[2])));
    }
    km = pa_block_max(km, red);
    vm = pa_block_max(vm, red);
    if (threadIdx.x == 0) {
        atomicMax(p.new_kmax + (size_t)block * p.num_kv_heads + h, __float_as_uint(km));
        atomicMax(p.new_vmax + (size_t)block * p.num_kv_heads + h, __float_as_uint(vm));
        if (h == 0) {
            atomicMin(p.min_off + block, slot & p.mask);
        }
    }
}

// Maxima of four values over a workgroup of 128 threads (two wavefronts): lanes first, then the two wavefronts
// through LDS. `red` holds 8 floats and is free again on return.
__device__ __forceinline__ void pa_block_max4(float (&v)[4], float *red) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = fmaxf(v[i], __shfl_xor(v[i], s));
        }
    }
    if ((threadIdx.x & 63u) == 0u) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            red[(threadIdx.x >> 6) * 4 + i] = v[i];
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = fmaxf(red[i], red[4 + i]);
    }
    __syncthreads();
}

// The rows already in one (block, kv head): the first `existing` positions. `vec`: rows of a multiple of 16 codes at
// 16-byte aligned addresses, taken 16 codes at a time.
struct PaFp8Rows {
    uint8_t *kc, *vc;
    size_t si;
    uint32_t existing;
    bool vec;
};

__device__ __forceinline__ PaFp8Rows pa_fp8_rows(const PaParams &p, uint32_t b, uint32_t h, uint32_t existing) {
    PaFp8Rows r;
    const size_t base = (size_t)b * p.kv_stride[0] + (size_t)p.layer_idx * p.kv_stride[1] + (size_t)h * p.kv_stride[2];
    r.kc = (uint8_t *)p.kv_k + base, r.vc = (uint8_t *)p.kv_v + base;
    r.si = (size_t)b * p.scale_stride[0] + (size_t)p.layer_idx * p.scale_stride[1] + (size_t)h * p.scale_stride[2];
    r.existing = existing;
    r.vec = p.kv_stride[4] == 1 && (p.head_dim & 15u) == 0u && (p.kv_stride[3] & 15u) == 0u &&
            (((uintptr_t)r.kc | (uintptr_t)r.vc) & 15u) == 0u;
    return r;
}

__device__ __forceinline__ uint32_t pa_fp8_big_field(uint32_t big, uint32_t word) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t c = (word >> (8 * e)) & 0x7fu;
        big = c < 0x78u && c > big ? c : big;
    }
    return big;
}

// This thread's share of the largest finite magnitude fields (low seven bits) among the rows already there: a finite
// code's magnitude grows with that field, so the largest one is found first and decoded once (NaN codes, field 15
// of the exponent, never win a maximum).
__device__ __forceinline__ void pa_fp8_scan_rows(const PaParams &p, const PaFp8Rows &r, uint32_t &kbig, uint32_t &vbig) {
    kbig = vbig = 0u;
    if (r.vec) {
        const uint32_t per_row = p.head_dim >> 4, chunks = r.existing * per_row;
        for (uint32_t c = threadIdx.x; c < chunks; c += 128u) {
            const uint32_t pos = c / per_row;
            const size_t at = (size_t)pos * p.kv_stride[3] + (size_t)(c - pos * per_row) * 16u;
            const uint4 k = *(const uint4 *)(r.kc + at), v = *(const uint4 *)(r.vc + at);
            kbig = pa_fp8_big_field(pa_fp8_big_field(pa_fp8_big_field(pa_fp8_big_field(kbig, k.x), k.y), k.z), k.w);
            vbig = pa_fp8_big_field(pa_fp8_big_field(pa_fp8_big_field(pa_fp8_big_field(vbig, v.x), v.y), v.z), v.w);
        }
        return;
    }
    const uint32_t cells = r.existing * p.head_dim;
    for (uint32_t c = threadIdx.x; c < cells; c += 128u) {
        const uint32_t pos = c / p.head_dim, d = c - pos * p.head_dim;
        const size_t at = (size_t)pos * p.kv_stride[3] + (size_t)d * p.kv_stride[4];
        const uint32_t kb = r.kc[at] & 0x7fu, vb = r.vc[at] & 0x7fu;
        kbig = kb < 0x78u && kb > kbig ? kb : kbig;
        vbig = vb < 0x78u && vb > vbig ? vb : vbig;
    }
}

__device__ __forceinline__ uint32_t pa_fp8_recode4(uint32_t word, float old_scale, float new_scale) {
    uint32_t out = 0u;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        out |= pa_fp8_quant(pa_fp8_dequant((word >> (8 * e)) & 0xffu, old_scale), new_scale) << (8 * e);
    }
    return out;
}

// The new scale of one cache tensor of the block from the largest magnitude field found in it and the largest new
// magnitude; the rows already there are re-encoded when the scale changes. `old_scale` was read before any thread
// could have written the new one (a barrier lies between).
__device__ __forceinline__ float pa_fp8_rescale_rows(const PaParams &p, const PaFp8Rows &r, int which, uint32_t big_field,
                                                     float new_max, float old_scale) {
    uint8_t *cache = which ? r.vc : r.kc;
    const float big = fmaxf(pa_fp8_dequant(big_field, old_scale), new_max);
    const float new_scale = big > 0.0f ? big / 240.0f : 1.0f;
    if (r.existing > 0 && new_scale != old_scale) {
        if (r.vec) {
            const uint32_t per_row = p.head_dim >> 4, chunks = r.existing * per_row;
            for (uint32_t c = threadIdx.x; c < chunks; c += 128u) {
                const uint32_t pos = c / per_row;
                uint4 *cell = (uint4 *)(cache + (size_t)pos * p.kv_stride[3] + (size_t)(c - pos * per_row) * 16u);
                uint4 w = *cell;
                w.x = pa_fp8_recode4(w.x, old_scale, new_scale), w.y = pa_fp8_recode4(w.y, old_scale, new_scale);
                w.z = pa_fp8_recode4(w.z, old_scale, new_scale), w.w = pa_fp8_recode4(w.w, old_scale, new_scale);
                *cell = w;
            }
        } else {
            const uint32_t cells = r.existing * p.head_dim;
            for (uint32_t c = threadIdx.x; c < cells; c += 128u) {
                const uint32_t pos = c / p.head_dim, d = c - pos * p.head_dim;
                uint8_t *cell = cache + (size_t)pos * p.kv_stride[3] + (size_t)d * p.kv_stride[4];
                *cell = (uint8_t)pa_fp8_quant(pa_fp8_dequant(*cell, old_scale), new_scale);
            }
        }
    }
    if (threadIdx.x == 0) {
        (which ? p.v_scale : p.k_scale)[r.si] = new_scale;
    }
    return new_scale;
}

// The work on one (block, kv head): the new scales from the rows already there (the first `existing` positions) and
// this thread's share of the largest new magnitudes; the rows already there are re-encoded where a scale changes.
// Whole workgroup of 128.
__device__ __forceinline__ void pa_fp8_rescale_block(const PaParams &p, uint32_t b, uint32_t h, uint32_t existing,
                                                     float new_km, float new_vm, float *red, float *new_scales) {
    const PaFp8Rows r = pa_fp8_rows(p, b, h, existing);
    const float old_k = p.k_scale[r.si], old_v = p.v_scale[r.si];
    uint32_t kbig, vbig;
    pa_fp8_scan_rows(p, r, kbig, vbig);
    float m[4] = {new_km, new_vm, (float)kbig, (float)vbig};
    pa_block_max4(m, red);
    new_scales[0] = pa_fp8_rescale_rows(p, r, 0, (uint32_t)m[2], m[0], old_k);
    new_scales[1] = pa_fp8_rescale_rows(p, r, 1, (uint32_t)m[3], m[1], old_v);
}

// 3. per (touched block, kv head): the new scale; rows already in the block are re-encoded when it changes. A token
//    that writes the block's first new row does the block's work, so the launch grows with the call, not the cache;
//    when several tokens of a call carry that offset (the same kv_slot twice), the first workgroup to claim the block
//    does it alone: two of them would read each other's new scale as the old one and encode the rows twice. The
//    reference touches each block once, whatever duplicates a call holds (paged_attention_ref.c:866-946).
__global__ __launch_bounds__(128) void k_pa_fp8_rescale(const PaParams p) {
    __shared__ float red[128];
    const uint32_t t = blockIdx.x, h = blockIdx.y;
    const uint32_t slot = p.meta[t * p.meta_stride[0] + 2 * p.meta_stride[1]];
    const uint32_t b = slot >> p.shift;
    if (b >= p.kv_blocks) {
        return;
    }
    const uint32_t existing = p.min_off[b];
    if ((slot & p.mask) != existing) {
        return;
    }
    if (threadIdx.x == 0) {
        red[0] = __uint_as_float(atomicCAS(p.claim + (size_t)b * p.num_kv_heads + h, 0xffffffffu, t));
    }
    __syncthreads();
    const bool mine = __float_as_uint(red[0]) == 0xffffffffu;
    __syncthreads();
    if (!mine) {
        return;
    }
    float scales[2];
    pa_fp8_rescale_block(p, b, h, existing, __uint_as_float(p.new_kmax[(size_t)b * p.num_kv_heads + h]),
                         __uint_as_float(p.new_vmax[(size_t)b * p.num_kv_heads + h]), red, scales);
}

// 4. per (token, kv head): the new rows, encoded with their block's scale
__global__ __launch_bounds__(128) void k_pa_fp8_store(const PaParams p) {
    const uint32_t t = blockIdx.x, h = blockIdx.y;
    const uint32_t slot = p.meta[t * p.meta_stride[0] + 2 * p.meta_stride[1]];
    const uint32_t block = slot >> p.shift;
    if (block >= p.kv_blocks) {
        return;
    }
    const size_t si = (size_t)block * p.scale_stride[0] + (size_t)p.layer_idx * p.scale_stride[1] + (size_t)h * p.scale_stride[2];
    const float ks = p.k_scale[si], vs = p.v_scale[si];
    const size_t dst0 = (size_t)block * p.kv_stride[0] + (size_t)p.layer_idx * p.kv_stride[1] + (size_t)h * p.kv_stride[2] +
                        (size_t)(slot & p.mask) * p.kv_stride[3];
    for (uint32_t d = threadIdx.x; d < p.head_dim; d += 128u) {
        const float kx = pa_load(p.k_new, p.act_dtype, (size_t)t * p.k_stride[0] + (size_t)h * p.k_stride[1] + d * p.k_stride[2]);
        const float vx = pa_load(p.v_new, p.act_dtype, (size_t)t * p.v_stride[0] + (size_t)h * p.v_stride[1] + d * p.v_stride[2]);
        ((uint8_t *)p.kv_k)[dst0 + d * p.kv_stride[4]] = (uint8_t)pa_fp8_quant(kx, ks);
        ((uint8_t *)p.kv_v)[dst0 + d * p.kv_stride[4]] = (uint8_t)pa_fp8_quant(vx, vs);
    }
}

// The same update in one launch, for calls of at most PA_FP8_ONE_TOKENS tokens. Every (token, kv head) workgroup finds
// the tokens of the call that write its block; the workgroup of the first of them does the block's work alone (largest
// new magnitudes, new scales, re-encoding, then the new rows in token order, so of two tokens with one kv_slot the
// later one stays, as in the reference's token loop) and the others leave. No scratch memory, no order between
// workgroups: each (block, kv head) is touched by exactly one.
constexpr uint32_t PA_FP8_ONE_TOKENS = 1024;
__global__ __launch_bounds__(128) void k_pa_fp8_update(const PaParams p) {
    __shared__ float red[128];
    __shared__ uint32_t members[PA_FP8_ONE_TOKENS / 32];
    __shared__ uint32_t first_off;
    const uint32_t t = blockIdx.x, h = blockIdx.y;
    const uint32_t b = p.meta[t * p.meta_stride[0] + 2 * p.meta_stride[1]] >> p.shift;
    if (b >= p.kv_blocks) {
        return;
    }
    if (threadIdx.x < PA_FP8_ONE_TOKENS / 32) {
        members[threadIdx.x] = 0u;
    }
    if (threadIdx.x == 0) {
        first_off = p.block_size;
    }
    __syncthreads();
    for (uint32_t u = threadIdx.x; u < p.token_count; u += 128u) {
        const uint32_t slot = p.meta[u * p.meta_stride[0] + 2 * p.meta_stride[1]];
        if ((slot >> p.shift) == b) {
            atomicOr(members + (u >> 5), 1u << (u & 31u));
            atomicMin(&first_off, slot & p.mask);
        }
    }
    __syncthreads();
    bool first = (members[t >> 5] & ((1u << (t & 31u)) - 1u)) == 0u;
    for (uint32_t w = 0; w < (t >> 5); ++w) {
        first = first && members[w] == 0u;
    }
    if (!first) {
        return;
    }
    const uint32_t words = (p.token_count + 31u) >> 5;
    float km = 0.0f, vm = 0.0f;
    for (uint32_t w = t >> 5; w < words; ++w) {
        for (uint32_t bits = members[w]; bits != 0u; bits &= bits - 1u) {
            const uint32_t u = w * 32u + (uint32_t)__ffs(bits) - 1u;
            for (uint32_t d = threadIdx.x; d < p.head_dim; d += 128u) {
                km = fmaxf(km, fabsf(pa_load(p.k_new, p.act_dtype, (size_t)u * p.k_stride[0] + (size_t)h * p.k_stride[1] + d * p.k_stride[2])));
                vm = fmaxf(vm, fabsf(pa_load(p.v_new, p.act_dtype, (size_t)u * p.v_stride[0] + (size_t)h * p.v_stride[1] + d * p.v_stride[2])));
            }
        }
    }
    float scales[2];
    pa_fp8_rescale_block(p, b, h, first_off, km, vm, red, scales);
    const size_t dst0 = (size_t)b * p.kv_stride[0] + (size_t)p.layer_idx * p.kv_stride[1] + (size_t)h * p.kv_stride[2];
    for (uint32_t w = t >> 5; w < words; ++w) {
        for (uint32_t bits = members[w]; bits != 0u; bits &= bits - 1u) {
            const uint32_t u = w * 32u + (uint32_t)__ffs(bits) - 1u;
            const uint32_t slot = p.meta[u * p.meta_stride[0] + 2 * p.meta_stride[1]];
            const size_t dst = dst0 + (size_t)(slot & p.mask) * p.kv_stride[3];
            for (uint32_t d = threadIdx.x; d < p.head_dim; d += 128u) {
                const float kx = pa_load(p.k_new, p.act_dtype, (size_t)u * p.k_stride[0] + (size_t)h * p.k_stride[1] + d * p.k_stride[2]);
                const float vx = pa_load(p.v_new, p.act_dtype, (size_t)u * p.v_stride[0] + (size_t)h * p.v_stride[1] + d * p.v_stride[2]);
                ((uint8_t *)p.kv_k)[dst + d * p.kv_stride[4]] = (uint8_t)pa_fp8_quant(kx, scales[0]);
                ((uint8_t *)p.kv_v)[dst + d * p.kv_stride[4]] = (uint8_t)pa_fp8_quant(vx, scales[1]);
            }
        }
    }
}

// ---- attention (cpu_paged_attention_attention_range, :398-569)
// One workgroup of 16 groups of 16 lanes per (token, QH query heads that share a key / value head): every key and
// value row is fetched, converted and located once for the QH heads. A group takes two positions per step and
// requests both before it works on either.
constexpr int PA_GROUPS = 16;

template <int EPL, int QH>
__global__ __launch_bounds__(16 * PA_GROUPS) void k_pa_attend(const PaParams p) {
    warm_kernel_arguments<sizeof(PaParams), sizeof(PaParams)>();
    __shared__ float s_acc[PA_GROUPS][QH][16 * EPL];
    __shared__ float s_m[PA_GROUPS][QH], s_l[PA_GROUPS][QH];
    const uint32_t t = blockIdx.x;
    const uint32_t qh0 = blockIdx.y * QH;  // first query head of this workgroup; QH divides the heads per kv head
    const int tid = threadIdx.x, g = tid >> 4, l = tid & 15;
    const uint32_t seq = p.meta[t * p.meta_stride[0]];
    const uint32_t pos = p.meta[t * p.meta_stride[0] + p.meta_stride[1]];
    const uint32_t kv_len = seq < p.max_seqs ? pos + 1u : 0u;
    const uint32_t kvh = qh0 / p.group;
    const uint32_t d0 = (uint32_t)l * EPL;  // this lane's first value of the head dimension

    float qv[QH][EPL];
#pragma unroll
    for (int h = 0; h < QH; ++h) {
        const size_t q_base = (size_t)t * p.q_stride[0] + (size_t)(qh0 + h) * p.q_stride[1];
        if (p.q_vec) {
            pa_load_run<EPL>(p.q, p.act_dtype, q_base + d0, qv[h]);
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                qv[h][e] = d0 + e < p.head_dim ? pa_load(p.q, p.act_dtype, q_base + (size_t)(d0 + e) * p.q_stride[2]) : 0.0f;
            }
        }
        if (p.scale != 1.0f) {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                qv[h][e] *= p.scale;
            }
        }
    }

    float m[QH], lsum[QH], acc[QH][EPL];
#pragma unroll
    for (int h = 0; h < QH; ++h) {
        m[h] = -INFINITY;
        lsum[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            acc[h][e] = 0.0f;
        }
    }
    const size_t head_base = (size_t)p.layer_idx * p.kv_stride[1] + (size_t)kvh * p.kv_stride[2];
    const uint32_t *table_row = p.table + (size_t)seq * p.table_stride[0];
    // the cache row of position pp, or false when the position has no block (beyond the table, or a hole)
    const bool fp8 = p.kv_dtype == MARMOT_HIP_DTYPE_F8_E4M3;
    auto locate = [&](uint32_t pp, size_t &base, uint32_t &tb_out) -> bool {
        if (pp >= kv_len) {
            return false;
        }
        const uint32_t logical = pp >> p.shift;
        if (logical >= p.max_blocks) {
            return false;
        }
        const uint32_t tb = table_row[(size_t)logical * p.table_stride[1]];
        if (tb == PA_NO_BLOCK || tb >= p.kv_blocks) {
            return false;
        }
        base = (size_t)tb * p.kv_stride[0] + head_base + (size_t)(pp & p.mask) * p.kv_stride[3];
        tb_out = tb;
        return true;
    };
    auto fetch = [&](size_t base, uint32_t tb, float (&kr)[EPL], float (&vr)[EPL]) {
        if (p.kv_vec) {
            pa_load_run<EPL>(p.kv_k, p.kv_dtype, base + d0, kr);
            pa_load_run<EPL>(p.kv_v, p.kv_dtype, base + d0, vr);
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const bool in = d0 + e < p.head_dim;
                const size_t i = base + (size_t)(d0 + e) * p.kv_stride[4];
                kr[e] = in ? pa_load(p.kv_k, p.kv_dtype, i) : 0.0f;
                vr[e] = in ? pa_load(p.kv_v, p.kv_dtype, i) : 0.0f;
            }
        }
        if (fp8) {  // code value times the block's scale: the reference's decoded element (:474-498)
            const size_t si = (size_t)tb * p.scale_stride[0] + (size_t)p.layer_idx * p.scale_stride[1] +
                              (size_t)kvh * p.scale_stride[2];
            const float ks = p.k_scale[si], vs = p.v_scale[si];
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                kr[e] = ks > 0.0f ? kr[e] * ks : 0.0f;
                vr[e] = vs > 0.0f ? vr[e] * vs : 0.0f;
            }
        }
    };
    auto absorb = [&](const float (&kr)[EPL], const float (&vr)[EPL]) {
#pragma unroll
        for (int h = 0; h < QH; ++h) {
            float dot = 0.0f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                dot = __builtin_fmaf(qv[h][e], kr[e], dot);
            }
            dot = row16_sum(dot);
            if (dot > m[h]) {  // the same decision in all 16 lanes of the group
                const float corr = m[h] == -INFINITY ? 0.0f : pa_exp(m[h] - dot);
                lsum[h] *= corr;
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    acc[h][e] *= corr;
                }
                m[h] = dot;
            }
            const float w = pa_exp(dot - m[h]);
            lsum[h] += w;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                acc[h][e] = __builtin_fmaf(w, vr[e], acc[h][e]);
            }
        }
    };
    // this workgroup's share of the history (the whole of it without a split)
    const uint32_t chunk = (kv_len + p.splits - 1u) / p.splits;
    const uint32_t first = blockIdx.z * chunk;
    const uint32_t stop = first + chunk < kv_len ? first + chunk : kv_len;
    for (uint32_t pp = first + (uint32_t)g; pp < stop; pp += 2u * PA_GROUPS) {
        size_t base0 = 0, base1 = 0;
        uint32_t tb0 = 0, tb1 = 0;
        const bool have0 = locate(pp, base0, tb0), have1 = pp + PA_GROUPS < stop && locate(pp + PA_GROUPS, base1, tb1);
        float k0[EPL], v0[EPL], k1[EPL], v1[EPL];
        if (have0) {
            fetch(base0, tb0, k0, v0);
        }
        if (have1) {
            fetch(base1, tb1, k1, v1);
        }
        if (have0) {
            absorb(k0, v0);
        }
        if (have1) {
            absorb(k1, v1);
        }
    }

    // the groups meet: out = sum_g acc_g * exp(m_g - M) / sum_g l_g * exp(m_g - M)
#pragma unroll
    for (int h = 0; h < QH; ++h) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            s_acc[g][h][d0 + e] = acc[h][e];
        }
        if (l == 0) {
            s_m[g][h] = m[h];
            s_l[g][h] = lsum[h];
        }
    }
    __syncthreads();
    for (uint32_t idx = (uint32_t)tid; idx < (uint32_t)QH * p.head_dim; idx += 16u * PA_GROUPS) {
        uint32_t h = 0, d = idx;  // idx = h * head_dim + d
        while (d >= p.head_dim) {
            d -= p.head_dim;
            ++h;
        }
        float big = -INFINITY;
#pragma unroll
        for (int gg = 0; gg < PA_GROUPS; ++gg) {
            big = fmaxf(big, s_m[gg][h]);
        }
        float o = 0.0f, total = 0.0f;
        // a NaN score (NaN in the query or in a row of the history) leaves a NaN sum of weights in its group: the head's
        // output is NaN then, as in the reference, whatever the maxima say (they skip NaN)
        bool bad = false;
#pragma unroll
        for (int gg = 0; gg < PA_GROUPS; ++gg) {
            bad = bad || s_l[gg][h] != s_l[gg][h];
        }
        if (big != -INFINITY) {  // has_any (:552-557)
#pragma unroll
            for (int gg = 0; gg < PA_GROUPS; ++gg) {
                const float f = s_m[gg][h] == -INFINITY ? 0.0f : pa_exp(s_m[gg][h] - big);
                total = __builtin_fmaf(s_l[gg][h], f, total);
                o = __builtin_fmaf(s_acc[gg][h][d], f, o);
            }
        }
        if (p.splits > 1u) {  // the shares of the history meet in k_pa_merge
            float *part = p.partial + (((size_t)t * p.num_q_heads + qh0 + h) * p.splits + blockIdx.z) * (p.head_dim + 2u);
            if (d == 0) {
                part[0] = big;
                part[1] = bad ? __uint_as_float(0x7fc00000u) : total;
            }
            part[2 + d] = o;
            continue;
        }
        o = bad ? __uint_as_float(0x7fc00000u) : (total > 0.0f ? o * (1.0f / total) : 0.0f);
        const size_t out_base = (size_t)t * p.out_stride[0] + (size_t)(qh0 + h) * p.out_stride[1];
        pa_store(p.out, p.act_dtype, out_base + (size_t)d * p.out_stride[2], o);
    }
}

// ---- attention with the scores on the matrix cores (FLOAT16 or BFLOAT16 cache rows of 128 values, blocks of 16
// positions or more)
// One workgroup of four wavefronts per (token, QH query heads of one key / value head, share of the history); a
// wavefront takes tiles of 16 consecutive positions (one cache block, or a 16-aligned part of one).
//   * Scores: S[position][head] = K[position][:] . q[head][:] as v_mfma_f32_16x16x16_f16 with the KEY ROWS as the row
//     operand, read from the cache straight into operand registers (lane (r, j) = (lane % 16, lane / 16) reads the 64
//     contiguous bytes of dimensions 32 j .. 32 j + 31 of position r: the k index of the c-th instruction stands for
//     dimensions 32 j + 4 c .. + 3, the same in both operands, so no value moves between lanes and none is converted).
//     The query is the column operand, scaled and split once into a FLOAT16 high part and a FLOAT16 remainder (two
//     instructions per step: products of FLOAT16 values are exact in fp32, the split leaves 2^-22 of the query); for
//     a BFLOAT16 cache (v_mfma_f32_16x16x16_bf16) into three BFLOAT16 parts of 8 bits each. Columns beyond QH are zero.
//   * The result layout puts positions 4 j + i (i = 0..3) of head n in lane (n, j): the online softmax of a head runs in
//     the four lanes n, n + 16, n + 32, n + 48 (two cross-lane exchanges per maximum and per sum).
//   * Output: the 16 lanes of group j hold dimensions 8 n .. 8 n + 7 of the value rows of THEIR four positions; the
//     weights of head h for these positions are fetched from lane (h, j) with ds_swizzle broadcasts; fp32
//     multiply-adds as before. The running output is rescaled only when a maximum moved (wavefront-wide test).
// The 16 partial outputs (4 wavefronts x 4 groups) meet in LDS like the 16 groups of k_pa_attend. fp32 accumulation
// everywhere; only the order of the sums differs from the reference.
typedef _Float16 pa_half4 __attribute__((ext_vector_type(4)));
typedef short pa_short4 __attribute__((ext_vector_type(4)));
typedef float pa_float4 __attribute__((ext_vector_type(4)));

template <int PATTERN>
__device__ __forceinline__ float pa_swizzle(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), PATTERN));
}
// value of lane (h, j) in every lane of the 16-lane group j (bit-mask mode: lane' = (lane & 0x10) | h inside each half)
template <int H>
__device__ __forceinline__ float pa_group_bcast(float v) {
    return pa_swizzle<0x10 | (H << 5)>(v);
}
// exchange with the lane 16 / 32 lanes away
__device__ __forceinline__ float pa_xor16(float v) {
    return pa_swizzle<0x1f | (0x10 << 10)>(v);
}
__device__ __forceinline__ float pa_xor32(float v) {
    return __shfl_xor(v, 32);
}

// Two e4m3 codes of a word (bytes 0, 1 or 2, 3) as a pair of FLOAT16 values in one instruction (gfx950's conversion
// with a power-of-two scale, here 1): exact, denormal codes included (both formats are linear there). Codes with all
// exponent bits set (NaN in the reference's e4m3, finite or NaN in the hardware's) are found by pa_fp8_nan_bits and
// take the reference's decoder.
typedef _Float16 pa_half2 __attribute__((ext_vector_type(2)));
template <int HI>
__device__ __forceinline__ uint32_t pa_fp8x2_to_f16(uint32_t w) {
    const pa_half2 v = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, HI != 0);
    return __builtin_bit_cast(uint32_t, v);
}
// bit 7 of a byte is set iff that byte of w is a NaN code (exponent field 15)
__device__ __forceinline__ uint32_t pa_fp8_nan_bits(uint32_t w) {
    return (w & 0x78787878u) + 0x08080808u;
}
// the same two words through the reference's decoder (NaN codes become NaN)
template <int HI>
__device__ __forceinline__ uint32_t pa_fp8x2_to_f16_slow(uint32_t w) {
    const uint32_t c0 = (w >> (HI ? 16 : 0)) & 0xffu, c1 = (w >> (HI ? 24 : 8)) & 0xffu;
    return (uint32_t)f2h(pa_fp8_to_f32(c0)) | ((uint32_t)f2h(pa_fp8_to_f32(c1)) << 16);
}

constexpr int PA_KV_F16 = 0, PA_KV_BF16 = 1, PA_KV_FP8 = 2;
constexpr uint32_t PA_PIPELINE_TILES = 24;  // tiles per workgroup (six per wavefront) from which the tile loop is pipelined

template <int QH, int KVT, bool PIPE>
__global__ __launch_bounds__(256) void k_pa_attend_mfma(const PaParams p) {
    constexpr bool BF16 = KVT == PA_KV_BF16, FP8 = KVT == PA_KV_FP8;
    constexpr int EPL = 8;  // head_dim == 128
    __shared__ float s_acc[PA_GROUPS][QH][16 * EPL];
    __shared__ float s_m[PA_GROUPS][QH], s_l[PA_GROUPS][QH];
    const uint32_t t = blockIdx.x;
    const uint32_t qh0 = blockIdx.y * QH;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, j = lane >> 4;
    const uint32_t seq = p.meta[t * p.meta_stride[0]];
    const uint32_t pos = p.meta[t * p.meta_stride[0] + p.meta_stride[1]];
    const uint32_t kv_len = seq < p.max_seqs ? pos + 1u : 0u;
    const uint32_t kvh = qh0 / p.group;

    // the query: head n (zero beyond QH), dimensions 32 j .. 32 j + 31, scaled, as high part + remainder(s)
    constexpr int PARTS = BF16 ? 3 : 2;
    uint2 qpart[PARTS][8];  // four 16-bit values of the storage type each
    {
        float qv[32];
#pragma unroll
        for (int e = 0; e < 32; ++e) {
            qv[e] = 0.0f;
        }
        if (n < QH) {
            const size_t q_base = (size_t)t * p.q_stride[0] + (size_t)(qh0 + n) * p.q_stride[1];
            if (p.q_vec) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float part[8];
                    pa_load_run<8>(p.q, p.act_dtype, q_base + 32u * j + 8u * c, part);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        qv[8 * c + e] = part[e];
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 32; ++e) {
                    qv[e] = pa_load(p.q, p.act_dtype, q_base + (size_t)(32 * j + e) * p.q_stride[2]);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            uint16_t bits[PARTS][4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float v = p.scale != 1.0f ? qv[4 * c + e] * p.scale : qv[4 * c + e];
#pragma unroll
                for (int part = 0; part < PARTS; ++part) {  // each remainder is exact in fp32
                    if constexpr (BF16) {
                        bits[part][e] = pa_f2bf(v);
                        v -= pa_bf2f(bits[part][e]);
                    } else {
                        bits[part][e] = f2h(v);
                        v -= h2f(bits[part][e]);
                    }
                }
            }
#pragma unroll
            for (int part = 0; part < PARTS; ++part) {
                qpart[part][c] = make_uint2((uint32_t)bits[part][0] | ((uint32_t)bits[part][1] << 16),
                                            (uint32_t)bits[part][2] | ((uint32_t)bits[part][3] << 16));
            }
        }
    }
    auto mma = [&](const uint2 kbits, const uint2 qbits, const pa_float4 c_in) -> pa_float4 {
        if constexpr (BF16) {
            return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(pa_short4, kbits),
                                                             __builtin_bit_cast(pa_short4, qbits), c_in, 0, 0, 0);
        } else {
            return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(pa_half4, kbits),
                                                         __builtin_bit_cast(pa_half4, qbits), c_in, 0, 0, 0);
        }
    };

    float m = -INFINITY, lsum = 0.0f;  // of head n (replicated in the four lanes n + 16 j)
    float acc[QH][EPL];
#pragma unroll
    for (int h = 0; h < QH; ++h) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            acc[h][e] = 0.0f;
        }
    }
    const size_t head_base = (size_t)p.layer_idx * p.kv_stride[1] + (size_t)kvh * p.kv_stride[2];
    const uint32_t *table_row = p.table + (size_t)seq * p.table_stride[0];
    // this workgroup's share of the history, in whole tiles of 16 positions
    const uint32_t tiles = (kv_len + 15u) >> 4;
    const uint32_t tiles_per_split = (tiles + p.splits - 1u) / p.splits;
    const uint32_t tile_first = blockIdx.z * tiles_per_split;
    const uint32_t tile_stop = tile_first + tiles_per_split < tiles ? tile_first + tiles_per_split : tiles;
    // Tiles of this wavefront: tile_first + wave, + 4, ... Two memory latencies lie in front of a tile's arithmetic, the
    // block table entry and then the rows it points to; with a handful of tiles per wavefront they were most of the
    // kernel's time. So the loop of the PIPE form runs a pipeline: while tile k is worked on, the rows of tile k + 1 and the table entry
    // of tile k + 2 are in flight. All of these loads are unconditional (a tile that does not exist or has no block
    // reads block 0 and is marked): a load behind a branch would make the compiler wait for everything in flight.
    struct TileRaw {
        uint4 k[4], v[4];  // FLOAT8_E4M3: k[0..1] = the 32 key codes, v[0..1] = 4 x 8 value codes
        float ks, vs;
        uint32_t p0;
        bool ok;
    };
    const uint32_t table_last = p.max_blocks > 0u ? p.max_blocks - 1u : 0u;
    auto table_entry = [&](uint32_t tile) -> uint32_t {
        const uint32_t logical = (tile << 4) >> p.shift;
        return table_row[(size_t)(logical < table_last ? logical : table_last) * p.table_stride[1]];
    };
    auto request = [&](TileRaw &r, uint32_t tile, uint32_t tb) {
        const uint32_t logical = (tile << 4) >> p.shift;
        r.ok = tile < tile_stop && logical < p.max_blocks && tb != PA_NO_BLOCK && tb < p.kv_blocks;  // else: a hole
        r.p0 = r.ok ? tile << 4 : 0u;
        const uint32_t tbs = r.ok ? tb : 0u;
        const size_t tile_base = (size_t)tbs * p.kv_stride[0] + head_base + (size_t)(r.p0 & p.mask) * p.kv_stride[3];
        // key rows: position n of the tile, dimensions 32 j .. + 31; value rows: positions 4 j + i, dimensions 8 n .. + 7
        if constexpr (FP8) {
            const size_t si = (size_t)tbs * p.scale_stride[0] + (size_t)p.layer_idx * p.scale_stride[1] +
                              (size_t)kvh * p.scale_stride[2];
            r.ks = p.k_scale[si];
            r.vs = p.v_scale[si];
            const uint8_t *krow = (const uint8_t *)p.kv_k + tile_base + (size_t)n * p.kv_stride[3] + 32u * j;
            r.k[0] = *(const uint4 *)krow;
            r.k[1] = *(const uint4 *)(krow + 16);
            uint2 vr[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                vr[i] = *(const uint2 *)((const uint8_t *)p.kv_v + tile_base + (size_t)(4 * j + i) * p.kv_stride[3] + 8u * n);
            }
            r.v[0] = make_uint4(vr[0].x, vr[0].y, vr[1].x, vr[1].y);
            r.v[1] = make_uint4(vr[2].x, vr[2].y, vr[3].x, vr[3].y);
        } else {
            const uint16_t *krow = (const uint16_t *)p.kv_k + tile_base + (size_t)n * p.kv_stride[3] + 32u * j;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                r.k[c] = *(const uint4 *)(krow + 8 * c);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                r.v[i] = *(const uint4 *)((const uint16_t *)p.kv_v + tile_base + (size_t)(4 * j + i) * p.kv_stride[3] + 8u * n);
            }
        }
    };
    auto consume = [&](const TileRaw &r) {
        if (!r.ok) {
            return;
        }
        const uint32_t p0 = r.p0;  // first position of the tile
        uint4 kq[4], vq[4];
        float k_unit = 1.0f, v_unit = 1.0f;  // FLOAT8_E4M3: what one unit of the FLOAT16 operands stands for
        if constexpr (FP8) {
            // codes -> FLOAT16 operands in registers (exact); the block's scale is applied to the scores and to the
            // softmax weights. A scale that is not positive decodes to zeros (the reference's
            // cpu_paged_attention_fp8_dequant); a tile that holds a NaN code takes the reference's decoder.
            const float ks = r.ks, vs = r.vs;
            const uint32_t kw[8] = {r.k[0].x, r.k[0].y, r.k[0].z, r.k[0].w, r.k[1].x, r.k[1].y, r.k[1].z, r.k[1].w};
            const uint2 vr[4] = {make_uint2(r.v[0].x, r.v[0].y), make_uint2(r.v[0].z, r.v[0].w),
                                 make_uint2(r.v[1].x, r.v[1].y), make_uint2(r.v[1].z, r.v[1].w)};
                uint32_t nan_k = 0, nan_v = 0;
    #pragma unroll
                for (int c = 0; c < 8; ++c) {
                    nan_k |= pa_fp8_nan_bits(kw[c]);
                }
    #pragma unroll
                for (int i = 0; i < 4; ++i) {
                    nan_v |= pa_fp8_nan_bits(vr[i].x) | pa_fp8_nan_bits(vr[i].y);
                }
                const bool k_live = ks > 0.0f, v_live = vs > 0.0f;
                const bool slow = ((nan_k & 0x80808080u) != 0 && k_live) || ((nan_v & 0x80808080u) != 0 && v_live);
                if (__builtin_amdgcn_ballot_w64(slow) == 0) {
    #pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        kq[c] = make_uint4(pa_fp8x2_to_f16<0>(kw[2 * c]), pa_fp8x2_to_f16<1>(kw[2 * c]),
                                           pa_fp8x2_to_f16<0>(kw[2 * c + 1]), pa_fp8x2_to_f16<1>(kw[2 * c + 1]));
                    }
    #pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        vq[i] = make_uint4(pa_fp8x2_to_f16<0>(vr[i].x), pa_fp8x2_to_f16<1>(vr[i].x),
                                           pa_fp8x2_to_f16<0>(vr[i].y), pa_fp8x2_to_f16<1>(vr[i].y));
                    }
                } else {
    #pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        kq[c] = make_uint4(pa_fp8x2_to_f16_slow<0>(kw[2 * c]), pa_fp8x2_to_f16_slow<1>(kw[2 * c]),
                                           pa_fp8x2_to_f16_slow<0>(kw[2 * c + 1]), pa_fp8x2_to_f16_slow<1>(kw[2 * c + 1]));
                    }
    #pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        vq[i] = make_uint4(pa_fp8x2_to_f16_slow<0>(vr[i].x), pa_fp8x2_to_f16_slow<1>(vr[i].x),
                                           pa_fp8x2_to_f16_slow<0>(vr[i].y), pa_fp8x2_to_f16_slow<1>(vr[i].y));
                    }
                }
                if (!k_live) {
    #pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        kq[c] = make_uint4(0, 0, 0, 0);
                    }
                }
                if (!v_live) {
    #pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        vq[i] = make_uint4(0, 0, 0, 0);
                    }
                }
                k_unit = k_live ? ks : 0.0f;
                v_unit = v_live ? vs : 0.0f;
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                kq[c] = r.k[c];
                vq[c] = r.v[c];
            }
        }
            pa_float4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
    #pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint2 k0 = make_uint2(kq[c].x, kq[c].y), k1 = make_uint2(kq[c].z, kq[c].w);
    #pragma unroll
                for (int part = 0; part < PARTS; ++part) {
                    sc = mma(k0, qpart[part][2 * c], sc);
                }
    #pragma unroll
                for (int part = 0; part < PARTS; ++part) {
                    sc = mma(k1, qpart[part][2 * c + 1], sc);
                }
            }
            // positions beyond the sequence (the last tile): no score, no value
            const bool whole = p0 + 16u <= kv_len;
            float s4[4] = {sc[0], sc[1], sc[2], sc[3]};
            if constexpr (FP8) {
    #pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s4[i] *= k_unit;
                }
            }
            if (!whole) {
    #pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (p0 + 4u * j + (uint32_t)i >= kv_len) {
                        s4[i] = -INFINITY;
                        vq[i] = make_uint4(0, 0, 0, 0);
                    }
                }
            }
            // online softmax of head n over the tile's 16 positions (lanes n, n + 16, n + 32, n + 48)
            float big = fmaxf(fmaxf(s4[0], s4[1]), fmaxf(s4[2], s4[3]));
            big = fmaxf(big, pa_xor16(big));
            big = fmaxf(big, pa_xor32(big));
            const float m_new = fmaxf(m, big);
            const float corr = m == -INFINITY ? 0.0f : pa_exp(m - m_new);
            float w4[4];
    #pragma unroll
            for (int i = 0; i < 4; ++i) {
                w4[i] = pa_exp(s4[i] - m_new);
            }
            float tsum = (w4[0] + w4[1]) + (w4[2] + w4[3]);
            tsum += pa_xor16(tsum);
            tsum += pa_xor32(tsum);
            lsum = lsum * corr + tsum;
            const bool moved = m_new != m;
            m = m_new;
            // rescale the running output of the heads whose maximum moved
            if (__builtin_amdgcn_ballot_w64(moved && n < QH) != 0) {
                float f[QH];
                f[0] = pa_group_bcast<0>(corr);
                if constexpr (QH > 1) {
                    f[1] = pa_group_bcast<1>(corr);
                }
                if constexpr (QH > 2) {
                    f[2] = pa_group_bcast<2>(corr);
                    f[3] = pa_group_bcast<3>(corr);
                }
    #pragma unroll
                for (int h = 0; h < QH; ++h) {
    #pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        acc[h][e] *= f[h];
                    }
                }
            }
            // values: this group's four positions, dimensions 8 n .. 8 n + 7
    #pragma unroll
            for (int i = 0; i < 4; ++i) {
                float vr[EPL];
                const uint32_t vw[4] = {vq[i].x, vq[i].y, vq[i].z, vq[i].w};
    #pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if constexpr (BF16) {
                        vr[2 * e] = __uint_as_float(vw[e] << 16);
                        vr[2 * e + 1] = __uint_as_float(vw[e] & 0xffff0000u);
                    } else {
                        vr[2 * e] = h2f((uint16_t)(vw[e] & 0xffffu));
                        vr[2 * e + 1] = h2f((uint16_t)(vw[e] >> 16));
                    }
                }
                float wh[QH];
                const float wi = FP8 ? w4[i] * v_unit : w4[i];  // the value rows' unit goes with the weight
                wh[0] = pa_group_bcast<0>(wi);
                if constexpr (QH > 1) {
                    wh[1] = pa_group_bcast<1>(wi);
                }
                if constexpr (QH > 2) {
                    wh[2] = pa_group_bcast<2>(wi);
                    wh[3] = pa_group_bcast<3>(wi);
                }
    #pragma unroll
                for (int h = 0; h < QH; ++h) {
    #pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        acc[h][e] = __builtin_fmaf(wh[h], vr[e], acc[h][e]);
                    }
                }
            }
    };
    const bool any_tile = p.kv_blocks > 0u && p.max_blocks > 0u && tile_first + (uint32_t)wave < tile_stop;
    // Few tiles per wavefront (short histories, the tokens of a prompt): one after the other; the pipeline's extra
    // requests (a tile and two table entries beyond the end) cost more than they hide there (16 x 512 positions
    // 18.7 -> 22.9 us, a prompt of 512 tokens 76 -> 101 us with the pipeline everywhere).
    if (any_tile && (!PIPE || tile_stop - tile_first < PA_PIPELINE_TILES)) {
        TileRaw r;
        for (uint32_t tile = tile_first + (uint32_t)wave; tile < tile_stop; tile += 4u) {
            request(r, tile, table_entry(tile));
            consume(r);
        }
    } else if (any_tile) {
        if constexpr (PIPE) {
            uint32_t tile = tile_first + (uint32_t)wave;
            TileRaw ra, rb;
            uint32_t e1 = table_entry(tile + 4u), e2 = table_entry(tile + 8u);
            request(ra, tile, table_entry(tile));
            for (; tile < tile_stop; tile += 8u) {
                request(rb, tile + 4u, e1);
                const uint32_t e3 = table_entry(tile + 12u);
                consume(ra);
                request(ra, tile + 8u, e2);
                const uint32_t e4 = table_entry(tile + 16u);
                consume(rb);
                e1 = e3;
                e2 = e4;
            }
        }
    }

    // the 16 partial outputs meet: group g = 4 wave + j; a wavefront's sum of weights is counted once (its group 0)
    const int g = 4 * wave + j;
    const uint32_t d0 = (uint32_t)n * EPL;
#pragma unroll
    for (int h = 0; h < QH; ++h) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            s_acc[g][h][d0 + e] = acc[h][e];
        }
    }
    if (n < QH) {
        s_m[g][n] = m;
        s_l[g][n] = j == 0 ? lsum : 0.0f;
    }
    __syncthreads();
    for (uint32_t idx = (uint32_t)tid; idx < (uint32_t)QH * 128u; idx += 256u) {
        const uint32_t h = idx >> 7, d = idx & 127u;
        float top = -INFINITY;
#pragma unroll
        for (int gg = 0; gg < PA_GROUPS; ++gg) {
            top = fmaxf(top, s_m[gg][h]);
        }
        float o = 0.0f, total = 0.0f;
        // a NaN score (NaN in the query or in a row of the history) leaves a NaN sum of weights in its group: the head's
        // output is NaN then, as in the reference, whatever the maxima say (they skip NaN)
        bool bad = false;
#pragma unroll
        for (int gg = 0; gg < PA_GROUPS; ++gg) {
            bad = bad || s_l[gg][h] != s_l[gg][h];
        }
        if (top != -INFINITY) {
#pragma unroll
            for (int gg = 0; gg < PA_GROUPS; ++gg) {
                const float f = s_m[gg][h] == -INFINITY ? 0.0f : pa_exp(s_m[gg][h] - top);
                total = __builtin_fmaf(s_l[gg][h], f, total);
                o = __builtin_fmaf(s_acc[gg][h][d], f, o);
            }
        }
        if (p.splits > 1u) {
            float *part = p.partial + (((size_t)t * p.num_q_heads + qh0 + h) * p.splits + blockIdx.z) * (p.head_dim + 2u);
            if (d == 0) {
                part[0] = top;
                part[1] = bad ? __uint_as_float(0x7fc00000u) : total;
            }
            part[2 + d] = o;
            continue;
        }
        o = bad ? __uint_as_float(0x7fc00000u) : (total > 0.0f ? o * (1.0f / total) : 0.0f);
        const size_t out_base = (size_t)t * p.out_stride[0] + (size_t)(qh0 + h) * p.out_stride[1];
        pa_store(p.out, p.act_dtype, out_base + (size_t)d * p.out_stride[2], o);
    }
}

// the shares of a (token, head) pair's history: out = sum_s o_s * exp(M_s - M) / sum_s l_s * exp(M_s - M)
__global__ __launch_bounds__(256) void k_pa_merge(const PaParams p) {
    __shared__ float s_big[64], s_tot[64];  // splits <= 64
    const uint32_t t = blockIdx.x, qh = blockIdx.y;
    const float *part = p.partial + ((size_t)t * p.num_q_heads + qh) * p.splits * (p.head_dim + 2u);
    if (threadIdx.x < p.splits) {
        s_big[threadIdx.x] = part[(size_t)threadIdx.x * (p.head_dim + 2u)];
        s_tot[threadIdx.x] = part[(size_t)threadIdx.x * (p.head_dim + 2u) + 1];
    }
    __syncthreads();
    float big = -INFINITY;
    for (uint32_t z = 0; z < p.splits; ++z) {
        big = fmaxf(big, s_big[z]);
    }
    const size_t out_base = (size_t)t * p.out_stride[0] + (size_t)qh * p.out_stride[1];
    for (uint32_t d = threadIdx.x; d < p.head_dim; d += blockDim.x) {
        float o = 0.0f, total = 0.0f;
        bool bad = false;  // a share saw a NaN score
        for (uint32_t z = 0; z < p.splits; ++z) {
            bad = bad || s_tot[z] != s_tot[z];
        }
        if (big != -INFINITY) {
            for (uint32_t z = 0; z < p.splits; ++z) {
                const float f = s_big[z] == -INFINITY ? 0.0f : pa_exp(s_big[z] - big);
                total = __builtin_fmaf(s_tot[z], f, total);
                o = __builtin_fmaf(part[(size_t)z * (p.head_dim + 2u) + 2 + d], f, o);
            }
        }
        o = bad ? __uint_as_float(0x7fc00000u) : (total > 0.0f ? o * (1.0f / total) : 0.0f);
        pa_store(p.out, p.act_dtype, out_base + (size_t)d * p.out_stride[2], o);
    }
}

template <int EPL, int QH>
static void pa_launch(marmot_hip_device *dev, const PaParams &p) {
    hipLaunchKernelGGL((k_pa_attend<EPL, QH>), dim3(p.token_count, p.num_q_heads / QH, p.splits),
                       dim3(16 * PA_GROUPS), 0, dev->stream, p);
}

static bool pa_float_dtype(int d) {
    return d == MARMOT_HIP_DTYPE_F32 || d == MARMOT_HIP_DTYPE_F16 || d == MARMOT_HIP_DTYPE_BF16;
}

static size_t pa_elem_size(int d) {
    return d == MARMOT_HIP_DTYPE_F32 ? 4 : (d == MARMOT_HIP_DTYPE_F8_E4M3 ? 1 : 2);
}

} // namespace mh

using namespace mh;

extern "C" int marmot_hip_fill_bytes_internal(marmot_hip_device_t *dev, void *d_dst, int value, size_t size);

extern "C" int marmot_hip_paged_attention(marmot_hip_device_t *dev, const marmot_hip_paged_attention_t *a,
                                          int validate_meta) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (a == nullptr || a->d_token_meta == nullptr || a->d_q == nullptr || a->d_k_new == nullptr ||
        a->d_v_new == nullptr || a->d_kv_k == nullptr || a->d_kv_v == nullptr || a->d_block_table == nullptr ||
        a->d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "paged_attention descriptor invalid");
    }
    if (a->token_count == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (a->num_q_heads == 0 || a->num_kv_heads == 0 || a->head_dim == 0 || a->block_size == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "paged_attention requires non-zero dimensions");
    }
    if ((a->block_size & (a->block_size - 1u)) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "paged_attention block_size must be power of two");
    }
    if (a->num_q_heads % a->num_kv_heads != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "paged_attention requires num_q_heads divisible by num_kv_heads");
    }
    const bool fp8 = a->kv_dtype == MARMOT_HIP_DTYPE_F8_E4M3;
    if (!pa_float_dtype(a->act_dtype) || (!fp8 && !pa_float_dtype(a->kv_dtype))) {
        return set_error(MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE, "paged_attention dtype not supported");
    }
    if (fp8 && (a->d_kv_k_scale == nullptr || a->d_kv_v_scale == nullptr)) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "paged_attention FP8 KV requires scale tensors");
    }
    if (!fp8 && (a->d_kv_k_scale != nullptr || a->d_kv_v_scale != nullptr)) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "paged_attention scale tensors require FP8 KV");
    }
    if (a->kv_layers <= a->layer_idx) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "paged_attention layer_idx out of range");
    }
    if (a->head_dim > 256) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "paged_attention: head_dim %u is more than 256", a->head_dim);
    }
    if (a->num_q_heads > 65535u || a->num_kv_heads > 65535u) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "paged_attention: more than 65535 heads");
    }
    MH_HIP(hipSetDevice(dev->device_index));
    PaParams p;
    p.token_count = a->token_count, p.layer_idx = a->layer_idx, p.num_q_heads = a->num_q_heads;
    p.num_kv_heads = a->num_kv_heads, p.head_dim = a->head_dim, p.block_size = a->block_size;
    p.scale = a->scale, p.act_dtype = a->act_dtype, p.kv_dtype = a->kv_dtype;
    p.meta = a->d_token_meta, p.q = a->d_q, p.k_new = a->d_k_new, p.v_new = a->d_v_new;
    p.kv_k = a->d_kv_k, p.kv_v = a->d_kv_v, p.table = a->d_block_table, p.out = a->d_out;
    for (int i = 0; i < 2; ++i) {
        p.meta_stride[i] = a->meta_stride[i];
        p.table_stride[i] = a->table_stride[i];
    }
    for (int i = 0; i < 3; ++i) {
        p.q_stride[i] = a->q_stride[i], p.k_stride[i] = a->k_stride[i], p.v_stride[i] = a->v_stride[i];
        p.out_stride[i] = a->out_stride[i];
    }
    for (int i = 0; i < 5; ++i) {
        p.kv_stride[i] = a->kv_stride[i];
    }
    p.kv_blocks = a->kv_blocks, p.kv_layers = a->kv_layers, p.max_seqs = a->max_seqs, p.max_blocks = a->max_blocks_per_seq;
    p.shift = 0;
    while ((1u << p.shift) < a->block_size) {
        ++p.shift;
    }
    p.mask = a->block_size - 1u;
    p.group = a->num_q_heads / a->num_kv_heads;
    const int epl = a->head_dim <= 64 ? 4 : (a->head_dim <= 128 ? 8 : 16);
    // 16-byte runs: the head dimension is exactly 16 lanes x EPL values, unit stride, every row start 16-byte aligned
    const size_t asz = pa_elem_size(a->act_dtype), ksz = pa_elem_size(a->kv_dtype);
    const size_t run_a = (size_t)epl * asz < 16 ? (size_t)epl * asz : 16, run_k = (size_t)epl * ksz < 16 ? (size_t)epl * ksz : 16;
    const bool exact = a->head_dim == (uint32_t)(16 * epl);
    p.q_vec = exact && a->q_stride[2] == 1 && (((uintptr_t)a->d_q) % run_a) == 0 && (a->q_stride[0] * asz) % run_a == 0 &&
              (a->q_stride[1] * asz) % run_a == 0;
    p.kv_vec = exact && a->kv_stride[4] == 1 && (((uintptr_t)a->d_kv_k) % run_k) == 0 &&
               (((uintptr_t)a->d_kv_v) % run_k) == 0;
    for (int i = 0; i < 4 && p.kv_vec; ++i) {
        p.kv_vec = (a->kv_stride[i] * ksz) % run_k == 0;
    }
    p.k_scale = a->d_kv_k_scale, p.v_scale = a->d_kv_v_scale;
    for (int i = 0; i < 3; ++i) {
        p.scale_stride[i] = a->scale_stride[i];
    }
    p.new_kmax = p.new_vmax = p.min_off = p.claim = nullptr;
    p.flag = nullptr;
    if (validate_meta != 0 && !dev->capturing) {
        void *ws = nullptr;
        MH_TRY(workspace_reserve(dev, 256, &ws));
        p.flag = (int *)ws;
        MH_TRY(marmot_hip_fill_bytes_internal(dev, ws, 0, sizeof(int)));
        hipLaunchKernelGGL(k_pa_check, dim3((a->token_count + 255) / 256), dim3(256), 0, dev->stream, p);
        MH_HIP(hipGetLastError());
        int host_flag = 0;
        MH_HIP(hipMemcpyAsync(&host_flag, p.flag, sizeof(int), hipMemcpyDeviceToHost, dev->stream));
        MH_HIP(hipStreamSynchronize(dev->stream));
        if (host_flag != 0) {
            return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH,
                             "paged_attention seq_slot or kv_slot block out of range at token %u",
                             a->token_count - (uint32_t)host_flag);
        }
    }
    // workspace: [fp8 scratch][partial results of split histories]
    const size_t fp8_words = fp8 ? 3 * a->kv_blocks * a->num_kv_heads + a->kv_blocks : 0;
    const size_t fp8_bytes = (fp8_words * sizeof(uint32_t) + 255) & ~(size_t)255;
    // query heads per workgroup: as many heads of one key / value head as the LDS tile of the final merge allows
    const int qh_max = epl == 16 ? 2 : 4;
    const int qh = (p.group % 4 == 0 && qh_max >= 4) ? 4 : (p.group % 2 == 0 ? 2 : 1);
    // few (token, heads) pairs (a decode step): the history is split over workgroups until the chip is about eight
    // (three for the matrix-core kernel) workgroups per compute unit deep, and a second kernel joins the shares
    const size_t pairs = (size_t)a->token_count * (a->num_q_heads / (uint32_t)qh);
    // FLOAT16 cache rows of 128 contiguous values in blocks of 16 positions or more: the scores on the matrix cores
    const bool kv_bf16 = a->kv_dtype == MARMOT_HIP_DTYPE_BF16;
    bool rows16 = (((uintptr_t)a->d_kv_k) & 15) == 0;  // FLOAT8_E4M3: 16 codes per load of a key row
    for (int i = 0; i < 4; ++i) {
        rows16 = rows16 && (a->kv_stride[i] * ksz) % 16 == 0;
    }
    const bool mfma_scores = (a->kv_dtype == MARMOT_HIP_DTYPE_F16 || kv_bf16 || (fp8 && rows16)) && p.kv_vec &&
                             a->head_dim == 128 && a->block_size >= 16 && !dev->knobs.no_attention_mfma;
    // (measured, 16 sequences x 4096 / x 512 positions, 32 / 8 heads: the matrix-core kernel 57.6 / 22.1 us at eight
    // workgroups per compute unit, 56.2 / 16.2 at four, 50.5 / 17.0 at three, 52.1 / 15.5 at two, 76.1 / 17.0 at one)
    const size_t want = (mfma_scores ? 3u : 8u) * (size_t)dev->props.multiProcessorCount;
    p.splits = 1;
    p.partial = nullptr;
    if (pairs * 2 <= want) {
        size_t sp = (want + pairs - 1) / pairs;
        p.splits = (uint32_t)(sp > 64 ? 64 : sp);
    }
    const size_t partial_bytes =
        p.splits > 1u ? (size_t)a->token_count * a->num_q_heads * p.splits * (a->head_dim + 2u) * sizeof(float) : 0;
    if (fp8_bytes + partial_bytes != 0) {
        void *ws = nullptr;
        MH_TRY(workspace_reserve(dev, fp8_bytes + partial_bytes, &ws));
        if (fp8) {
            p.new_kmax = (uint32_t *)ws;
            p.new_vmax = p.new_kmax + a->kv_blocks * a->num_kv_heads;
            p.min_off = p.new_vmax + a->kv_blocks * a->num_kv_heads;
            p.claim = p.min_off + a->kv_blocks;
        }
        p.partial = p.splits > 1u ? (float *)((uint8_t *)ws + fp8_bytes) : nullptr;
    }
    const dim3 per_token(a->token_count, a->num_kv_heads);
    if (fp8) {
        const size_t cells = a->kv_blocks * a->num_kv_heads;
        if (cells > ((size_t)1 << 32)) {
            return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "paged_attention: FP8 cache of %zu blocks", a->kv_blocks);
        }
        if (a->token_count <= PA_FP8_ONE_TOKENS && !dev->knobs.no_fp8_update_fused) {
            hipLaunchKernelGGL(k_pa_fp8_update, per_token, dim3(128), 0, dev->stream, p);
        } else {
            hipLaunchKernelGGL(k_pa_fp8_init, dim3((unsigned)((cells + 255) / 256)), dim3(256), 0, dev->stream, p);
            hipLaunchKernelGGL(k_pa_fp8_scan_new, per_token, dim3(128), 0, dev->stream, p);
            hipLaunchKernelGGL(k_pa_fp8_rescale, per_token, dim3(128), 0, dev->stream, p);
            hipLaunchKernelGGL(k_pa_fp8_store, per_token, dim3(128), 0, dev->stream, p);
        }
    } else {
        hipLaunchKernelGGL(k_pa_write, per_token, dim3(a->head_dim <= 64 ? 64 : 128), 0, dev->stream, p);
    }
    MH_HIP(hipGetLastError());
    if (mfma_scores) {
        const dim3 grid(p.token_count, p.num_q_heads / (uint32_t)qh, p.splits), block(256);
        // FLOAT8_E4M3 decode steps over long contexts (few tokens, a block table of 2048 positions or more): the form
        // whose tile loop is pipelined (16 x 4096 positions 60.7 -> 48.7 us). It needs the registers of a third
        // resident wavefront per SIMD, which short histories and prompts miss more than they gain (FLOAT16, pipeline
        // compiled in: 16 x 512 positions 18.7 -> 23.9 us, a prompt of 512 tokens 76 -> 105 us), and a FLOAT16 cache at
        // 4096 positions runs at the memory's rate either way (53.0 / 53.0 us).
        const bool pipe = fp8 && p.splits > 1u && (size_t)p.max_blocks * a->block_size >= 2048u;
        if (fp8 && pipe) {
            if (qh == 4) {
                hipLaunchKernelGGL((k_pa_attend_mfma<4, PA_KV_FP8, true>), grid, block, 0, dev->stream, p);
            } else if (qh == 2) {
                hipLaunchKernelGGL((k_pa_attend_mfma<2, PA_KV_FP8, true>), grid, block, 0, dev->stream, p);
            } else {
                hipLaunchKernelGGL((k_pa_attend_mfma<1, PA_KV_FP8, true>), grid, block, 0, dev->stream, p);
            }
        } else if (fp8) {
            if (qh == 4) {
                hipLaunchKernelGGL((k_pa_attend_mfma<4, PA_KV_FP8, false>), grid, block, 0, dev->stream, p);
            } else if (qh == 2) {
                hipLaunchKernelGGL((k_pa_attend_mfma<2, PA_KV_FP8, false>), grid, block, 0, dev->stream, p);
            } else {
                hipLaunchKernelGGL((k_pa_attend_mfma<1, PA_KV_FP8, false>), grid, block, 0, dev->stream, p);
            }
        } else if (kv_bf16) {
            if (qh == 4) {
                hipLaunchKernelGGL((k_pa_attend_mfma<4, PA_KV_BF16, false>), grid, block, 0, dev->stream, p);
            } else if (qh == 2) {
                hipLaunchKernelGGL((k_pa_attend_mfma<2, PA_KV_BF16, false>), grid, block, 0, dev->stream, p);
            } else {
                hipLaunchKernelGGL((k_pa_attend_mfma<1, PA_KV_BF16, false>), grid, block, 0, dev->stream, p);
            }
        } else if (qh == 4) {
            hipLaunchKernelGGL((k_pa_attend_mfma<4, PA_KV_F16, false>), grid, block, 0, dev->stream, p);
        } else if (qh == 2) {
            hipLaunchKernelGGL((k_pa_attend_mfma<2, PA_KV_F16, false>), grid, block, 0, dev->stream, p);
        } else {
            hipLaunchKernelGGL((k_pa_attend_mfma<1, PA_KV_F16, false>), grid, block, 0, dev->stream, p);
        }
    } else if (epl == 4) {
        qh == 4 ? pa_launch<4, 4>(dev, p) : qh == 2 ? pa_launch<4, 2>(dev, p) : pa_launch<4, 1>(dev, p);
    } else if (epl == 8) {
        qh == 4 ? pa_launch<8, 4>(dev, p) : qh == 2 ? pa_launch<8, 2>(dev, p) : pa_launch<8, 1>(dev, p);
    } else {
        qh == 2 ? pa_launch<16, 2>(dev, p) : pa_launch<16, 1>(dev, p);
    }
    MH_HIP(hipGetLastError());
    if (p.splits > 1u) {
        hipLaunchKernelGGL(k_pa_merge, dim3(a->token_count, a->num_q_heads), dim3(a->head_dim <= 64 ? 64 : 128), 0,
                           dev->stream, p);
        MH_HIP(hipGetLastError());
    }
    set_route(mfma_scores ? "paged_attention_mfma_scores" : "paged_attention");
    return MARMOT_HIP_SUCCESS;
}

// Decode matvec / small-batch kernels for block-quantized weights with quantized activations
// (the "packed" route of the reference's CPU backend: Q8_K activations for K-quants, Q8_0 for Q4_0/Q8_0).
//
// Work decomposition (same for every format):
//   * A weight row is a run of GGUF blocks. One "wave-load" is 64 lanes x 16 bytes of packed values:
//     Q4_K: 8 blocks (8 lanes per block), Q6_K: 16 blocks (4 lanes per block), Q8_0/Q4_0: 64 blocks.
//   * A workgroup of W wavefronts covers the whole row: wavefront w owns wave-loads w*C .. w*C+C-1, so a lane
//     always sees the same block position and the same bytes inside the block. Its share of the quantized
//     activations is therefore loop-invariant and lives in registers for all rows the workgroup visits.
//   * The workgroup walks `rows_per_wg` consecutive rows, R rows per iteration; all R*C*(2..4) 16-byte loads
//     of an iteration are issued before any is consumed, which is what keeps HBM busy.
//   * Per row and column the lanes' fp32 partial sums are reduced with DPP; with W > 1 the per-wavefront sums
//     meet in LDS once, after the last row.
//   * For fp32 activations the Q8_K / Q8_0 quantization of the activations is fused into the kernel prologue:
//     the lanes that share a block (8 / 4 / 1 lanes) quantize exactly their own values, with the same arithmetic
//     as the standalone quantizer kernels, so no separate launch and no scratch round trip is needed.
// Integer sub-block dots use v_dot4c_i32_i8; the fp32 scale-accumulate matches
// cpu_vec_dot_{q4_k,q6_k}_q8_k / cpu_vec_dot_{q8_0,q4_0}_q8_0 (vec_dot_impl.h) up to summation order.
#include "mh_common.h"

#include <type_traits>

#include <float.h>
#include <stdlib.h>

namespace mh {

struct ActView {
    const int8_t *qs;
    const float *d;
    const int16_t *sums;
    size_t kp;
    size_t nb;
};

template <int N>
struct U4N {
    uint4 v[N];
};

__device__ __forceinline__ uint4 ld16(const void *p) {
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}
__device__ __forceinline__ uint2 ld8(const void *p) {
    uint2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}
__device__ __forceinline__ uint32_t ld4(const void *p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}
__device__ __forceinline__ uint16_t ld2(const void *p) {
    uint16_t v;
    __builtin_memcpy(&v, p, 2);
    return v;
}

__device__ __forceinline__ int dot16(const uint4 &w, const uint4 &a, int acc) {
    acc = sdot4(w.x, a.x, acc);
    acc = sdot4(w.y, a.y, acc);
    acc = sdot4(w.z, a.z, acc);
    acc = sdot4(w.w, a.w, acc);
    return acc;
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) | ((uint32_t)(d & 0xff) << 24);
}

// 16 consecutive fp32 activations (64-byte aligned when K is a multiple of 16)
__device__ __forceinline__ void ld16f(const float *p, float *v) {
    const float4 a = ((const float4 *)p)[0], b = ((const float4 *)p)[1], c = ((const float4 *)p)[2],
                 d = ((const float4 *)p)[3];
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w;
    v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
    v[8] = c.x, v[9] = c.y, v[10] = c.z, v[11] = c.w;
    v[12] = d.x, v[13] = d.y, v[14] = d.z, v[15] = d.w;
}

// Q8_K quantization (matmul_quant_pack.c:106-142) of one 256-value block whose values are spread over LPB
// adjacent lanes: this lane owns RUNS runs of 16 consecutive values starting at block offsets off[r].
// Produces this lane's int8 values (RUNS uint4), the sums of each run (= bsums entries) and the block scale d.
// SIGNAL: a workgroup barrier right after the loads have been issued (not returned); a loader wavefront waits on it
// so that its own, much larger, requests queue up behind these.
template <int RUNS, int LPB, bool SIGNAL = false>
__device__ __forceinline__ void q8k_quantize_runs(const float *xblk, const int (&off)[RUNS], uint4 (&q)[RUNS],
                                                  int (&bs)[RUNS], float &d) {
    float v[RUNS][16];
#pragma unroll
    for (int r = 0; r < RUNS; ++r) {
        ld16f(xblk + off[r], v[r]);
    }
    if (SIGNAL) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    float best_abs = 0.0f, best_val = 0.0f;
    int best_idx = 0x7fffffff;
#pragma unroll
    for (int r = 0; r < RUNS; ++r) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float ax = fabsf(v[r][i]);
            const bool gt = ax > best_abs;  // runs are visited in increasing offset order: first occurrence wins
            best_abs = gt ? ax : best_abs;
            best_val = gt ? v[r][i] : best_val;
            best_idx = gt ? off[r] + i : best_idx;
        }
    }
#pragma unroll
    for (int o = 1; o < LPB; o <<= 1) {
        const float o_abs = __shfl_xor(best_abs, o);
        const float o_val = __shfl_xor(best_val, o);
        const int o_idx = __shfl_xor(best_idx, o);
        const bool take = o_abs > best_abs || (o_abs == best_abs && o_idx < best_idx);
        best_abs = take ? o_abs : best_abs;
        best_val = take ? o_val : best_val;
        best_idx = take ? o_idx : best_idx;
    }
    d = 0.0f;
#pragma unroll
    for (int r = 0; r < RUNS; ++r) {
        q[r] = make_uint4(0, 0, 0, 0);
        bs[r] = 0;
    }
    if (best_abs > 0.0f) {
        const float iscale = -127.0f / best_val;
#pragma unroll
        for (int r = 0; r < RUNS; ++r) {
            int t[16];
            int s = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int z = nearest_int_clamped(iscale * v[r][i]);
                t[i] = z > 127 ? 127 : z;
                s += t[i];
            }
            q[r].x = pack4(t[0], t[1], t[2], t[3]);
            q[r].y = pack4(t[4], t[5], t[6], t[7]);
            q[r].z = pack4(t[8], t[9], t[10], t[11]);
            q[r].w = pack4(t[12], t[13], t[14], t[15]);
            bs[r] = s;
        }
        d = 1.0f / iscale;
    }
}

// Q8_0 quantization (matmul_quant_pack.c:23-62, scalar rounding) of one 32-value block owned by this lane.
template <bool SIGNAL = false>
__device__ __forceinline__ void q80_quantize_block(const float *xblk, uint4 &q0, uint4 &q1, float &d, int &sum) {
    float v[32];
    ld16f(xblk, v);
    ld16f(xblk + 16, v + 16);
    if (SIGNAL) {  // see q8k_quantize_runs
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    float max_abs = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        max_abs = fmaxf(max_abs, fabsf(v[i]));
    }
    float scale = max_abs / 127.0f;
    if (scale < FLT_MIN) {
        scale = 1.0f;
    }
    const float inv = 1.0f / scale;
    int t[32];
    sum = 0;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        int z = (int)roundf(v[i] * inv);
        z = z < -127 ? -127 : (z > 127 ? 127 : z);
        t[i] = z;
        sum += z;
    }
    q0 = make_uint4(pack4(t[0], t[1], t[2], t[3]), pack4(t[4], t[5], t[6], t[7]), pack4(t[8], t[9], t[10], t[11]),
                    pack4(t[12], t[13], t[14], t[15]));
    q1 = make_uint4(pack4(t[16], t[17], t[18], t[19]), pack4(t[20], t[21], t[22], t[23]),
                    pack4(t[24], t[25], t[26], t[27]), pack4(t[28], t[29], t[30], t[31]));
    d = h2f(f2h(scale));
}

// ------------------------------------------------------------------ Q4_K x Q8_K
struct FmtQ4K {
    static constexpr int BYTES = Q4_K_BYTES;
    static constexpr int LPB = 8;  // lanes per block
    static constexpr int BPW = 8;  // blocks per wave-load
    static constexpr int BV = QK_K;
    static constexpr int ACT_DW = 11, WT_DW = 8, QUANT_TMP = 56;  // registers per lane (estimates)
    struct Act {
        uint4 lo, hi;  // int8 activations under the low / high nibbles of this lane's 16 bytes
        float d;
        int bs_lo, bs_hi;
    };
    struct Wt {
        uint4 hdr;  // d, dmin, scales[12]
        uint4 q;
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int sub) {
        const int g = sub >> 1, h = sub & 1;
        const int8_t *base = av.qs + n * av.kp + blk * QK_K + 64 * g + 16 * h;
        a.lo = *(const uint4 *)base;
        a.hi = *(const uint4 *)(base + 32);
        a.d = av.d[n * av.nb + blk];
        const int16_t *bs = av.sums + (n * av.nb + blk) * 16;
        a.bs_lo = bs[4 * g + h];
        a.bs_hi = bs[4 * g + 2 + h];
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int sub) {
        const int g = sub >> 1, h = sub & 1;
        const int off[2] = {64 * g + 16 * h, 64 * g + 32 + 16 * h};
        uint4 q[2];
        int bs[2];
        q8k_quantize_runs<2, 8, SIGNAL>(xrow + blk * QK_K, off, q, bs, a.d);
        a.lo = q[0];
        a.hi = q[1];
        a.bs_lo = bs[0];
        a.bs_hi = bs[1];
    }
    __device__ static void zero_act(Act &a) {
        a.lo = a.hi = make_uint4(0, 0, 0, 0);
        a.d = 0.0f;
        a.bs_lo = a.bs_hi = 0;
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int sub) {
        w.hdr = *(const uint4 *)blk;  // rows and blocks of Q4_K are 16-byte aligned (144 = 9 * 16)
        w.q = *(const uint4 *)(blk + 16 + 16 * sub);
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int sub) {
        const int g = sub >> 1;
        const float d = h2f((uint16_t)(w.hdr.x & 0xffffu));
        const float dmin = h2f((uint16_t)(w.hdr.x >> 16));
        // 6-bit scale / min pairs of sub-blocks 2g and 2g+1 (get_scale_min_k4, kquant_common.h:29-37), without
        // branches: for g < 2 the pair is (s[j] & 63, s[j+4] & 63); for g >= 2 the low nibbles come from s[j+4]
        // and the two high bits from s[j-4] / s[j]. All selectors below are per-lane constants.
        const int sh = 16 * (g & 1);
        const uint32_t sa = w.hdr.y >> sh;
        const uint32_t sb = w.hdr.z >> sh;
        const uint32_t sc_ = w.hdr.w >> sh;
        const bool hi_grp = g >= 2;
        const uint32_t m_lo = hi_grp ? 0x0f0fu : 0x3f3fu;
        const uint32_t m_hi = hi_grp ? 0x3030u : 0u;
        const uint32_t scp = ((hi_grp ? sc_ : sa) & m_lo) | ((sa >> 2) & m_hi);
        const uint32_t mp = ((hi_grp ? (sc_ >> 4) : sb) & m_lo) | ((sb >> 2) & m_hi);
        const int sc0 = (int)(scp & 0xffu), sc1 = (int)((scp >> 8) & 0xffu);
        const int m0 = (int)(mp & 0xffu), m1 = (int)((mp >> 8) & 0xffu);
        uint4 lo, hi;
        lo.x = w.q.x & 0x0f0f0f0fu;
        lo.y = w.q.y & 0x0f0f0f0fu;
        lo.z = w.q.z & 0x0f0f0f0fu;
        lo.w = w.q.w & 0x0f0f0f0fu;
        hi.x = (w.q.x >> 4) & 0x0f0f0f0fu;
        hi.y = (w.q.y >> 4) & 0x0f0f0f0fu;
        hi.z = (w.q.z >> 4) & 0x0f0f0f0fu;
        hi.w = (w.q.w >> 4) & 0x0f0f0f0fu;
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            const int dl = dot16(lo, a[n].lo, 0);
            const int dh = dot16(hi, a[n].hi, 0);
            const int isum = __mul24(sc0, dl) + __mul24(sc1, dh);
            const int msum = __mul24(m0, a[n].bs_lo) + __mul24(m1, a[n].bs_hi);
            acc[n] += (a[n].d * d) * (float)isum - (a[n].d * dmin) * (float)msum;
        }
    }
};

// ------------------------------------------------------------------ Q5_K x Q8_K
// The Q4_K decomposition (8 lanes per block, lane sub owns 16 bytes of qs = 16 low-nibble and 16 high-nibble values)
// plus the fifth bits: the 16 bytes of qh that belong to this lane's positions, bit 2 g for the low nibbles and bit
// 2 g + 1 for the high ones (q5k_gguf.c:162-198, vec_dot_impl.h:734-781). Blocks are 176 = 11 * 16 bytes: aligned.
struct FmtQ5K {
    static constexpr int BYTES = Q5_K_BYTES;
    static constexpr int LPB = 8;
    static constexpr int BPW = 8;
    static constexpr int BV = QK_K;
    static constexpr int ACT_DW = 11, WT_DW = 12, QUANT_TMP = 56;
    using Act = FmtQ4K::Act;
    struct Wt {
        uint4 hdr;  // d, dmin, scales[12]
        uint4 qh;
        uint4 q;
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int sub) {
        FmtQ4K::load_act(a, av, n, blk, sub);
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int sub) {
        FmtQ4K::quant_act<SIGNAL>(a, xrow, blk, sub);
    }
    __device__ static void zero_act(Act &a) {
        FmtQ4K::zero_act(a);
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int sub) {
        w.hdr = *(const uint4 *)blk;
        w.qh = *(const uint4 *)(blk + 16 + 16 * (sub & 1));
        w.q = *(const uint4 *)(blk + 48 + 16 * sub);
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int sub) {
        const int g = sub >> 1;
        const float d = h2f((uint16_t)(w.hdr.x & 0xffffu));
        const float dmin = h2f((uint16_t)(w.hdr.x >> 16));
        // scale / min pairs of sub-blocks 2g and 2g+1: as in FmtQ4K::accumulate
        const int sh = 16 * (g & 1);
        const uint32_t sa = w.hdr.y >> sh;
        const uint32_t sb = w.hdr.z >> sh;
        const uint32_t sc_ = w.hdr.w >> sh;
        const bool hi_grp = g >= 2;
        const uint32_t m_lo = hi_grp ? 0x0f0fu : 0x3f3fu;
        const uint32_t m_hi = hi_grp ? 0x3030u : 0u;
        const uint32_t scp = ((hi_grp ? sc_ : sa) & m_lo) | ((sa >> 2) & m_hi);
        const uint32_t mp = ((hi_grp ? (sc_ >> 4) : sb) & m_lo) | ((sb >> 2) & m_hi);
        const int sc0 = (int)(scp & 0xffu), sc1 = (int)((scp >> 8) & 0xffu);
        const int m0 = (int)(mp & 0xffu), m1 = (int)((mp >> 8) & 0xffu);
        const int b0 = 2 * g;  // bit of the low-nibble values; b0 + 1: of the high-nibble values
        uint4 lo, hi;
#define MH_Q5_UNPACK(c)                                                                                                \
    lo.c = (w.q.c & 0x0f0f0f0fu) | (((w.qh.c >> b0) & 0x01010101u) << 4);                                              \
    hi.c = ((w.q.c >> 4) & 0x0f0f0f0fu) | (((w.qh.c >> (b0 + 1)) & 0x01010101u) << 4);
        MH_Q5_UNPACK(x)
        MH_Q5_UNPACK(y)
        MH_Q5_UNPACK(z)
        MH_Q5_UNPACK(w)
#undef MH_Q5_UNPACK
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            const int dl = dot16(lo, a[n].lo, 0);
            const int dh = dot16(hi, a[n].hi, 0);
            const int isum = __mul24(sc0, dl) + __mul24(sc1, dh);
            const int msum = __mul24(m0, a[n].bs_lo) + __mul24(m1, a[n].bs_hi);
            acc[n] += (a[n].d * d) * (float)isum - (a[n].d * dmin) * (float)msum;
        }
    }
};

// ------------------------------------------------------------------ Q6_K x Q8_K
struct FmtQ6K {
    static constexpr int BYTES = Q6_K_BYTES;
    static constexpr int LPB = 4;
    static constexpr int BPW = 16;
    static constexpr int BV = QK_K;
    static constexpr int ACT_DW = 21, WT_DW = 15, QUANT_TMP = 100;
    struct Act {
        uint4 a[4];  // 16 int8 each, under q1..q4 of this lane's 16 positions
        float d;
        int bs[4];
    };
    struct Wt {
        uint4 ql0, ql1, qh;
        uint2 sc;  // the 8 int8 scales of this lane's half
        uint16_t d;
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int sub) {
        const int hh = sub >> 1, t = sub & 1;
        const int8_t *base = av.qs + n * av.kp + blk * QK_K + 128 * hh + 16 * t;
        const int16_t *bs = av.sums + (n * av.nb + blk) * 16 + 8 * hh + t;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a.a[j] = *(const uint4 *)(base + 32 * j);
            a.bs[j] = bs[2 * j];
        }
        a.d = av.d[n * av.nb + blk];
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int sub) {
        const int hh = sub >> 1, t = sub & 1;
        const int base = 128 * hh + 16 * t;
        const int off[4] = {base, base + 32, base + 64, base + 96};
        q8k_quantize_runs<4, 4, SIGNAL>(xrow + blk * QK_K, off, a.a, a.bs, a.d);
    }
    __device__ static void zero_act(Act &a) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a.a[j] = make_uint4(0, 0, 0, 0);
            a.bs[j] = 0;
        }
        a.d = 0.0f;
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int sub) {
        const int hh = sub >> 1, t = sub & 1;
        // 210-byte blocks are only 2-byte aligned: the hardware's unaligned global loads are used
        w.ql0 = ld16(blk + 64 * hh + 16 * t);
        w.ql1 = ld16(blk + 64 * hh + 32 + 16 * t);
        w.qh = ld16(blk + 128 + 32 * hh + 16 * t);
        w.sc = ld8(blk + 192 + 8 * hh);
        w.d = ld2(blk + 208);
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int sub) {
        const int t = sub & 1;
        const float d = h2f(w.d);
        // scales t, t+2, t+4, t+6 of this half (is = l/16 = t; q1..q4 use is+0,2,4,6: q6k_gguf.c:63-99)
        const uint32_t s01 = w.sc.x >> (8 * t);  // bytes t, (t+2 at bit 16)
        const uint32_t s23 = w.sc.y >> (8 * t);
        const int sc0 = (int)(int8_t)(s01 & 0xff);
        const int sc1 = (int)(int8_t)((s01 >> 16) & 0xff);
        const int sc2 = (int)(int8_t)(s23 & 0xff);
        const int sc3 = (int)(int8_t)((s23 >> 16) & 0xff);
        // 6-bit values 0..63 (the -32 offset is applied through the activation group sums)
        uint4 q1, q2, q3, q4;
#define MH_Q6_UNPACK(c)                                                                                                \
    q1.c = (w.ql0.c & 0x0f0f0f0fu) | ((w.qh.c << 4) & 0x30303030u);                                                    \
    q2.c = (w.ql1.c & 0x0f0f0f0fu) | ((w.qh.c << 2) & 0x30303030u);                                                    \
    q3.c = ((w.ql0.c >> 4) & 0x0f0f0f0fu) | (w.qh.c & 0x30303030u);                                                    \
    q4.c = ((w.ql1.c >> 4) & 0x0f0f0f0fu) | ((w.qh.c >> 2) & 0x30303030u);
        MH_Q6_UNPACK(x)
        MH_Q6_UNPACK(y)
        MH_Q6_UNPACK(z)
        MH_Q6_UNPACK(w)
#undef MH_Q6_UNPACK
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            const int d1 = dot16(q1, a[n].a[0], 0) - 32 * a[n].bs[0];
            const int d2 = dot16(q2, a[n].a[1], 0) - 32 * a[n].bs[1];
            const int d3 = dot16(q3, a[n].a[2], 0) - 32 * a[n].bs[2];
            const int d4 = dot16(q4, a[n].a[3], 0) - 32 * a[n].bs[3];
            const int isum = __mul24(sc0, d1) + __mul24(sc1, d2) + __mul24(sc2, d3) + __mul24(sc3, d4);
            acc[n] += (a[n].d * d) * (float)isum;
        }
    }
};

// ------------------------------------------------------------------ Q2_K, Q3_K x Q8_K
// The Q6_K decomposition (4 lanes per block; lane (hh, t) owns 16 bytes of qs = positions 16 t .. 16 t + 15 of the four
// 32-value rows j = 0..3 of half hh, i.e. groups 8 hh + 2 j + t) and the Q6_K activation registers.
// Q2_K (q2k_gguf.c:113-149, vec_dot_impl.h:565-618): two-bit values, group scale / min in one byte.
struct FmtQ2K {
    static constexpr int BYTES = Q2_K_BYTES;
    static constexpr int LPB = 4;
    static constexpr int BPW = 16;
    static constexpr int BV = QK_K;
    static constexpr int ACT_DW = 21, WT_DW = 7, QUANT_TMP = 100;
    using Act = FmtQ6K::Act;
    struct Wt {
        uint4 q;
        uint2 sc;     // the 8 scale bytes of this lane's half
        uint32_t dd;  // d | dmin << 16
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int sub) {
        FmtQ6K::load_act(a, av, n, blk, sub);
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int sub) {
        FmtQ6K::quant_act<SIGNAL>(a, xrow, blk, sub);
    }
    __device__ static void zero_act(Act &a) {
        FmtQ6K::zero_act(a);
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int sub) {
        const int hh = sub >> 1, t = sub & 1;
        w.sc = ld8(blk + 8 * hh);  // blocks are 4-byte aligned
        w.q = ld16(blk + 16 + 32 * hh + 16 * t);
        w.dd = ld4(blk + 80);
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int sub) {
        const int t = sub & 1;
        const float d = h2f((uint16_t)(w.dd & 0xffffu));
        const float dmin = h2f((uint16_t)(w.dd >> 16));
        const uint32_t s01 = w.sc.x >> (8 * t);  // groups t (bits 0..7) and t + 2 (bits 16..23)
        const uint32_t s23 = w.sc.y >> (8 * t);
        const int sc[4] = {(int)(s01 & 0xf), (int)((s01 >> 16) & 0xf), (int)(s23 & 0xf), (int)((s23 >> 16) & 0xf)};
        const int mn[4] = {(int)((s01 >> 4) & 0xf), (int)((s01 >> 20) & 0xf), (int)((s23 >> 4) & 0xf),
                           (int)((s23 >> 20) & 0xf)};
        uint4 q[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            q[j].x = (w.q.x >> (2 * j)) & 0x03030303u;
            q[j].y = (w.q.y >> (2 * j)) & 0x03030303u;
            q[j].z = (w.q.z >> (2 * j)) & 0x03030303u;
            q[j].w = (w.q.w >> (2 * j)) & 0x03030303u;
        }
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            int isum = 0, msum = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                isum += __mul24(sc[j], dot16(q[j], a[n].a[j], 0));
                msum += __mul24(mn[j], a[n].bs[j]);
            }
            acc[n] += (a[n].d * d) * (float)isum - (a[n].d * dmin) * (float)msum;
        }
    }
};

// Q3_K (q3k_gguf.c:126-175, vec_dot_impl.h:620-687): Q2_K's two-bit layout plus a high bit per value in hmask
// (bit 4 hh + j of hmask[l]); value = (q2 | high << 2) - 4, six-bit group scales offset by 32, no minimum.
struct FmtQ3K {
    static constexpr int BYTES = Q3_K_BYTES;
    static constexpr int LPB = 4;
    static constexpr int BPW = 16;
    static constexpr int BV = QK_K;
    static constexpr int ACT_DW = 21, WT_DW = 12, QUANT_TMP = 100;
    using Act = FmtQ6K::Act;
    struct Wt {
        uint4 q, hm;
        uint32_t s0, s1, s2;  // the 12 scale bytes
        uint16_t d;
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int sub) {
        FmtQ6K::load_act(a, av, n, blk, sub);
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int sub) {
        FmtQ6K::quant_act<SIGNAL>(a, xrow, blk, sub);
    }
    __device__ static void zero_act(Act &a) {
        FmtQ6K::zero_act(a);
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int sub) {
        const int hh = sub >> 1, t = sub & 1;
        // 110-byte blocks are only 2-byte aligned
        w.hm = ld16(blk + 16 * t);
        w.q = ld16(blk + 32 + 32 * hh + 16 * t);
        w.s0 = ld4(blk + 96);
        w.s1 = ld4(blk + 100);
        w.s2 = ld4(blk + 104);
        w.d = ld2(blk + 108);
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int sub) {
        const int hh = sub >> 1, t = sub & 1;
        const float d = h2f(w.d);
        // group is = 8 hh + 2 j + t: low nibble from byte is % 8 of (s0, s1) (high nibble for hh = 1), the two high
        // bits from byte is % 4 of s2 at bit 2 (is / 4)
        int sc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int is8 = 2 * j + t;  // is % 8
            const uint32_t lo_word = is8 < 4 ? w.s0 : w.s1;
            const uint32_t low = (lo_word >> (8 * (is8 & 3) + 4 * hh)) & 0xfu;
            const uint32_t high = (w.s2 >> (8 * (is8 & 3) + 2 * (2 * hh + (is8 >> 2)))) & 3u;
            sc[j] = (int)(low | (high << 4)) - 32;
        }
        uint4 q[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int hb = 4 * hh + j;  // bit of hmask; moved to bit 2 of each byte
#define MH_Q3_UNPACK(c)                                                                                                \
    q[j].c = ((w.q.c >> (2 * j)) & 0x03030303u) | ((((w.hm.c >> hb) & 0x01010101u)) << 2);
            MH_Q3_UNPACK(x)
            MH_Q3_UNPACK(y)
            MH_Q3_UNPACK(z)
            MH_Q3_UNPACK(w)
#undef MH_Q3_UNPACK
        }
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            int isum = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                isum += __mul24(sc[j], dot16(q[j], a[n].a[j], 0) - 4 * a[n].bs[j]);
            }
            acc[n] += (a[n].d * d) * (float)isum;
        }
    }
};

// ------------------------------------------------------------------ Q8_0, Q8_1 x Q8_0
// HDR: bytes in front of the 32 int8 values: the fp16 scale (Q8_0), or the scale and the fp16 sum that Q8_1 carries
// and neither the dequantizer nor the dot uses (q8_gguf.c:202-213, vec_dot_impl.h:481-510).
template <int HDR>
struct FmtQ8x {
    static constexpr int BYTES = HDR + 32;
    static constexpr int LPB = 1;
    static constexpr int BPW = 64;
    static constexpr int BV = QK;
    static constexpr int ACT_DW = 9, WT_DW = 9, QUANT_TMP = 80;
    struct Act {
        uint4 a0, a1;
        float d;
    };
    struct Wt {
        uint4 q0, q1;
        uint16_t s;
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int) {
        const int8_t *base = av.qs + n * av.kp + blk * QK;
        a.a0 = *(const uint4 *)base;
        a.a1 = *(const uint4 *)(base + 16);
        a.d = av.d[n * av.nb + blk];
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int) {
        int sum;
        q80_quantize_block<SIGNAL>(xrow + blk * QK, a.a0, a.a1, a.d, sum);
    }
    __device__ static void zero_act(Act &a) {
        a.a0 = a.a1 = make_uint4(0, 0, 0, 0);
        a.d = 0.0f;
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int) {
        w.s = ld2(blk);
        w.q0 = ld16(blk + HDR);
        w.q1 = ld16(blk + HDR + 16);
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int) {
        const float sw = h2f(w.s);
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            int isum = dot16(w.q0, a[n].a0, 0);
            isum = dot16(w.q1, a[n].a1, isum);
            acc[n] += (float)isum * (sw * a[n].d);  // vec_dot_impl.h:452-479
        }
    }
};

using FmtQ80 = FmtQ8x<2>;
using FmtQ81 = FmtQ8x<4>;
static_assert(FmtQ80::BYTES == Q8_0_BYTES && FmtQ81::BYTES == Q8_1_BYTES, "layouts");

// ------------------------------------------------------------------ Q4_0 x Q8_0
struct FmtQ40 {
    static constexpr int BYTES = Q4_0_BYTES;
    static constexpr int LPB = 1;
    static constexpr int BPW = 64;
    static constexpr int BV = QK;
    static constexpr int ACT_DW = 10, WT_DW = 5, QUANT_TMP = 80;
    struct Act {
        uint4 a0, a1;
        float d;
        int sum;
    };
    struct Wt {
        uint4 q;
        uint16_t s;
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int) {
        const int8_t *base = av.qs + n * av.kp + blk * QK;
        a.a0 = *(const uint4 *)base;
        a.a1 = *(const uint4 *)(base + 16);
        a.d = av.d[n * av.nb + blk];
        a.sum = av.sums[n * av.nb + blk];
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int) {
        q80_quantize_block<SIGNAL>(xrow + blk * QK, a.a0, a.a1, a.d, a.sum);
    }
    __device__ static void zero_act(Act &a) {
        a.a0 = a.a1 = make_uint4(0, 0, 0, 0);
        a.d = 0.0f;
        a.sum = 0;
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int) {
        w.s = ld2(blk);
        w.q = ld16(blk + 2);
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int) {
        const float sw = h2f(w.s);
        uint4 lo, hi;
        lo.x = w.q.x & 0x0f0f0f0fu;
        lo.y = w.q.y & 0x0f0f0f0fu;
        lo.z = w.q.z & 0x0f0f0f0fu;
        lo.w = w.q.w & 0x0f0f0f0fu;
        hi.x = (w.q.x >> 4) & 0x0f0f0f0fu;
        hi.y = (w.q.y >> 4) & 0x0f0f0f0fu;
        hi.z = (w.q.z >> 4) & 0x0f0f0f0fu;
        hi.w = (w.q.w >> 4) & 0x0f0f0f0fu;
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            int isum = dot16(lo, a[n].a0, 0);
            isum = dot16(hi, a[n].a1, isum);
            isum -= 8 * a[n].sum;  // (q - 8) . a
            acc[n] += (float)isum * (sw * a[n].d);  // vec_dot_impl.h:157-186
        }
    }
};

// ------------------------------------------------------------------ Q4_1, Q5_0, Q5_1 x Q8_0
// The Q4_0 decomposition (one lane per 32-value block). HAS_MIN: the block carries a minimum, values are unsigned and
// the dot adds min * scale_a * sum(a) (vec_dot_impl.h:186-217, 317-349); otherwise (Q5_0) values are centred by 16
// (:288-315). FIVE: a fifth bit per value in 32 bits of qh, bit j for value j (low nibbles are values 0..15).
template <bool HAS_MIN, bool FIVE>
struct FmtLegacy {
    static constexpr int QH_OFF = HAS_MIN ? 4 : 2;
    static constexpr int QS_OFF = QH_OFF + (FIVE ? 4 : 0);
    static constexpr int BYTES = QS_OFF + 16;
    static constexpr int LPB = 1;
    static constexpr int BPW = 64;
    static constexpr int BV = QK;
    static constexpr int ACT_DW = 10, WT_DW = 7, QUANT_TMP = 80;
    using Act = FmtQ40::Act;
    struct Wt {
        uint4 q;
        uint32_t qh;
        uint16_t s, m;
    };
    __device__ static void load_act(Act &a, const ActView &av, size_t n, size_t blk, int sub) {
        FmtQ40::load_act(a, av, n, blk, sub);
    }
    template <bool SIGNAL = false>
    __device__ static void quant_act(Act &a, const float *xrow, size_t blk, int sub) {
        FmtQ40::quant_act<SIGNAL>(a, xrow, blk, sub);
    }
    __device__ static void zero_act(Act &a) {
        FmtQ40::zero_act(a);
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int) {
        w.s = ld2(blk);
        w.m = HAS_MIN ? ld2(blk + 2) : (uint16_t)0;
        w.qh = FIVE ? ((uint32_t)ld2(blk + QH_OFF) | ((uint32_t)ld2(blk + QH_OFF + 2) << 16)) : 0u;
        w.q = ld16(blk + QS_OFF);
    }
    // bits 0..3 of nib to bit 4 of bytes 0..3 (0x00204081 = 1 + 2^7 + 2^14 + 2^21 moves bit i to bit 8 i; no carries)
    __device__ static uint32_t fifth(uint32_t qh, int shift) {
        return ((((qh >> shift) & 0xfu) * 0x00204081u) & 0x01010101u) << 4;
    }
    template <int NC>
    __device__ static void accumulate(const Wt &w, const Act (&a)[NC], float (&acc)[NC], int) {
        const float sw = h2f(w.s);
        const float mw = h2f(w.m);
        uint4 lo, hi;
        lo.x = w.q.x & 0x0f0f0f0fu;
        lo.y = w.q.y & 0x0f0f0f0fu;
        lo.z = w.q.z & 0x0f0f0f0fu;
        lo.w = w.q.w & 0x0f0f0f0fu;
        hi.x = (w.q.x >> 4) & 0x0f0f0f0fu;
        hi.y = (w.q.y >> 4) & 0x0f0f0f0fu;
        hi.z = (w.q.z >> 4) & 0x0f0f0f0fu;
        hi.w = (w.q.w >> 4) & 0x0f0f0f0fu;
        if constexpr (FIVE) {
            lo.x |= fifth(w.qh, 0);
            lo.y |= fifth(w.qh, 4);
            lo.z |= fifth(w.qh, 8);
            lo.w |= fifth(w.qh, 12);
            hi.x |= fifth(w.qh, 16);
            hi.y |= fifth(w.qh, 20);
            hi.z |= fifth(w.qh, 24);
            hi.w |= fifth(w.qh, 28);
        }
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            int isum = dot16(lo, a[n].a0, 0);
            isum = dot16(hi, a[n].a1, isum);
            if constexpr (HAS_MIN) {
                acc[n] += (sw * a[n].d) * (float)isum + (mw * a[n].d) * (float)a[n].sum;
            } else {
                isum -= 16 * a[n].sum;  // (q - 16) . a
                acc[n] += (float)isum * (sw * a[n].d);
            }
        }
    }
};
using FmtQ41 = FmtLegacy<true, false>;
using FmtQ50 = FmtLegacy<false, true>;
using FmtQ51 = FmtLegacy<true, true>;
static_assert(FmtQ41::BYTES == Q4_1_BYTES && FmtQ50::BYTES == Q5_0_BYTES && FmtQ51::BYTES == Q5_1_BYTES, "layouts");

struct MatvecParams {
    const uint8_t *w[3];  // weights of one shape sharing the activations; blockIdx.y selects one
    void *out[3];
    ActView act;       // packed activations (prepacked variant)
    const float *x;    // fp32 activations [N][K] (fused variant)
    size_t K;
    const void *bias[3];
    int bias_is_f16;
    int bias_first;    // fp16 output: f16(dot + bias) instead of f16(f16(dot) + bias)
    int out_is_f16;
    size_t n0;         // first activation row of this column tile
    size_t M;
    size_t nb;         // blocks per weight row
    size_t row_bytes;
    int rows_per_wg;
    // grouped (MoE) mode: blockIdx.z selects a work item = up to NC consecutive routes of one expert
    const int4 *items;            // (expert, first route, route count, -) or nullptr
    const int *n_items;           // number of valid items (device memory)
    const uint32_t *act_index;    // packed-activation row of each route (token id), or nullptr = identity
    size_t expert_stride;         // bytes between the experts' weight slices
};

// out / bias: this launch's entries of p.out / p.bias, fetched by the caller before the final barrier (two scalar
// loads whose latency would otherwise sit, one after the other, between the reduction and the store)
__device__ __forceinline__ void store_out(const MatvecParams &p, void *out, const void *bias, size_t n, size_t row,
                                          float v) {
    const size_t idx = n * p.M + row;
    float b = 0.0f;
    if (bias != nullptr) {
        b = p.bias_is_f16 ? h2f(((const uint16_t *)bias)[row]) : ((const float *)bias)[row];
    }
    if (!p.out_is_f16) {
        ((float *)out)[idx] = bias != nullptr ? v + b : v;
    } else if (p.bias_first) {
        // q/k/v projection: the fp32 accumulator starts from the bias, one rounding at the store
        ((uint16_t *)out)[idx] = f2h(bias != nullptr ? v + b : v);
    } else {
        // matmul: store f16(dot), then the epilogue adds the bias to the stored f16 value
        uint16_t h = f2h(v);
        if (bias != nullptr) {
            h = f2h(h2f(h) + b);
        }
        ((uint16_t *)out)[idx] = h;
    }
}

// Largest workgroup a configuration may use: the register estimate decides how many wavefronts fit per SIMD
// (512 VGPRs per lane per SIMD on gfx950) without spilling.
template <class Fmt, int NC, int C, int R, bool FUSED>
constexpr int matvec_max_threads() {
    constexpr int loop_need = NC * C * Fmt::ACT_DW + 2 * R * C * Fmt::WT_DW + 2 * NC + 36;
    constexpr int prologue_need = NC * C * Fmt::ACT_DW + (FUSED ? Fmt::QUANT_TMP : 0) + 24;
    constexpr int need = loop_need > prologue_need ? loop_need : prologue_need;
    return need <= 120 ? 1024 : (need <= 240 ? 512 : 256);
}

// FUSED: quantize fp32 activations in the prologue instead of reading packed ones.
// EXACT: every lane owns a real block in every slot and M is a multiple of rows_per_wg (no masking in the loop).
template <class Fmt, int NC, int C, int R, bool FUSED, bool EXACT>
__global__ __launch_bounds__((matvec_max_threads<Fmt, NC, C, R, FUSED>())) void k_matvec(const MatvecParams p) {
    extern __shared__ float partial[];  // [rows_per_wg][NC][4 * W]: one partial per 16-lane row of each wavefront
    warm_kernel_arguments<sizeof(MatvecParams), sizeof(MatvecParams)>();
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int W = blockDim.x >> 6;
    const int sub = lane % Fmt::LPB;
    const uint8_t *__restrict__ wbase = p.w[blockIdx.y];
    size_t n0 = p.n0;
    int ncols = NC;
    if (!FUSED && p.items != nullptr) {
        if ((int)blockIdx.z >= *p.n_items) {
            return;  // uniform for the whole workgroup
        }
        const int4 it = p.items[blockIdx.z];
        wbase += (size_t)it.x * p.expert_stride;
        n0 = (size_t)it.y;
        ncols = it.z;
    }

    typename Fmt::Act act[C][NC];
    size_t blk[C];
    bool valid[C];
#pragma unroll
    for (int i = 0; i < C; ++i) {
        blk[i] = (size_t)(wave * C + i) * Fmt::BPW + lane / Fmt::LPB;
        valid[i] = EXACT || blk[i] < p.nb;
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            if (valid[i] && n < ncols) {
                if constexpr (FUSED) {
                    Fmt::quant_act(act[i][n], p.x + (n0 + n) * p.K, blk[i], sub);
                } else {
                    const size_t arow = p.act_index != nullptr ? (size_t)p.act_index[n0 + n] : n0 + n;
                    Fmt::load_act(act[i][n], p.act, arow, blk[i], sub);
                }
            } else {
                Fmt::zero_act(act[i][n]);
            }
        }
    }

    const size_t row0 = (size_t)blockIdx.x * p.rows_per_wg;
    const int pslot = wave * 4 + (lane >> 4);
    const int pstride = 4 * W;

    // Two register buffers of R rows each: the loads of the next R rows are in flight while the current R rows
    // are consumed, so a wavefront keeps requests outstanding for its whole lifetime.
    typename Fmt::Wt wa[R][C], wb[R][C];
    auto issue = [&](typename Fmt::Wt(&wt)[R][C], int r) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            size_t row = row0 + r + rr;
            if (!EXACT && row >= p.M) {
                row = p.M - 1;  // harmless re-read; the result is discarded in the epilogue
            }
            const uint8_t *rowp = wbase + row * p.row_bytes;
#pragma unroll
            for (int i = 0; i < C; ++i) {
                if (valid[i]) {
                    Fmt::load_w(wt[rr][i], rowp + blk[i] * Fmt::BYTES, sub);
                }
            }
        }
    };
    auto consume = [&](const typename Fmt::Wt(&wt)[R][C], int r) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float acc[NC];
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                acc[n] = 0.0f;
            }
#pragma unroll
            for (int i = 0; i < C; ++i) {
                if (valid[i]) {
                    Fmt::template accumulate<NC>(wt[rr][i], act[i], acc, sub);
                }
            }
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                const float s = row16_sum(acc[n]);
                if ((lane & 15) == 0) {
                    partial[((r + rr) * NC + n) * pstride + pslot] = s;
                }
            }
        }
    };
    const int rows = p.rows_per_wg;  // a multiple of R
    issue(wa, 0);
    for (int r = 0; r < rows; r += 2 * R) {
        if (r + R < rows) {
            issue(wb, r + R);
        }
        consume(wa, r);
        if (r + 2 * R < rows) {
            issue(wa, r + 2 * R);
        }
        if (r + R < rows) {
            consume(wb, r + R);
        }
    }
    void *const out = p.out[blockIdx.y];
    const void *const bias = p.bias[blockIdx.y];
    asm volatile("" ::"s"(out), "s"(bias));  // keeps the two loads in front of the barrier
    __syncthreads();
    for (int idx = threadIdx.x; idx < p.rows_per_wg * NC; idx += blockDim.x) {
        const size_t row = row0 + idx / NC;
        const int n = idx % NC;
        if ((EXACT || row < p.M) && n < ncols) {
            // W <= 16 float4 partials, all read before the first add so that only one LDS latency is exposed
            const float4 *pv = (const float4 *)(partial + idx * pstride);
            float4 v[16];
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                v[w] = pv[w < W ? w : 0];
            }
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                const float t = (v[w].x + v[w].y) + (v[w].z + v[w].w);
                s += w < W ? t : 0.0f;
            }
            store_out(p, out, bias, n0 + n, row, s);
        }
    }
}

// ------------------------------------------------------------------ loader / consumer variant (rows of an even number of bytes)
// Same arithmetic, lane mapping and reduction order as k_matvec, but the weights take the way global -> LDS ->
// registers and the wavefronts are specialised: W consumers quantize the activations, read weight rows from an LDS
// ring and compute; one loader copies the workgroup's rows (contiguous in memory) into the ring with direct-to-LDS
// loads, R rows per step, every stage of the ring requested before the consumers have finished the activation
// prologue. In k_matvec a wavefront that wants to issue the loads of its next rows is held at the issue stage while
// the memory queues of the CU are full (under a saturated HBM: most of the time) and cannot compute on the rows it
// already has; measured with the cycle counter, its life is 20 % activation prologue, 40 % load issue, 27 % compute,
// 10 % reduction, one after the other. Here the loader absorbs the issue stalls and the prologue overlaps the first
// loads. Steps are separated by a bare s_barrier (no implied memory wait).
typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef const __attribute__((address_space(1))) uint8_t glb_u8;
constexpr int MV_LS_STAGES = 3;

// Consumers per workgroup: up to 8 for Q4_K (one wave-load = 8 blocks of 256), up to 4 for the other formats, whose
// wave-loads are wider and whose kernels need more registers per lane (the bound decides the register budget).
template <class Fmt>
constexpr int matvec_ls_max_consumers() {
    return Fmt::LPB == 8 ? 8 : 4;
}

// ALIGNED: every row is a multiple of 16 bytes. The steps are then whole 16-byte chunks from their first byte on and
// the loader's loop holds nothing but the direct-to-LDS loads; the general form (a lead of up to 14 bytes per step,
// the tensor's last bytes through registers) costs the aligned formats 10 - 17 % (14336 x 4096: Q5_K 11.2 -> 13.1 us,
// Q4_1 9.8 -> 11.2 us), so both are instantiated and the launcher picks.
template <class Fmt, int NC, int C, int R, bool FUSED, bool ALIGNED>
__global__ __launch_bounds__((matvec_ls_max_consumers<Fmt>() + 1) * 64) void k_matvec_ls(const MatvecParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    warm_kernel_arguments<offsetof(MatvecParams, items), sizeof(MatvecParams)>();  // the grouped-mode fields behind it are never read here
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int W = (int)(blockDim.x >> 6) - 1;  // consumers
    const bool loader = wave == W;
    const int sub = lane % Fmt::LPB;
    const uint8_t *__restrict__ wbase = p.w[blockIdx.y];
    void *const out = p.out[blockIdx.y];
    const void *const bias = p.bias[blockIdx.y];
    asm volatile("" ::"s"(out), "s"(bias));  // fetched here, not between the reduction and the store
    const size_t n0 = p.n0;
    const size_t row0 = (size_t)blockIdx.x * p.rows_per_wg;
    const int rows = p.rows_per_wg;  // a multiple of R
    const int load_steps = rows / R;
    // LDS: [partial sums: rows x NC x 4W floats][ring: STAGES x stage_stride bytes]
    float *partial = (float *)lds_raw;
    const int pstride = 4 * W;
    const uint32_t stage_bytes = (uint32_t)(R * p.row_bytes);
    // Rows need not be multiples of 16 bytes: a step is copied from the 16-byte boundary below its first row (`lead`
    // bytes early, rows of a workgroup are contiguous in memory) and read `lead` bytes into its stage.
    const uint32_t stage_stride = (stage_bytes + (ALIGNED ? 0u : 15u) + 1023u) & ~1023u;
    uint8_t *ring = lds_raw + (((size_t)rows * NC * pstride * sizeof(float) + 15) & ~(size_t)15);

    if (loader) {
        const int chunks = (int)(stage_stride >> 10);  // direct-to-LDS instructions per step (1 KiB each)
        // Some step is cut short (rows beyond M), or the tensor ends inside this workgroup off a 16-byte boundary (its
        // last chunk then comes through registers): the loads in flight are not whole steps of `chunks` instructions.
        const bool ragged = row0 + rows > p.M || (!ALIGNED && row0 + rows == p.M && ((p.M * p.row_bytes) & 15) != 0);
        int step_loads[MV_LS_STAGES];  // direct-to-LDS instructions of the step in each stage (general form only)
        auto issue_step = [&](int t) {
            const size_t r = row0 + (size_t)t * R;
            uint32_t valid = stage_bytes;  // bytes of this step that exist (rows beyond M are not read)
            if (r + R > p.M) {
                valid = r < p.M ? (uint32_t)((p.M - r) * p.row_bytes) : 0u;
            }
            if constexpr (ALIGNED) {
                const uint8_t *src = wbase + r * p.row_bytes;
                uint8_t *dst = ring + (size_t)(t % MV_LS_STAGES) * stage_stride;
                for (int c = 0; c < chunks; ++c) {
                    const uint32_t off = (uint32_t)c * 1024u + (uint32_t)lane * 16u;
                    if (off < valid) {
                        __builtin_amdgcn_global_load_lds((glb_u8 *)(src + off), (lds_u8 *)(dst + c * 1024), 16, 0, 0);
                    }
                }
                return;
            }
            const size_t first = r * p.row_bytes;
            const uint32_t lead = (uint32_t)(first & 15);
            const uint8_t *src = wbase + (first - lead);
            valid = valid != 0 ? valid + lead : 0u;
            // bytes of the tensor from src on: a chunk that would end behind the tensor (its size need not be a multiple
            // of 16) is brought two bytes at a time, only the bytes that exist
            const size_t left = p.M * p.row_bytes - (first - lead);
            uint8_t *dst = ring + (size_t)(t % MV_LS_STAGES) * stage_stride;
            step_loads[t % MV_LS_STAGES] = (int)((valid + 1023u) >> 10);  // chunks that hold a byte of the step
            for (int c = 0; c < chunks; ++c) {
                const uint32_t off = (uint32_t)c * 1024u + (uint32_t)lane * 16u;
                if (off < valid) {
                    if ((size_t)off + 16 <= left) {
                        __builtin_amdgcn_global_load_lds((glb_u8 *)(src + off), (lds_u8 *)(dst + c * 1024), 16, 0, 0);
                    } else {
                        for (uint32_t e = 0; e < 16u && (size_t)off + e < left; e += 2u) {
                            *(uint16_t *)(dst + off + e) = *(const uint16_t *)(src + off + e);
                        }
                    }
                }
            }
        };
        // every stage is free at the start: all of them are requested while the consumers prepare the activations;
        // with fused quantization, after the consumers have issued their first activation loads
        if (FUSED) {
            __builtin_amdgcn_s_barrier();
        }
        for (int t = 0; t < MV_LS_STAGES && t < load_steps; ++t) {
            issue_step(t);
        }
        for (int b = 0; b < load_steps; ++b) {
            // Loads complete in order: step b has landed once at most the loads of the steps issued after it are
            // outstanding. Steps up to b + STAGES - 2 have been issued here (all STAGES of them when b == 0).
            int newer = (b == 0 ? MV_LS_STAGES - 1 : MV_LS_STAGES - 2);
            if (newer > load_steps - 1 - b) {
                newer = load_steps - 1 - b;
            }
            int in_flight = newer * chunks;  // instructions of the steps issued after step b
            if constexpr (!ALIGNED) {
                in_flight = 0;
                for (int k2 = 1; k2 <= newer; ++k2) {
                    in_flight += step_loads[(b + k2) % MV_LS_STAGES];
                }
            }
            wait_vmcnt_at_most(ragged ? 0 : in_flight);
            __builtin_amdgcn_s_barrier();  // barrier b: step b may be read; the consumers are done with step b - 1
            if (b >= 1 && b + MV_LS_STAGES - 1 < load_steps) {
                issue_step(b + MV_LS_STAGES - 1);  // into the stage of step b - 1
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __builtin_amdgcn_s_barrier();  // final barrier: partial sums complete
    } else {
        typename Fmt::Act act[C][NC];
        size_t blk[C];
        bool valid[C];
#pragma unroll
        for (int i = 0; i < C; ++i) {
            blk[i] = (size_t)(wave * C + i) * Fmt::BPW + lane / Fmt::LPB;
            valid[i] = blk[i] < p.nb;
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                if constexpr (FUSED) {
                    // wave-load 0 of a consumer is never empty (W is the number of wave-loads that hold blocks, and
                    // lanes beyond nb clamp to the last block), so every consumer signals exactly once
                    if (i == 0 && n == 0) {
                        const size_t bq = valid[i] ? blk[i] : p.nb - 1;
                        Fmt::template quant_act<true>(act[i][n], p.x + (n0 + n) * p.K, bq, sub);
                        if (!valid[i]) {
                            Fmt::zero_act(act[i][n]);
                        }
                    } else if (valid[i]) {
                        Fmt::quant_act(act[i][n], p.x + (n0 + n) * p.K, blk[i], sub);
                    } else {
                        Fmt::zero_act(act[i][n]);
                    }
                } else if (valid[i]) {
                    Fmt::load_act(act[i][n], p.act, n0 + n, blk[i], sub);
                } else {
                    Fmt::zero_act(act[i][n]);
                }
            }
        }
        const int pslot = wave * 4 + (lane >> 4);
        for (int b = 0; b < load_steps; ++b) {
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the previous stage has been read before it is reused
            __builtin_amdgcn_s_barrier();        // barrier b
            const uint8_t *stage = ring + (size_t)(b % MV_LS_STAGES) * stage_stride +
                                   (ALIGNED ? 0 : (((row0 + (size_t)b * R) * p.row_bytes) & 15));  // the step's first row
            typename Fmt::Wt wt[R][C];
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
#pragma unroll
                for (int i = 0; i < C; ++i) {
                    if (valid[i]) {
                        Fmt::load_w(wt[rr][i], stage + (size_t)rr * p.row_bytes + blk[i] * Fmt::BYTES, sub);
                    }
                }
            }
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                float acc[NC];
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    acc[n] = 0.0f;
                }
#pragma unroll
                for (int i = 0; i < C; ++i) {
                    if (valid[i]) {
                        Fmt::template accumulate<NC>(wt[rr][i], act[i], acc, sub);
                    }
                }
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    const float sum = row16_sum(acc[n]);
                    if ((lane & 15) == 0) {
                        partial[((b * R + rr) * NC + n) * pstride + pslot] = sum;
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();  // final barrier: partial sums complete
    }
    for (int idx = threadIdx.x; idx < rows * NC; idx += blockDim.x) {
        const size_t row = row0 + idx / NC;
        const int n = idx % NC;
        if (row < p.M) {
            // W <= 8 float4 partials, all read before the first add so that only one LDS latency is exposed
            const float4 *pv = (const float4 *)(partial + idx * pstride);
            float4 v[8];
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                v[w] = pv[w < W ? w : 0];
            }
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                const float t = (v[w].x + v[w].y) + (v[w].z + v[w].w);
                sum += w < W ? t : 0.0f;
            }
            store_out(p, out, bias, n0 + n, row, sum);
        }
    }
}

// rows whose bytes can be copied as 16-byte chunks: base address a multiple of 16, even row pitch, at most 8 K slices
template <class Fmt>
static bool matvec_ls_usable(const marmot_hip_device *dev, const MatvecParams &p, size_t K, int C) {
    const size_t nb = (K + Fmt::BV - 1) / Fmt::BV;
    const size_t wave_loads = (nb + Fmt::BPW - 1) / Fmt::BPW;
    return p.items == nullptr && K % Fmt::BV == 0 && p.row_bytes % 2 == 0 && (((uintptr_t)p.w[0]) & 15) == 0 &&
           (((uintptr_t)p.w[1]) & 15) == 0 && (((uintptr_t)p.w[2]) & 15) == 0 && wave_loads <= (size_t)(matvec_ls_max_consumers<Fmt>() * C) &&
           !dev->knobs.no_lds_ring;
}

template <class Fmt, int NC, int C, int R, bool FUSED>
static int launch_ls(marmot_hip_device *dev, MatvecParams p, int W, size_t M, int nw) {
    const dim3 grid((unsigned)((M + p.rows_per_wg - 1) / p.rows_per_wg), nw, 1);
    const size_t part = (((size_t)p.rows_per_wg * NC * 4 * W * sizeof(float)) + 15) & ~(size_t)15;
    const bool aligned = p.row_bytes % 16 == 0;
    const size_t stage_stride = ((size_t)R * p.row_bytes + (aligned ? 0 : 15) + 1023) & ~(size_t)1023;
    const size_t lds = part + MV_LS_STAGES * stage_stride;
    if (aligned) {
        MH_TRY(allow_large_lds(dev, (const void *)k_matvec_ls<Fmt, NC, C, R, FUSED, true>));
        hipLaunchKernelGGL((k_matvec_ls<Fmt, NC, C, R, FUSED, true>), grid, dim3((W + 1) * 64), lds, dev->stream, p);
    } else {
        MH_TRY(allow_large_lds(dev, (const void *)k_matvec_ls<Fmt, NC, C, R, FUSED, false>));
        hipLaunchKernelGGL((k_matvec_ls<Fmt, NC, C, R, FUSED, false>), grid, dim3((W + 1) * 64), lds, dev->stream, p);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

template <class Fmt, int NC, int C, int R, bool FUSED, bool EXACT>
static int launch_one(marmot_hip_device *dev, const MatvecParams &p, int W, size_t M, int nw) {
    const dim3 grid((unsigned)((M + p.rows_per_wg - 1) / p.rows_per_wg), nw,
                    p.items != nullptr ? (unsigned)p.n0 : 1u);  // grouped mode: n0 carries the item-count bound
    const size_t lds = (size_t)p.rows_per_wg * NC * 4 * W * sizeof(float);
    hipLaunchKernelGGL((k_matvec<Fmt, NC, C, R, FUSED, EXACT>), grid, dim3(W * 64), lds, dev->stream, p);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

// Picks wavefronts per workgroup (W), wave-loads per wavefront (C) and rows per workgroup for one column tile.
// Returns MARMOT_HIP_ERROR_NOT_IMPLEMENTED (without setting the error text) when K is too long for this NC.
template <class Fmt, int NC, int R>
static int launch_tile_r(marmot_hip_device *dev, MatvecParams p, size_t K, size_t M, int nw, const char *name) {
    const size_t nb = (K + Fmt::BV - 1) / Fmt::BV;
    const size_t wave_loads = (nb + Fmt::BPW - 1) / Fmt::BPW;
    const bool fused = p.x != nullptr;
    constexpr bool can_fuse = NC <= 4;
    const size_t maxw1 = (fused ? matvec_max_threads<Fmt, NC, 1, R, can_fuse>()
                                : matvec_max_threads<Fmt, NC, 1, R, false>()) / 64;
    const size_t maxw2 = (fused ? matvec_max_threads<Fmt, NC, 2, R, can_fuse>()
                                : matvec_max_threads<Fmt, NC, 2, R, false>()) / 64;
    int C;
    if (wave_loads <= maxw1) {
        C = 1;
    } else if (wave_loads <= 2 * maxw2) {
        C = 2;
    } else {
        return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
    }
    const int W = (int)((wave_loads + C - 1) / C);
    // Rows per workgroup: enough workgroups to fill the chip several times over (the hardware hides latency by
    // switching between resident workgroups), but enough rows that the activation prologue is amortized.
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t wgs_per_cu = 16 / (size_t)W;
    if (wgs_per_cu < 1) {
        wgs_per_cu = 1;
    }
    if (wgs_per_cu > 8) {
        wgs_per_cu = 8;
    }
    size_t rows_per_wg = (M + cus * wgs_per_cu - 1) / (cus * wgs_per_cu);
    if (p.items != nullptr) {
        rows_per_wg = 8;  // grouped mode: the item dimension supplies the parallelism
    }
    if (fused && rows_per_wg < 8) {
        rows_per_wg = 8;
    }
    rows_per_wg = ((rows_per_wg + R - 1) / R) * R;
    if (rows_per_wg < (size_t)R) {
        rows_per_wg = R;
    }
    if (rows_per_wg > 32) {
        rows_per_wg = 32;
    }
    p.rows_per_wg = (int)rows_per_wg;
    set_route(name);
    if constexpr (NC <= 4) {
        // With packed activations there is no prologue to hide: worth it from about 16 MB of weights. Formats other
        // than Q4_K have 16-byte aligned rows when a row holds a multiple of 8 blocks; their blocks inside the LDS copy
        // are not aligned and the reads rely on unaligned LDS access. Measured faster for rows up to 8192 values
        // (14336 x 4096, N = 1 / 2 / 4: Q6_K 15.5 -> 12.9, 18.0 -> 16.7, 24.0 -> 23.5 us; Q8_0 18.4 -> 15.2,
        // 22.8 -> 16.4, 29.8 -> 22.5 us; Q8_0 5632 x 2048: 6.8 -> 6.1 us), slower for Q6_K at K = 14336.
        const bool fmt_ok = Fmt::BYTES % 16 == 0 || K <= 8192;
        if (fmt_ok && matvec_ls_usable<Fmt>(dev, p, K, C) && (fused || M * p.row_bytes >= ((size_t)16 << 20))) {
            // rows per workgroup: two workgroups per CU when M allows, between 8 (the activation prologue must pay
            // off) and 16 (more rows per workgroup leave CUs idle at the usual M)
            size_t rows_ls = (M + 2 * cus - 1) / (2 * cus);
            rows_ls = ((rows_ls + 3) / 4) * 4;
            rows_ls = rows_ls < 8 ? 8 : (rows_ls > 16 ? 16 : rows_ls);
            p.rows_per_wg = (int)rows_ls;
            if (C == 1) {
                return fused ? launch_ls<Fmt, NC, 1, 2, true>(dev, p, W, M, nw)
                             : launch_ls<Fmt, NC, 1, 2, false>(dev, p, W, M, nw);
            }
            return fused ? launch_ls<Fmt, NC, 2, 2, true>(dev, p, W, M, nw)
                         : launch_ls<Fmt, NC, 2, 2, false>(dev, p, W, M, nw);
        }
    }
    const bool exact = (size_t)W * C * Fmt::BPW == nb && K % Fmt::BV == 0 && M % rows_per_wg == 0;
    if constexpr (NC <= 4) {
        if (fused) {
            if (C == 1) {
                return exact ? launch_one<Fmt, NC, 1, R, true, true>(dev, p, W, M, nw)
                             : launch_one<Fmt, NC, 1, R, true, false>(dev, p, W, M, nw);
            }
            return launch_one<Fmt, NC, 2, R, true, false>(dev, p, W, M, nw);
        }
    } else if (fused) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "fused activation quantization is limited to 4 columns");
    }
    if (C == 1) {
        return launch_one<Fmt, NC, 1, R, false, false>(dev, p, W, M, nw);
    }
    return launch_one<Fmt, NC, 2, R, false, false>(dev, p, W, M, nw);
}

template <class Fmt, int NC>
static int launch_tile(marmot_hip_device *dev, MatvecParams p, size_t K, size_t M, int nw, const char *name) {
    if constexpr (NC == 1) {
        const int st = launch_tile_r<Fmt, NC, 4>(dev, p, K, M, nw, name);
        // a format with wide weight registers (Q5_K) covers long rows with fewer rows in flight
        return st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED ? launch_tile_r<Fmt, NC, 2>(dev, p, K, M, nw, name) : st;
    } else if constexpr (NC == 2) {
        const int st = launch_tile_r<Fmt, NC, 4>(dev, p, K, M, nw, name);
        return st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED ? launch_tile_r<Fmt, NC, 2>(dev, p, K, M, nw, name) : st;
    } else {
        return launch_tile_r<Fmt, NC, 2>(dev, p, K, M, nw, name);
    }
}

template <class Fmt>
static int launch_fmt(marmot_hip_device *dev, MatvecParams p, size_t N, size_t K, size_t M, int nw,
                      const char *name) {
    // Column tiles of up to 8 activation rows; each tile streams the weights once. A tile width whose
    // register budget cannot cover K in one pass falls back to the next narrower one.
    size_t n0 = 0;
    int cap = 8;
    while (n0 < N) {
        const size_t left = N - n0;
        p.n0 = n0;
        int st = MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
        size_t step = 0;
        if (left >= 8 && cap >= 8) {
            st = launch_tile<Fmt, 8>(dev, p, K, M, nw, name);
            step = 8;
            if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                cap = 4;
            }
        }
        if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED && left >= 4 && cap >= 4) {
            st = launch_tile<Fmt, 4>(dev, p, K, M, nw, name);
            step = 4;
            if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                cap = 2;
            }
        }
        if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED && left >= 2 && cap >= 2) {
            st = launch_tile<Fmt, 2>(dev, p, K, M, nw, name);
            step = 2;
            if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                cap = 1;
            }
        }
        if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
            st = launch_tile<Fmt, 1>(dev, p, K, M, nw, name);
            step = 1;
            if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED,
                                 "quantized matvec: K=%zu is beyond the single-pass limit of this kernel", K);
            }
        }
        if (st != MARMOT_HIP_SUCCESS) {
            return st;
        }
        n0 += step;
    }
    return MARMOT_HIP_SUCCESS;
}

bool matvec_can_fuse_quantization(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *d_x_f32) {
    const size_t bv = block_values(kind);
    return N <= 4 && bv != 0 && K % bv == 0 && (((uintptr_t)d_x_f32) & 15) == 0 && !dev->knobs.no_fused_quant;
}

int launch_matvec_packed(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, const ActScratch *act,
                         const float *d_x_f32, size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype,
                         void *d_out0, void *d_out1, int out_dtype) {
    WeightSet ws;
    ws.count = d_w1 != nullptr ? 2 : 1;
    ws.w[0] = d_w0;
    ws.w[1] = d_w1;
    ws.out[0] = d_out0;
    ws.out[1] = d_out1;
    ws.bias[0] = d_bias;
    ws.bias[1] = d_bias;
    ws.bias_dtype = bias_dtype;
    return launch_matvec_set(dev, kind, ws, act, d_x_f32, N, K, M, out_dtype);
}

int launch_matvec_set(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch *act,
                      const float *d_x_f32, size_t N, size_t K, size_t M, int out_dtype) {
    if (N == 0 || M == 0 || K == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    const size_t bv = block_values(kind);
    const size_t nb = (K + bv - 1) / bv;
    MatvecParams p;
    for (int i = 0; i < 3; ++i) {  // unused slots repeat weight 0 (the alignment checks look at all three)
        const int src = i < ws.count ? i : 0;
        p.w[i] = (const uint8_t *)ws.w[src];
        p.out[i] = ws.out[src];
        p.bias[i] = ws.bias[src];
    }
    if (act != nullptr) {
        p.act.qs = act->qs;
        p.act.d = act->d;
        p.act.sums = act->sums;
        p.act.kp = act->kp;
        p.act.nb = act->nb;
        p.x = nullptr;
    } else {
        p.act.qs = nullptr;
        p.act.d = nullptr;
        p.act.sums = nullptr;
        p.act.kp = 0;
        p.act.nb = nb;
        p.x = d_x_f32;
    }
    p.K = K;
    p.bias_is_f16 = ws.bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.bias_first = ws.bias_first ? 1 : 0;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.n0 = 0;
    p.M = M;
    p.nb = nb;
    p.row_bytes = nb * block_bytes(kind);
    p.rows_per_wg = 4;
    p.items = nullptr;
    p.n_items = nullptr;
    p.act_index = nullptr;
    p.expert_stride = 0;
    const int nw = ws.count;
    const bool fused = act == nullptr;
    if (kind == MARMOT_HIP_KIND_Q4_K && fused && N == 1 && nw == 1 && !dev->knobs.no_row_kernels &&
        !dev->knobs.no_resident_rows) {
        const int st = launch_matvec_rows2_q4k(dev, ws, d_x_f32, N, K, M, out_dtype);
        if (st != MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
            return st;
        }
    }
    if (kind == MARMOT_HIP_KIND_Q4_K && fused && N <= 2 && !dev->knobs.no_row_kernels) {
        const int st = launch_matvec_rows_q4k(dev, ws, d_x_f32, N, K, M, out_dtype);
        if (st != MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
            return st;
        }
    }
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_K:
        return launch_fmt<FmtQ4K>(dev, p, N, K, M, nw, fused ? "matvec_q4_k_q8_k_fused" : "matvec_q4_k_q8_k");
    case MARMOT_HIP_KIND_Q5_K:
        return launch_fmt<FmtQ5K>(dev, p, N, K, M, nw, fused ? "matvec_q5_k_q8_k_fused" : "matvec_q5_k_q8_k");
    case MARMOT_HIP_KIND_Q2_K:
        return launch_fmt<FmtQ2K>(dev, p, N, K, M, nw, fused ? "matvec_q2_k_q8_k_fused" : "matvec_q2_k_q8_k");
    case MARMOT_HIP_KIND_Q3_K:
        return launch_fmt<FmtQ3K>(dev, p, N, K, M, nw, fused ? "matvec_q3_k_q8_k_fused" : "matvec_q3_k_q8_k");
    case MARMOT_HIP_KIND_Q6_K:
        return launch_fmt<FmtQ6K>(dev, p, N, K, M, nw, fused ? "matvec_q6_k_q8_k_fused" : "matvec_q6_k_q8_k");
    case MARMOT_HIP_KIND_Q8_0:
        return launch_fmt<FmtQ80>(dev, p, N, K, M, nw, fused ? "matvec_q8_0_q8_0_fused" : "matvec_q8_0_q8_0");
    case MARMOT_HIP_KIND_Q4_0:
        return launch_fmt<FmtQ40>(dev, p, N, K, M, nw, fused ? "matvec_q4_0_q8_0_fused" : "matvec_q4_0_q8_0");
    case MARMOT_HIP_KIND_Q8_1:
        return launch_fmt<FmtQ81>(dev, p, N, K, M, nw, fused ? "matvec_q8_1_q8_0_fused" : "matvec_q8_1_q8_0");
    case MARMOT_HIP_KIND_Q4_1:
        return launch_fmt<FmtQ41>(dev, p, N, K, M, nw, fused ? "matvec_q4_1_q8_0_fused" : "matvec_q4_1_q8_0");
    case MARMOT_HIP_KIND_Q5_0:
        return launch_fmt<FmtQ50>(dev, p, N, K, M, nw, fused ? "matvec_q5_0_q8_0_fused" : "matvec_q5_0_q8_0");
    case MARMOT_HIP_KIND_Q5_1:
        return launch_fmt<FmtQ51>(dev, p, N, K, M, nw, fused ? "matvec_q5_1_q8_0_fused" : "matvec_q5_1_q8_0");
    default:
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "quantized matmul: unsupported quant kind %d", kind);
    }
}

// Grouped (MoE) launch: one work item = up to 8 routes of one expert; see MatvecParams.
int launch_matvec_grouped(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, size_t expert_stride,
                          const ActScratch &act, const uint32_t *d_act_index, const int4 *d_items, const int *d_n_items,
                          size_t max_items, size_t K, size_t M, void *d_out0, void *d_out1) {
    if (max_items == 0 || M == 0 || K == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    const size_t bv = block_values(kind);
    const size_t nb = (K + bv - 1) / bv;
    MatvecParams p;
    p.w[0] = (const uint8_t *)d_w0;
    p.w[1] = (const uint8_t *)(d_w1 != nullptr ? d_w1 : d_w0);
    p.w[2] = p.w[0];
    p.out[0] = d_out0;
    p.out[1] = d_out1 != nullptr ? d_out1 : d_out0;
    p.out[2] = p.out[0];
    p.act.qs = act.qs;
    p.act.d = act.d;
    p.act.sums = act.sums;
    p.act.kp = act.kp;
    p.act.nb = act.nb;
    p.x = nullptr;
    p.K = K;
    p.bias[0] = p.bias[1] = p.bias[2] = nullptr;
    p.bias_is_f16 = 0;
    p.bias_first = 0;
    p.out_is_f16 = 0;
    p.n0 = max_items;
    p.M = M;
    p.nb = nb;
    p.row_bytes = nb * block_bytes(kind);
    p.rows_per_wg = 4;
    p.items = d_items;
    p.n_items = d_n_items;
    p.act_index = d_act_index;
    p.expert_stride = expert_stride;
    const int nw = d_w1 != nullptr ? 2 : 1;
    int st;
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_K:
        st = launch_tile<FmtQ4K, 8>(dev, p, K, M, nw, "moe_grouped_q4_k_q8_k");
        break;
    case MARMOT_HIP_KIND_Q5_K:
        st = launch_tile<FmtQ5K, 8>(dev, p, K, M, nw, "moe_grouped_q5_k_q8_k");
        break;
    case MARMOT_HIP_KIND_Q2_K:
        st = launch_tile<FmtQ2K, 8>(dev, p, K, M, nw, "moe_grouped_q2_k_q8_k");
        break;
    case MARMOT_HIP_KIND_Q3_K:
        st = launch_tile<FmtQ3K, 8>(dev, p, K, M, nw, "moe_grouped_q3_k_q8_k");
        break;
    case MARMOT_HIP_KIND_Q6_K:
        st = launch_tile<FmtQ6K, 8>(dev, p, K, M, nw, "moe_grouped_q6_k_q8_k");
        break;
    case MARMOT_HIP_KIND_Q8_0:
        st = launch_tile<FmtQ80, 8>(dev, p, K, M, nw, "moe_grouped_q8_0_q8_0");
        break;
    case MARMOT_HIP_KIND_Q4_0:
        st = launch_tile<FmtQ40, 8>(dev, p, K, M, nw, "moe_grouped_q4_0_q8_0");
        break;
    case MARMOT_HIP_KIND_Q8_1:
        st = launch_tile<FmtQ81, 8>(dev, p, K, M, nw, "moe_grouped_q8_1_q8_0");
        break;
    case MARMOT_HIP_KIND_Q4_1:
        st = launch_tile<FmtQ41, 8>(dev, p, K, M, nw, "moe_grouped_q4_1_q8_0");
        break;
    case MARMOT_HIP_KIND_Q5_0:
        st = launch_tile<FmtQ50, 8>(dev, p, K, M, nw, "moe_grouped_q5_0_q8_0");
        break;
    case MARMOT_HIP_KIND_Q5_1:
        st = launch_tile<FmtQ51, 8>(dev, p, K, M, nw, "moe_grouped_q5_1_q8_0");
        break;
    default:
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "MoE experts: unsupported quant kind %d", kind);
    }
    if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "MoE experts: K=%zu is beyond the single-pass limit", K);
    }
    return st;
}

} // namespace mh

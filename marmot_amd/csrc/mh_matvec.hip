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
// Integer sub-block dots use v_dot4c_i32_i8; the fp32 scale-accumulate matches
// cpu_vec_dot_{q4_k,q6_k}_q8_k / cpu_vec_dot_{q8_0,q4_0}_q8_0 (vec_dot_impl.h) up to summation order.
#include "mh_common.h"

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

// ------------------------------------------------------------------ Q4_K x Q8_K
struct FmtQ4K {
    static constexpr int BYTES = Q4_K_BYTES;
    static constexpr int LPB = 8;  // lanes per block
    static constexpr int BPW = 8;  // blocks per wave-load
    static constexpr int BV = QK_K;
    static constexpr int ACT_DW = 11, WT_DW = 8;  // registers per lane (activation share, one row's loads)
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
        // 6-bit scale / min pairs of sub-blocks 2g and 2g+1 (get_scale_min_k4, kquant_common.h:29-37)
        const int sh = 16 * (g & 1);
        const uint32_t sa = (w.hdr.y >> sh) & 0xffffu;
        const uint32_t sb = (w.hdr.z >> sh) & 0xffffu;
        const uint32_t sc_ = (w.hdr.w >> sh) & 0xffffu;
        uint32_t scp, mp;
        if (g < 2) {
            scp = sa & 0x3f3fu;
            mp = sb & 0x3f3fu;
        } else {
            scp = (sc_ & 0x0f0fu) | ((sa >> 2) & 0x3030u);
            mp = ((sc_ >> 4) & 0x0f0fu) | ((sb >> 2) & 0x3030u);
        }
        const int sc0 = (int)(scp & 0xffu), sc1 = (int)(scp >> 8);
        const int m0 = (int)(mp & 0xffu), m1 = (int)(mp >> 8);
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
            const int isum = sc0 * dl + sc1 * dh;
            const int msum = m0 * a[n].bs_lo + m1 * a[n].bs_hi;
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
    static constexpr int ACT_DW = 21, WT_DW = 15;
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
            const int isum = sc0 * d1 + sc1 * d2 + sc2 * d3 + sc3 * d4;
            acc[n] += (a[n].d * d) * (float)isum;
        }
    }
};

// ------------------------------------------------------------------ Q8_0 x Q8_0
struct FmtQ80 {
    static constexpr int BYTES = Q8_0_BYTES;
    static constexpr int LPB = 1;
    static constexpr int BPW = 64;
    static constexpr int BV = QK;
    static constexpr int ACT_DW = 9, WT_DW = 9;
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
    __device__ static void zero_act(Act &a) {
        a.a0 = a.a1 = make_uint4(0, 0, 0, 0);
        a.d = 0.0f;
    }
    __device__ static void load_w(Wt &w, const uint8_t *blk, int) {
        w.s = ld2(blk);
        w.q0 = ld16(blk + 2);
        w.q1 = ld16(blk + 18);
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

// ------------------------------------------------------------------ Q4_0 x Q8_0
struct FmtQ40 {
    static constexpr int BYTES = Q4_0_BYTES;
    static constexpr int LPB = 1;
    static constexpr int BPW = 64;
    static constexpr int BV = QK;
    static constexpr int ACT_DW = 10, WT_DW = 5;
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

struct MatvecParams {
    const uint8_t *w[2];
    void *out[2];
    ActView act;
    const void *bias;
    int bias_is_f16;
    int out_is_f16;
    size_t n0;         // first activation row (column tile offset)
    size_t M;
    size_t nb;         // blocks per weight row
    size_t row_bytes;
    int rows_per_wg;
};

__device__ __forceinline__ void store_out(const MatvecParams &p, void *out, size_t n, size_t row, float v) {
    const size_t idx = n * p.M + row;
    if (!p.out_is_f16) {
        if (p.bias != nullptr) {
            v += ((const float *)p.bias)[row];
        }
        ((float *)out)[idx] = v;
    } else {
        // reference order: store f16(dot), then the epilogue adds the bias to the stored f16 value
        uint16_t h = f2h(v);
        if (p.bias != nullptr) {
            const float b = p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[row]) : ((const float *)p.bias)[row];
            h = f2h(h2f(h) + b);
        }
        ((uint16_t *)out)[idx] = h;
    }
}

// Largest workgroup a configuration may use: the register estimate decides how many wavefronts fit per SIMD
// (512 VGPRs per lane per SIMD on gfx950) without spilling.
template <class Fmt, int NC, int C, int R>
constexpr int matvec_max_threads() {
    constexpr int need = NC * C * Fmt::ACT_DW + R * C * Fmt::WT_DW + 2 * NC + 36;
    return need <= 120 ? 1024 : (need <= 240 ? 512 : 256);
}

template <class Fmt, int NC, int C, int R>
__global__ __launch_bounds__((matvec_max_threads<Fmt, NC, C, R>())) void k_matvec(const MatvecParams p) {
    extern __shared__ float partial[];  // [rows_per_wg][NC][W]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int W = blockDim.x >> 6;
    const int sub = lane % Fmt::LPB;
    const uint8_t *__restrict__ wbase = p.w[blockIdx.y];
    void *out = p.out[blockIdx.y];

    typename Fmt::Act act[C][NC];
    size_t blk[C];
    bool valid[C];
#pragma unroll
    for (int i = 0; i < C; ++i) {
        blk[i] = (size_t)(wave * C + i) * Fmt::BPW + lane / Fmt::LPB;
        valid[i] = blk[i] < p.nb;
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            if (valid[i]) {
                Fmt::load_act(act[i][n], p.act, p.n0 + n, blk[i], sub);
            } else {
                Fmt::zero_act(act[i][n]);
            }
        }
    }

    const size_t row0 = (size_t)blockIdx.x * p.rows_per_wg;
    for (int r = 0; r < p.rows_per_wg; r += R) {
        typename Fmt::Wt wt[R][C];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            size_t row = row0 + r + rr;
            if (row >= p.M) {
                row = p.M - 1;  // harmless re-read; the result is discarded below
            }
            const uint8_t *rowp = wbase + row * p.row_bytes;
#pragma unroll
            for (int i = 0; i < C; ++i) {
                if (valid[i]) {
                    Fmt::load_w(wt[rr][i], rowp + blk[i] * Fmt::BYTES, sub);
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
            const size_t row = row0 + r + rr;
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                const float s = wave_sum(acc[n]);
                if (lane == 0) {
                    if (W == 1) {
                        if (row < p.M) {
                            store_out(p, out, p.n0 + n, row, s);
                        }
                    } else {
                        partial[((r + rr) * NC + n) * W + wave] = s;
                    }
                }
            }
        }
    }
    if (W > 1) {
        __syncthreads();
        for (int idx = threadIdx.x; idx < p.rows_per_wg * NC; idx += blockDim.x) {
            const size_t row = row0 + idx / NC;
            const int n = idx % NC;
            if (row < p.M) {
                float s = 0.0f;
                for (int w = 0; w < W; ++w) {
                    s += partial[idx * W + w];
                }
                store_out(p, out, p.n0 + n, row, s);
            }
        }
    }
}

template <class Fmt, int NC, int C, int R>
static int launch_one(marmot_hip_device *dev, const MatvecParams &p, int W, size_t M, bool dual) {
    const dim3 grid((unsigned)((M + p.rows_per_wg - 1) / p.rows_per_wg), dual ? 2 : 1);
    const size_t lds = W > 1 ? (size_t)p.rows_per_wg * NC * W * sizeof(float) : 0;
    hipLaunchKernelGGL((k_matvec<Fmt, NC, C, R>), grid, dim3(W * 64), lds, dev->stream, p);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

// Picks wavefronts per workgroup (W), wave-loads per wavefront (C) and rows per workgroup for one column tile.
// Returns MARMOT_HIP_ERROR_NOT_IMPLEMENTED (without setting the error text) when K is too long for this NC.
template <class Fmt, int NC>
static int launch_tile(marmot_hip_device *dev, MatvecParams p, size_t K, size_t M, bool dual, const char *name) {
    constexpr int R = (NC <= 2) ? 4 : 2;
    const size_t nb = (K + Fmt::BV - 1) / Fmt::BV;
    const size_t wave_loads = (nb + Fmt::BPW - 1) / Fmt::BPW;
    constexpr size_t maxw1 = matvec_max_threads<Fmt, NC, 1, R>() / 64;
    constexpr size_t maxw2 = matvec_max_threads<Fmt, NC, 2, R>() / 64;
    int C;
    if (wave_loads <= maxw1) {
        C = 1;
    } else if (wave_loads <= 2 * maxw2) {
        C = 2;
    } else {
        return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
    }
    const int W = (int)((wave_loads + C - 1) / C);
    // Aim for about 16 resident wavefronts per CU; every workgroup re-reads the (small) activation set once.
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t wgs_per_cu = 16 / (size_t)W;
    if (wgs_per_cu < 1) {
        wgs_per_cu = 1;
    }
    if (wgs_per_cu > 8) {
        wgs_per_cu = 8;
    }
    size_t rows_per_wg = (M + cus * wgs_per_cu - 1) / (cus * wgs_per_cu);
    rows_per_wg = ((rows_per_wg + R - 1) / R) * R;
    if (rows_per_wg < (size_t)R) {
        rows_per_wg = R;
    }
    if (rows_per_wg > 32) {
        rows_per_wg = 32;
    }
    p.rows_per_wg = (int)rows_per_wg;
    set_route(name);
    if (C == 1) {
        return launch_one<Fmt, NC, 1, R>(dev, p, W, M, dual);
    }
    return launch_one<Fmt, NC, 2, R>(dev, p, W, M, dual);
}

template <class Fmt>
static int launch_fmt(marmot_hip_device *dev, MatvecParams p, size_t N, size_t K, size_t M, bool dual,
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
            st = launch_tile<Fmt, 8>(dev, p, K, M, dual, name);
            step = 8;
            if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                cap = 4;
            }
        }
        if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED && left >= 4 && cap >= 4) {
            st = launch_tile<Fmt, 4>(dev, p, K, M, dual, name);
            step = 4;
            if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                cap = 2;
            }
        }
        if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED && left >= 2 && cap >= 2) {
            st = launch_tile<Fmt, 2>(dev, p, K, M, dual, name);
            step = 2;
            if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
                cap = 1;
            }
        }
        if (st == MARMOT_HIP_ERROR_NOT_IMPLEMENTED) {
            st = launch_tile<Fmt, 1>(dev, p, K, M, dual, name);
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

int launch_matvec_packed(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, const ActScratch &act,
                         size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype, void *d_out0, void *d_out1,
                         int out_dtype) {
    if (N == 0 || M == 0 || K == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MatvecParams p;
    p.w[0] = (const uint8_t *)d_w0;
    p.w[1] = (const uint8_t *)(d_w1 != nullptr ? d_w1 : d_w0);
    p.out[0] = d_out0;
    p.out[1] = d_out1 != nullptr ? d_out1 : d_out0;
    p.act.qs = act.qs;
    p.act.d = act.d;
    p.act.sums = act.sums;
    p.act.kp = act.kp;
    p.act.nb = act.nb;
    p.bias = d_bias;
    p.bias_is_f16 = bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.n0 = 0;
    p.M = M;
    p.nb = act.nb;
    p.row_bytes = act.nb * block_bytes(kind);
    p.rows_per_wg = 4;
    const bool dual = d_w1 != nullptr;
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_K:
        return launch_fmt<FmtQ4K>(dev, p, N, K, M, dual, "matvec_q4_k_q8_k");
    case MARMOT_HIP_KIND_Q6_K:
        return launch_fmt<FmtQ6K>(dev, p, N, K, M, dual, "matvec_q6_k_q8_k");
    case MARMOT_HIP_KIND_Q8_0:
        return launch_fmt<FmtQ80>(dev, p, N, K, M, dual, "matvec_q8_0_q8_0");
    case MARMOT_HIP_KIND_Q4_0:
        return launch_fmt<FmtQ40>(dev, p, N, K, M, dual, "matvec_q4_0_q8_0");
    default:
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "quantized matmul: unsupported quant kind %d", kind);
    }
}

} // namespace mh

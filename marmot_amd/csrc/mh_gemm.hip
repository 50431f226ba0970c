// Prefill GEMM for Q4_K weights and fp16 activations on MFMA (v_mfma_f32_32x32x16_f16), fp32 accumulate.
//
// Arithmetic. The reference's direct fp16 route (cpu_vec_dot_q4_k_f16, vec_dot_impl.h:973-1023) computes
//     y[n,m] = sum_k (d*sc*q - dmin*mn)[m,k] * x[n,k]
// with fp32 dequantized weights. Rounding those weights to fp16 would cost 2^-11 per element, so the kernel does
// not form them. Per 256-value block it accumulates two exact-operand products on the matrix cores,
//     P[n,m] = sum_k (sc*q)[m,k] * x[n,k]            (sc*q <= 945 is an integer, exact in fp16; x is fp16)
//     Q[n,m] = sum_j (32*mn_j)[m] * (S_j[n] / 32)     (S_j = fp32 sum of x over sub-block j, split into hi+lo fp16)
// and then y += d*P - dmin*Q in fp32 on the vector ALU. The result differs from the reference only by fp32
// rounding / summation order.
//
// Tiling. Eight wavefronts per workgroup, two per SIMD; a wavefront owns 32 weight rows x (32 TA) tokens as TA MFMA
// tiles, so one unpacked weight operand feeds TA MFMAs. Two shapes:
//   * TA = 4, KG = 1: 128 tokens x 256 weight rows per workgroup, every wavefront walks all blocks of K: long prompts.
//   * TA = 2, KG = 2: 64 tokens x 128 weight rows; wavefronts 0..3 take the even blocks of K and 4..7 the odd ones
//     (each group stages its own activation tiles) and the two partial tiles meet in LDS at the end. 512 tokens x 4096
//     rows are 256 such tiles: the chip is full without splitting K across workgroups, so no partial sums go through
//     memory and no reduction kernel runs.
// The activation tile of a block is gathered straight from the row-major fp16 matrix into LDS in MFMA operand order
// with direct-to-LDS loads, double buffered. The sub-block sums S_j are computed from that staged tile by the
// workgroup itself (v_dot2_f32_f16 against (1, 1): exact products, fp32 accumulation) into the stage's own S area;
// the Q product of a block is taken one block later, behind the barrier that ends the block, so the sums need no
// barrier of their own. Weights are read straight from their GGUF blocks into registers, one block ahead, and unpacked
// with (q | 0x6400) as fp16 = 1024 + q, then fma(1024 + q, sc, -1024 * sc) = sc * q exactly.
// K is split across workgroups only when there are too few tiles to fill the chip (short prompts); those partial sums
// meet in a small second kernel in a fixed order.
#include "mh_common.h"
#include "mh_rows.h"

#include <stdlib.h>

namespace mh {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int G_WAVES = 8;
constexpr int G_THREADS = G_WAVES * 64;
constexpr int G_WROWS_WAVE = 32;  // weight rows per wavefront

template <int TA, int KG>
struct GemmShape {
    static constexpr int TOK = 32 * TA;                   // tokens per workgroup tile
    static constexpr int RG = G_WAVES / KG;               // row groups (wavefronts side by side along the weight rows)
    static constexpr int WROWS = G_WROWS_WAVE * RG;       // weight rows per workgroup
    static constexpr int GT = G_THREADS / KG;             // threads of one K group
    static constexpr int STAGE_A = 16 * TA * 64 * 16;     // 16 K-steps x TA token sub-tiles x 64 lanes x 16 bytes
    static constexpr int STAGE_S = TA * 64 * 16;          // sub-block sums operand: TA token sub-tiles x 64 lanes x 16 B
    static constexpr int STAGE = STAGE_A + STAGE_S;
    static constexpr int PIECES = STAGE_A / 16 / GT;      // direct-to-LDS pieces per thread and block
    static constexpr int LDS_BYTES = KG * 2 * STAGE;
    static_assert(PIECES * GT * 16 == STAGE_A, "the tile is staged in whole instructions");
    static_assert(GT == 4 * TOK, "two (token, sub-block pair) runs per thread in the sums pass");
};

// ------------------------------------------------------------------ main kernel
struct GemmParams {
    const uint8_t *w;       // Q4_K blocks, M rows of nb blocks
    const uint16_t *x;      // fp16 activations [N, K], row-major
    const uint8_t *sums;    // sub-block sums operand (k_gemm_sums), 128 x 256 tiles only
    size_t K;
    void *out;              // fp32/fp16 [N, M] (splits == 1) or fp32 partials [splits, N, M]
    const void *bias;
    int bias_is_f16;
    int out_is_f16;
    size_t N, M, nb;
    int splits;
    int blocks_per_split;
};

__device__ __forceinline__ __half2 as_h2(uint32_t v) {
    return __builtin_bit_cast(__half2, v);
}
__device__ __forceinline__ uint32_t as_u32(__half2 v) {
    return __builtin_bit_cast(uint32_t, v);
}

struct WeightRegs {
    uint4 hdr;
    uint4 q[4];  // this lane's 16 bytes of each 64-value group
};

__device__ __forceinline__ void load_weights(WeightRegs &r, const uint8_t *blk, int kh) {
    r.hdr = *(const uint4 *)blk;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        r.q[g] = *(const uint4 *)(blk + 16 + 32 * g + 16 * kh);
    }
}

struct Scales {
    uint32_t sc_lo, sc_hi;  // bytes: 6-bit scales of sub-blocks 0..3 / 4..7
    uint32_t mn_lo, mn_hi;  // bytes: 6-bit mins
    float d, dmin;
};

__device__ __forceinline__ void decode_header(const uint4 &hdr, Scales &s) {
    // vector form of get_scale_min_k4 (kquant_common.h:29-37; same packing as vec_dot_impl.h:541-556)
    s.d = h2f((uint16_t)(hdr.x & 0xffffu));
    s.dmin = h2f((uint16_t)(hdr.x >> 16));
    // Keep the two conversions as instructions of their own: folded into the 32 multiply-adds per tile that use them
    // they become mixed-precision multiply-adds, which issue at a fraction of the plain fp32 rate.
    asm volatile("" : "+v"(s.d), "+v"(s.dmin));
    s.sc_lo = hdr.y & 0x3f3f3f3fu;
    s.mn_lo = hdr.z & 0x3f3f3f3fu;
    s.sc_hi = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
    s.mn_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
}

// Two of the 8 weights of one K-step as fp16 sc*q: bytes (2*(I%2), 2*(I%2)+1) of the masked nibble dword m
template <int I>
__device__ __forceinline__ uint32_t dequant_pair(uint32_t m, __half2 sc, __half2 c) {
    // (byte n, 0x64) as fp16 bits = 1024 + n; then (1024 + q) * sc - 1024 * sc = sc * q, one rounding of an exact value
    const uint32_t t = __builtin_amdgcn_perm(0x64646464u, m, (I & 1) ? 0x04030402u : 0x04010400u);
    return as_u32(__hfma2(as_h2(t), sc, c));
}

// the B operand of the Q product: (32 * mn_e) for the 8 sub-blocks, the same in both halves of the wavefront
__device__ __forceinline__ half8 mins_operand(uint32_t lo, uint32_t hi) {
    uint4 r;
    const __half2 k32 = as_h2(0x50005000u);  // (32, 32)
    const __half2 m1024 = as_h2(0x64006400u);
    const uint32_t magic = 0x64646464u;
    r.x = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, lo, 0x04010400u)), m1024), k32));
    r.y = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, lo, 0x04030402u)), m1024), k32));
    r.z = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, hi, 0x04010400u)), m1024), k32));
    r.w = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, hi, 0x04030402u)), m1024), k32));
    return __builtin_bit_cast(half8, r);
}

// ------------------------------------------------------------------ long prompts: 128 tokens x 256 weight rows
// The workgroup tile that fills the chip by itself from about 2048 tokens on. Every wavefront walks all blocks of K with
// four MFMA tiles per unpacked weight operand; its 254 registers leave no room for the in-kernel sums, so the sub-block
// sums of the activations come from a small kernel of their own and are staged next to the activation tile.
constexpr int B_TOK = 128;        // tokens per workgroup tile
constexpr int B_WROWS_WG = G_WROWS_WAVE * G_WAVES;  // 256 weight rows per workgroup
constexpr int B_STAGE_A = 16 * 4 * 64 * 16;  // 16 K-steps x 4 token sub-tiles x 64 lanes x 16 bytes
constexpr int B_STAGE_S = 4 * 64 * 16;       // sub-block sums operand: 4 token sub-tiles x 64 lanes x 16 bytes
constexpr int B_STAGE = B_STAGE_A + B_STAGE_S;   // 69,632 bytes per (token tile, block)
constexpr int B_STAGE_CHUNKS = B_STAGE / 16;   // 4352

// ------------------------------------------------------------------ sub-block sums of the activations
// S operand of (token tile tt, block b, token sub-tile a): lane (i = lane % 32, kh = lane / 32), slot e:
//     kh == 0 ? hi : lo   of   (fp32 sum of X[128*tt + 32*a + i][256*b + 32*e .. +32]) / 32,   hi + lo in fp16.
// Tokens beyond N give zeros. One thread per (token, block, sub-block).
__global__ __launch_bounds__(256) void k_gemm_sums(const uint16_t *__restrict__ x, size_t N, size_t K, size_t nb,
                                                   uint8_t *__restrict__ sums) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t tiles = (N + B_TOK - 1) / B_TOK;
    if (idx >= tiles * B_TOK * nb * 8) {
        return;
    }
    const int e = (int)(idx & 7);
    const size_t b = (idx >> 3) % nb;
    const size_t token = (idx >> 3) / nb;
    float s = 0.0f;
    if (token < N) {
        const uint4 *p = (const uint4 *)(x + token * K + b * 256 + 32 * e);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint4 v = p[c];
            s += ((h2f((uint16_t)(v.x & 0xffffu)) + h2f((uint16_t)(v.x >> 16))) +
                  (h2f((uint16_t)(v.y & 0xffffu)) + h2f((uint16_t)(v.y >> 16)))) +
                ((h2f((uint16_t)(v.z & 0xffffu)) + h2f((uint16_t)(v.z >> 16))) +
                 (h2f((uint16_t)(v.w & 0xffffu)) + h2f((uint16_t)(v.w >> 16))));
        }
    }
    s *= 0.03125f;  // exact; keeps the value within fp16 range whatever the activations are
    const uint16_t hi = f2h(s);
    const uint16_t lo = f2h(s - h2f(hi));
    const size_t tt = token / B_TOK;
    const int a = (int)(token % B_TOK) >> 5, i = (int)(token & 31);
    uint16_t *base = (uint16_t *)(sums + ((tt * nb + b) * 4 + a) * 1024);
    base[(size_t)i * 8 + e] = hi;         // lane i       (kh = 0)
    base[(size_t)(32 + i) * 8 + e] = lo;  // lane 32 + i  (kh = 1)
}

__global__ __launch_bounds__(G_THREADS) void k_gemm_q4k_f16_big(const GemmParams p) {
    warm_kernel_arguments<sizeof(GemmParams)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // 2 stages
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int j = lane & 31, kh = lane >> 5;
    const size_t tt = blockIdx.y;
    const size_t wrow0 = (size_t)blockIdx.x * B_WROWS_WG + (size_t)wave * G_WROWS_WAVE;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    size_t wr = wrow0 + j;
    if (wr >= p.M) {
        wr = p.M - 1;  // harmless re-read; never stored
    }
    const uint8_t *wrow = p.w + wr * p.nb * Q4_K_BYTES;

    floatx16 total[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            total[a][r] = 0.0f;
        }
    }

    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    typedef const __attribute__((address_space(1))) uint8_t glb_u8;
    // One stage is moved global -> LDS with direct-to-LDS loads: every wavefront instruction moves 64 lanes x 16 bytes
    // from per-lane global addresses to a contiguous 1 KiB of LDS (no registers involved); vmcnt tracks completion.
    // LDS layout of the activation part: token t of the tile owns 512 bytes (its 256 halves of this block) as 32
    // chunks of 16 bytes, chunk c stored in slot c ^ (t % 16). One instruction covers tokens 2q and 2q+1, so its
    // global reads are two contiguous 512-byte rows; the slot swizzle makes the MFMA operand reads below (16 tokens
    // x the same chunk) fall into 16 different bank groups. Tokens beyond N re-read token N-1 (never stored).
    uint32_t gather_off[9];  // byte offset of this thread's piece from the tile's first row, block-independent
    const uint8_t *tile_x = (const uint8_t *)(p.x + tt * B_TOK * p.K);
#pragma unroll
    for (int c = 0; c < 9; ++c) {
        const int chunk = tid + G_THREADS * c;
        if (chunk < B_STAGE_A / 16) {
            const int t = chunk >> 5, slot = chunk & 31;
            size_t trow = t;
            if (tt * B_TOK + trow >= p.N) {
                trow = p.N - 1 - tt * B_TOK;
            }
            gather_off[c] = (uint32_t)(trow * p.K * 2 + 16 * (slot ^ (t & 15)));
        } else {
            gather_off[c] = 0;
        }
    }
    auto stage_piece = [&](size_t b, uint8_t *dst, int c) {
        const int chunk = tid + G_THREADS * c;
        const int wbase = chunk - lane;  // first chunk of this wavefront's instruction
        if (wbase < B_STAGE_CHUNKS) {      // wave-uniform
            const uint8_t *g;
            if (chunk < B_STAGE_A / 16) {
                g = tile_x + gather_off[c] + b * 512;
            } else {
                g = p.sums + (tt * p.nb + b) * B_STAGE_S + (size_t)(chunk - B_STAGE_A / 16) * 16;
            }
            uint8_t *l = dst + (size_t)wbase * 16;  // wave-uniform base; the hardware adds lane * 16
            __builtin_amdgcn_global_load_lds((glb_u8 *)g, (lds_u8 *)l, 16, 0, 0);
        }
    };
    // MFMA A operand of K-step ks, token sub-tile a, lane (i = j, kh): token 32a + i, chunk 4(ks/2) + 2kh + ks%2.
    // Per-lane part of its LDS offset for the 8 combinations of ((ks/2) % 4, ks % 2); the rest is a constant.
    uint32_t a_off[4][2];
#pragma unroll
    for (int s3 = 0; s3 < 4; ++s3) {
#pragma unroll
        for (int tp = 0; tp < 2; ++tp) {
            a_off[s3][tp] = (uint32_t)(j * 512 + 16 * ((4 * s3 + 2 * kh + tp) ^ (j & 15)));
        }
    }

    WeightRegs wnext;
    if (b0 < b1) {
#pragma unroll
        for (int c = 0; c < 9; ++c) {
            stage_piece(b0, lds, c);
        }
        load_weights(wnext, wrow + b0 * Q4_K_BYTES, kh);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    for (size_t b = b0; b < b1; ++b) {
        const int cur = (int)((b - b0) & 1);
        const uint8_t *stage = lds + (size_t)cur * B_STAGE;
        const bool more = b + 1 < b1;

        const WeightRegs wcur = wnext;
        Scales sc;
        decode_header(wcur.hdr, sc);
        // The next block's activations (straight into the other LDS stage) and weights (into registers) are
        // requested from inside the K loop.
        uint8_t *next_stage = lds + (size_t)(cur ^ 1) * B_STAGE;
        const uint8_t *next_blk = wrow + (b + 1) * Q4_K_BYTES;
        auto prefetch_piece = [&](int ks) {
            if (!more) {
                return;
            }
            // Weights (into registers) early, one load per K-step. The activation tile (direct-to-LDS) as late as
            // possible, all nine pieces in the last K-step. Measured with the cycle counter: a load issued inside the
            // K loop costs its wavefront about 230 clocks (the eight wavefronts issue in the same K-step, and one that
            // is held at the memory issue stage holds back its own MFMA chain), 2 K clocks per block, while the wait
            // at the end of the block is barrier skew and does not get shorter when the tile was requested earlier.
            // Issued here the loads overlap the min-term product and the scale pass.
            if (ks == 15) {
#pragma unroll
                for (int c = 0; c < 9; ++c) {
                    stage_piece(b + 1, next_stage, c);
                }
            } else if (ks == 1) {
                wnext.hdr = *(const uint4 *)next_blk;
            } else if (ks >= 2 && ks < 6) {
                wnext.q[ks - 2] = *(const uint4 *)(next_blk + 16 + 32 * (ks - 2) + 16 * kh);
            }
        };

        // Operand B of K-step ks is built in 4 pieces, one per MFMA of the previous K-step, so that the unpack
        // arithmetic runs in the shadow of the matrix core. The scheduling fences pin that order.
        __half2 scp, cp;
        uint32_t m0 = 0, m1 = 0;
        auto b_piece = [&](int ks, int i) -> uint32_t {
            const int s_ = ks >> 1, tp = ks & 1, g = s_ >> 1;
            if (i == 0) {
                if (tp == 0) {
                    const uint32_t scw = s_ < 4 ? sc.sc_lo : sc.sc_hi;
                    // (1024 + sc, 1024 + sc) - (1024, 1024)
                    const uint32_t sel = (s_ & 3) == 0 ? 0x04000400u : (s_ & 3) == 1 ? 0x04010401u
                                       : (s_ & 3) == 2 ? 0x04020402u : 0x04030403u;
                    scp = __hsub2(as_h2(__builtin_amdgcn_perm(0x64646464u, scw, sel)), as_h2(0x64006400u));
                    cp = __hmul2(scp, as_h2(0xe400e400u));  // -1024 * sc, exact
                }
                const uint32_t q0 = tp ? wcur.q[g].z : wcur.q[g].x;
                const uint32_t q1 = tp ? wcur.q[g].w : wcur.q[g].y;
                m0 = ((s_ & 1) ? (q0 >> 4) : q0) & 0x0f0f0f0fu;
                m1 = ((s_ & 1) ? (q1 >> 4) : q1) & 0x0f0f0f0fu;
            }
            switch (i) {
            case 0: return dequant_pair<0>(m0, scp, cp);
            case 1: return dequant_pair<1>(m0, scp, cp);
            case 2: return dequant_pair<0>(m1, scp, cp);
            default: return dequant_pair<1>(m1, scp, cp);
            }
        };
        auto read_a = [&](int ks, half8(&aop)[4]) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                aop[a] = __builtin_bit_cast(
                    half8, *(const uint4 *)(stage + a_off[(ks >> 1) & 3][ks & 1] + (a * 16384 + 256 * (ks >> 3))));
            }
        };

        floatx16 acc[4];
        half8 aop[2][4];  // A operands of the K-step in flight and of the next one
        uint32_t bop[2][4];
        read_a(0, aop[0]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bop[0][i] = b_piece(0, i);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 16; ++ks) {
            const int c = ks & 1, n = c ^ 1;
            if (ks < 15) {
                read_a(ks + 1, aop[n]);  // lands while the 4 MFMAs below run
            }
            __builtin_amdgcn_sched_barrier(0);
            const half8 bcur = __builtin_bit_cast(half8, make_uint4(bop[c][0], bop[c][1], bop[c][2], bop[c][3]));
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                if (ks == 0) {
                    const floatx16 zero = {0};
                    acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[c][a], bcur, zero, 0, 0, 0);
                } else {
                    acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[c][a], bcur, acc[a], 0, 0, 0);
                }
                if (ks < 15) {
                    bop[n][a] = b_piece(ks + 1, a);
                }
                if (a == 1) {
                    prefetch_piece(ks);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // min term and the per-block scales: total += d * P - dmin * Q
        half8 b2;
        {
            uint4 r;
            const uint32_t lo = sc.mn_lo, hi = sc.mn_hi;
            const __half2 k32 = as_h2(0x50005000u);  // (32, 32)
            const __half2 m1024 = as_h2(0x64006400u);
            const uint32_t magic = 0x64646464u;
            r.x = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, lo, 0x04010400u)), m1024), k32));
            r.y = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, lo, 0x04030402u)), m1024), k32));
            r.z = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, hi, 0x04010400u)), m1024), k32));
            r.w = as_u32(__hmul2(__hsub2(as_h2(__builtin_amdgcn_perm(magic, hi, 0x04030402u)), m1024), k32));
            b2 = __builtin_bit_cast(half8, r);
        }
        const float d = sc.d, nd = -sc.dmin;
        // Q-term MFMA of token sub-tile a runs while the vector ALU applies d to sub-tile a and dmin to sub-tile a-1
        floatx16 mq[2];
        half8 a2[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            a2[a] = __builtin_bit_cast(half8, *(const uint4 *)(stage + B_STAGE_A + ((size_t)a * 64 + lane) * 16));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int a = 0; a < 5; ++a) {
            if (a < 4) {
                const floatx16 zero = {0};
                mq[a & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2[a], b2, zero, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    total[a][r] = __builtin_fmaf(d, acc[a][r], total[a][r]);
                }
            }
            if (a > 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    total[a - 1][r] = __builtin_fmaf(nd, mq[(a - 1) & 1][r], total[a - 1][r]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_waitcnt(0);  // the next stage's direct-to-LDS loads have landed
        __syncthreads();
    }

    // epilogue: lane (j, kh) holds weight row m = wrow0 + j for tokens 32a + 8(r/4) + 4kh + r%4
    const size_t m = wrow0 + j;
    if (m >= p.M) {
        return;
    }
    const size_t n0 = tt * B_TOK + 4 * kh;
    if (p.splits > 1) {
        float *dst = (float *)p.out + (size_t)split * p.N * p.M + m;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t n = n0 + 32 * a + 8 * (r >> 2) + (r & 3);
                if (n < p.N) {
                    dst[n * p.M] = total[a][r];
                }
            }
        }
    } else if (!p.out_is_f16) {
        const float bias = p.bias != nullptr ? ((const float *)p.bias)[m] : 0.0f;
        float *dst = (float *)p.out + m;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t n = n0 + 32 * a + 8 * (r >> 2) + (r & 3);
                if (n < p.N) {
                    dst[n * p.M] = total[a][r] + bias;
                }
            }
        }
    } else {
        const bool has_bias = p.bias != nullptr;
        const float bias = !has_bias ? 0.0f
            : p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[m]) : ((const float *)p.bias)[m];
        uint16_t *dst = (uint16_t *)p.out + m;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t n = n0 + 32 * a + 8 * (r >> 2) + (r & 3);
                if (n < p.N) {
                    uint16_t h = f2h(total[a][r]);  // round to the output type first, then add the bias in it
                    if (has_bias) {
                        h = f2h(h2f(h) + bias);
                    }
                    dst[n * p.M] = h;
                }
            }
        }
    }
}


template <int TA, int KG>
__global__ __launch_bounds__(G_THREADS) void k_gemm_q4k_f16(const GemmParams p) {
    using S = GemmShape<TA, KG>;
    warm_kernel_arguments<sizeof(GemmParams)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // KG x 2 stages
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int kg = wave / S::RG;          // K group of this wavefront
    const int rgp = wave % S::RG;         // its row group
    const int gt = rgp * 64 + lane;       // thread index inside the K group
    const int j = lane & 31, kh = lane >> 5;
    const size_t tt = blockIdx.y;
    const size_t wrow0 = (size_t)blockIdx.x * S::WROWS + (size_t)rgp * G_WROWS_WAVE;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    size_t wr = wrow0 + j;
    if (wr >= p.M) {
        wr = p.M - 1;  // harmless re-read; never stored
    }
    const uint8_t *wrow = p.w + wr * p.nb * Q4_K_BYTES;
    uint8_t *const my_stages = lds + (size_t)kg * 2 * S::STAGE;

    floatx16 total[TA];
#pragma unroll
    for (int a = 0; a < TA; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            total[a][r] = 0.0f;
        }
    }

    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    typedef const __attribute__((address_space(1))) uint8_t glb_u8;
    // One stage is moved global -> LDS with direct-to-LDS loads: every wavefront instruction moves 64 lanes x 16 bytes
    // from per-lane global addresses to a contiguous 1 KiB of LDS (no registers involved); vmcnt tracks completion.
    // LDS layout of the activation part: token t of the tile owns 512 bytes (its 256 halves of this block) as 32
    // chunks of 16 bytes, chunk c stored in slot c ^ (t % 16). One instruction covers tokens 2q and 2q+1, so its
    // global reads are two contiguous 512-byte rows; the slot swizzle makes the MFMA operand reads below (16 tokens
    // x the same chunk) fall into 16 different bank groups. Tokens beyond N re-read token N-1 (never stored).
    // The byte offset of a thread's piece from the tile's first row is recomputed when the piece is requested (a few
    // integer operations per block) instead of living in registers through the K loop.
    const uint8_t *tile_x = (const uint8_t *)(p.x + tt * S::TOK * p.K);
    const uint32_t row_pitch = (uint32_t)(p.K * 2);
    const uint32_t last_row = (uint32_t)(p.N - 1 - tt * S::TOK);  // rows beyond it re-read it
    auto stage_piece = [&](size_t b, uint8_t *dst, int c) {
        const int chunk = gt + S::GT * c;
        const int t = chunk >> 5, slot = chunk & 31;
        const uint32_t trow = (uint32_t)t < last_row ? (uint32_t)t : last_row;
        const uint8_t *g = tile_x + (size_t)trow * row_pitch + 16 * (slot ^ (t & 15)) + b * 512;
        uint8_t *l = dst + (size_t)(chunk - lane) * 16;  // wave-uniform base; the hardware adds lane * 16
        __builtin_amdgcn_global_load_lds((glb_u8 *)g, (lds_u8 *)l, 16, 0, 0);
    };
    // MFMA A operand of K-step ks, token sub-tile a, lane (i = j, kh): token 32a + i, chunk 4(ks/2) + 2kh + ks%2.
    // Per-lane part of its LDS offset for the 8 combinations of ((ks/2) % 4, ks % 2); the rest is a constant.
    uint32_t a_off[4][2];
#pragma unroll
    for (int s3 = 0; s3 < 4; ++s3) {
#pragma unroll
        for (int tp = 0; tp < 2; ++tp) {
            a_off[s3][tp] = (uint32_t)(j * 512 + 16 * ((4 * s3 + 2 * kh + tp) ^ (j & 15)));
        }
    }
    // Sums pass: this thread adds up two neighbouring sub-blocks (64 halves = 8 chunks) of one token of the staged tile.
    const int sum_token = gt % S::TOK, sum_pair = gt / S::TOK;  // sub-blocks 2 sum_pair and 2 sum_pair + 1
    const uint32_t sum_src = (uint32_t)(sum_token * 512);
    const uint32_t sum_dst = (uint32_t)(S::STAGE_A + (sum_token >> 5) * 1024 + (sum_token & 31) * 16 + 4 * sum_pair);

    const size_t first = b0 + (size_t)kg;  // this K group's blocks: first, first + KG, ...
    WeightRegs wnext;
    if (first < b1) {
#pragma unroll
        for (int c = 0; c < S::PIECES; ++c) {
            stage_piece(first, my_stages, c);
        }
        load_weights(wnext, wrow + first * Q4_K_BYTES, kh);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    uint32_t prev_mn_lo = 0, prev_mn_hi = 0;
    float prev_ndmin = 0.0f;
    bool have_prev = false;
    int cur = 0;
    // Q product of the block whose sums sit in `stage_s` (written one block ago): total -= dmin * (S x mins)
    auto q_term = [&](const uint8_t *stage_s, uint32_t mn_lo, uint32_t mn_hi, float ndmin) {
        const half8 b2 = mins_operand(mn_lo, mn_hi);
#pragma unroll
        for (int a = 0; a < TA; ++a) {
            const half8 a2 = __builtin_bit_cast(half8, *(const uint4 *)(stage_s + ((size_t)a * 64 + lane) * 16));
            const floatx16 zero = {0};
            const floatx16 mq = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b2, zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                total[a][r] = __builtin_fmaf(ndmin, mq[r], total[a][r]);
            }
        }
    };

    // the loop runs the same number of times in both K groups (barriers inside): a group without a block idles through
    const size_t rounds = (b1 - b0 + KG - 1) / KG;
    for (size_t round = 0; round < rounds; ++round) {
        const size_t b = first + round * KG;
        const bool mine = b < b1;
        uint8_t *stage = my_stages + (size_t)cur * S::STAGE;
        uint8_t *other = my_stages + (size_t)(cur ^ 1) * S::STAGE;
        const bool more = b + KG < b1;
        if (mine) {
            // ---- sums of this block's tile into the stage's S area (read by the Q product one block later)
            {
                float s0 = 0.0f, s1 = 0.0f;
                const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const uint4 v = *(const uint4 *)(stage + sum_src + 16 * ((8 * sum_pair + c) ^ (sum_token & 15)));
                    float acc = c < 4 ? s0 : s1;
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.x), ones, acc, false);
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.y), ones, acc, false);
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.z), ones, acc, false);
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.w), ones, acc, false);
                    if (c < 4) {
                        s0 = acc;
                    } else {
                        s1 = acc;
                    }
                }
                s0 *= 0.03125f;  // exact; keeps the value within fp16 range whatever the activations are
                s1 *= 0.03125f;
                const uint16_t h0 = f2h(s0), h1 = f2h(s1);
                const uint16_t l0 = f2h(s0 - h2f(h0)), l1 = f2h(s1 - h2f(h1));
                // S operand of token sub-tile a: lane i (kh = 0) holds the 8 hi parts of token 32a + i, lane 32 + i the lo parts
                *(uint32_t *)(stage + sum_dst) = (uint32_t)h0 | ((uint32_t)h1 << 16);
                *(uint32_t *)(stage + sum_dst + 512) = (uint32_t)l0 | ((uint32_t)l1 << 16);
            }

            const WeightRegs wcur = wnext;
            Scales sc;
            decode_header(wcur.hdr, sc);
            // The next block's activations (straight into the other LDS stage) and weights (into registers) are
            // requested from inside the K loop.
            const uint8_t *next_blk = wrow + (b + KG) * Q4_K_BYTES;
            auto prefetch_piece = [&](int ks) {
                if (!more) {
                    return;
                }
                // Weights (into registers) early, one load per K-step. The activation tile (direct-to-LDS) as late as
                // possible, all pieces in the last K-step. Measured with the cycle counter: a load issued inside the K
                // loop costs its wavefront about 230 clocks (the eight wavefronts issue in the same K-step, and one
                // that is held at the memory issue stage holds back its own MFMA chain), while the wait at the end of
                // the block is barrier skew and does not get shorter when the tile was requested earlier.
                if (ks == 15) {
#pragma unroll
                    for (int c = 0; c < S::PIECES; ++c) {
                        stage_piece(b + KG, other, c);
                    }
                } else if (ks == 1) {
                    wnext.hdr = *(const uint4 *)next_blk;
                } else if (ks >= 2 && ks < 6) {
                    wnext.q[ks - 2] = *(const uint4 *)(next_blk + 16 + 32 * (ks - 2) + 16 * kh);
                }
            };

            // Operand B of K-step ks is built in 4 pieces spread over the MFMAs of the previous K-step, so that the
            // unpack arithmetic runs in the shadow of the matrix core. The scheduling fences pin that order.
            __half2 scp, cp;
            uint32_t m0 = 0, m1 = 0;
            auto b_piece = [&](int ks, int i) -> uint32_t {
                const int s_ = ks >> 1, tp = ks & 1, g = s_ >> 1;
                if (i == 0) {
                    if (tp == 0) {
                        const uint32_t scw = s_ < 4 ? sc.sc_lo : sc.sc_hi;
                        // (1024 + sc, 1024 + sc) - (1024, 1024)
                        const uint32_t sel = (s_ & 3) == 0 ? 0x04000400u : (s_ & 3) == 1 ? 0x04010401u
                                           : (s_ & 3) == 2 ? 0x04020402u : 0x04030403u;
                        scp = __hsub2(as_h2(__builtin_amdgcn_perm(0x64646464u, scw, sel)), as_h2(0x64006400u));
                        cp = __hmul2(scp, as_h2(0xe400e400u));  // -1024 * sc, exact
                    }
                    const uint32_t q0 = tp ? wcur.q[g].z : wcur.q[g].x;
                    const uint32_t q1 = tp ? wcur.q[g].w : wcur.q[g].y;
                    m0 = ((s_ & 1) ? (q0 >> 4) : q0) & 0x0f0f0f0fu;
                    m1 = ((s_ & 1) ? (q1 >> 4) : q1) & 0x0f0f0f0fu;
                }
                switch (i) {
                case 0: return dequant_pair<0>(m0, scp, cp);
                case 1: return dequant_pair<1>(m0, scp, cp);
                case 2: return dequant_pair<0>(m1, scp, cp);
                default: return dequant_pair<1>(m1, scp, cp);
                }
            };
            auto read_a = [&](int ks, half8(&aop)[TA]) {
#pragma unroll
                for (int a = 0; a < TA; ++a) {
                    aop[a] = __builtin_bit_cast(
                        half8, *(const uint4 *)(stage + a_off[(ks >> 1) & 3][ks & 1] + (a * 16384 + 256 * (ks >> 3))));
                }
            };

            floatx16 acc[TA];
            half8 aop[2][TA];  // A operands of the K-step in flight and of the next one
            uint32_t bop[2][4];
            read_a(0, aop[0]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                bop[0][i] = b_piece(0, i);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 16; ++ks) {
                const int c = ks & 1, n = c ^ 1;
                if (ks < 15) {
                    read_a(ks + 1, aop[n]);  // lands while the MFMAs below run
                }
                __builtin_amdgcn_sched_barrier(0);
                const half8 bcur = __builtin_bit_cast(half8, make_uint4(bop[c][0], bop[c][1], bop[c][2], bop[c][3]));
#pragma unroll
                for (int a = 0; a < TA; ++a) {
                    if (ks == 0) {
                        const floatx16 zero = {0};
                        acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[c][a], bcur, zero, 0, 0, 0);
                    } else {
                        acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[c][a], bcur, acc[a], 0, 0, 0);
                    }
                    if (ks < 15) {
#pragma unroll
                        for (int i = a * (4 / TA); i < (a + 1) * (4 / TA); ++i) {
                            bop[n][i] = b_piece(ks + 1, i);
                        }
                    }
                    if (a == (TA > 1 ? 1 : 0)) {
                        prefetch_piece(ks);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // per-block scale of the P product, and the Q product of the previous block of this K group
            const float d = sc.d;
#pragma unroll
            for (int a = 0; a < TA; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    total[a][r] = __builtin_fmaf(d, acc[a][r], total[a][r]);
                }
            }
            if (have_prev) {
                q_term(other + S::STAGE_A, prev_mn_lo, prev_mn_hi, prev_ndmin);
            }
            prev_mn_lo = sc.mn_lo;
            prev_mn_hi = sc.mn_hi;
            prev_ndmin = -sc.dmin;
            have_prev = true;
        }
        __builtin_amdgcn_s_waitcnt(0);  // the next stage's direct-to-LDS loads have landed, this stage's sums are stored
        __syncthreads();
        cur ^= 1;
    }
    if (have_prev) {  // the last block's sums sit in the stage that was current in the last round with a block
        const size_t mine_rounds = first < b1 ? (b1 - first + KG - 1) / KG : 0;
        const int last_stage = (int)((mine_rounds - 1) & 1);
        q_term(my_stages + (size_t)last_stage * S::STAGE + S::STAGE_A, prev_mn_lo, prev_mn_hi, prev_ndmin);
    }

    if (KG > 1) {
        // the K groups' partial tiles meet in LDS: group 1 stores, group 0 adds and goes on to the epilogue
        __syncthreads();  // every wavefront is done with the stages
        float *red = (float *)lds + (size_t)rgp * TA * 16 * 64 + lane;
        if (kg == 1) {
#pragma unroll
            for (int a = 0; a < TA; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    red[(a * 16 + r) * 64] = total[a][r];
                }
            }
        }
        __syncthreads();
        if (kg != 0) {
            return;
        }
#pragma unroll
        for (int a = 0; a < TA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                total[a][r] += red[(a * 16 + r) * 64];
            }
        }
    }

    // epilogue: lane (j, kh) holds weight row m = wrow0 + j for tokens 32a + 8(r/4) + 4kh + r%4
    if (KG > 1 && p.splits == 1 && wrow0 + G_WROWS_WAVE <= p.M && (p.M & 3) == 0 && (((uintptr_t)p.out) & 15) == 0) {
        // Stores straight from this layout are 4 bytes per lane, 32 of them per lane (measured: 280 clocks per
        // store instruction at issue, 9000 clocks for the tile). The wavefront's 32 rows x TOK tokens go through its
        // own 8 KiB of LDS (the region its K partner just used for the reduction, read only by this wavefront) and
        // leave as 16 bytes per lane: every instruction writes 8 tokens x 128 contiguous bytes.
        static_assert(G_WROWS_WAVE == 32, "the transposed epilogue assumes 32 weight rows per wavefront");
        float *tile = (float *)lds + (size_t)rgp * TA * 16 * 64;  // [token][32 rows]
        __builtin_amdgcn_s_waitcnt(0xc07f);  // the reduction's reads of this region are done
#pragma unroll
        for (int a = 0; a < TA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                tile[(32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * 32 + j] = total[a][r];
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        const int q4 = lane & 7, tl = lane >> 3;  // rows 4 q4 .. 4 q4 + 3 of token tl (+ 8 per step)
        const size_t m4 = wrow0 + 4 * (size_t)q4;
        float bias4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const bool has_bias = p.bias != nullptr;
        if (has_bias) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                bias4[e] = p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[m4 + e]) : ((const float *)p.bias)[m4 + e];
            }
        }
#pragma unroll
        for (int it = 0; it < S::TOK / 8; ++it) {
            const int t = it * 8 + tl;
            const size_t n = tt * S::TOK + (size_t)t;
            const float4 v = *(const float4 *)(tile + t * 32 + 4 * q4);
            if (n >= p.N) {
                continue;
            }
            float e4[4] = {v.x, v.y, v.z, v.w};
            if (!p.out_is_f16) {
                float4 o;  // bias4 is zero without a bias: the same addition as the per-element path
                o.x = e4[0] + bias4[0], o.y = e4[1] + bias4[1], o.z = e4[2] + bias4[2], o.w = e4[3] + bias4[3];
                *(float4 *)((float *)p.out + n * p.M + m4) = o;
            } else {
                uint16_t h[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    h[e] = f2h(e4[e]);  // round to the output type first, then add the bias in it
                    if (has_bias) {
                        h[e] = f2h(h2f(h[e]) + bias4[e]);
                    }
                }
                *(uint2 *)((uint16_t *)p.out + n * p.M + m4) =
                    make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
            }
        }
        return;
    }
    const size_t m = wrow0 + j;
    if (m >= p.M) {
        return;
    }
    const size_t n0 = tt * S::TOK + 4 * kh;
    if (p.splits > 1) {
        float *dst = (float *)p.out + (size_t)split * p.N * p.M + m;
#pragma unroll
        for (int a = 0; a < TA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t n = n0 + 32 * a + 8 * (r >> 2) + (r & 3);
                if (n < p.N) {
                    dst[n * p.M] = total[a][r];
                }
            }
        }
    } else if (!p.out_is_f16) {
        const float bias = p.bias != nullptr ? ((const float *)p.bias)[m] : 0.0f;
        float *dst = (float *)p.out + m;
#pragma unroll
        for (int a = 0; a < TA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t n = n0 + 32 * a + 8 * (r >> 2) + (r & 3);
                if (n < p.N) {
                    dst[n * p.M] = total[a][r] + bias;
                }
            }
        }
    } else {
        const bool has_bias = p.bias != nullptr;
        const float bias = !has_bias ? 0.0f
            : p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[m]) : ((const float *)p.bias)[m];
        uint16_t *dst = (uint16_t *)p.out + m;
#pragma unroll
        for (int a = 0; a < TA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t n = n0 + 32 * a + 8 * (r >> 2) + (r & 3);
                if (n < p.N) {
                    uint16_t h = f2h(total[a][r]);  // round to the output type first, then add the bias in it
                    if (has_bias) {
                        h = f2h(h2f(h) + bias);
                    }
                    dst[n * p.M] = h;
                }
            }
        }
    }
}

// ------------------------------------------------------------------ 64 tokens x 128 weight rows, loader wavefronts
// The same tile as the TA = 2, KG = 2 shape above with the memory work taken away from the wavefronts that drive the
// matrix cores. A vector-memory instruction costs the wavefront that issues it the time the compute unit's one
// address / tag pipeline needs for everything queued in front of it (measured on this kernel's predecessor: about
// 230 clocks per instruction when eight wavefronts issue in the same K-step, 13 instructions per wavefront and block),
// and a wavefront that waits at the memory issue stage issues no MFMA either. Here:
//   * wavefronts 0..3 (one per SIMD) compute: wavefront c owns weight rows 64 (c % 2) .. + 63 (two B operands) x all 64
//     tokens (two A operands), four MFMAs per K-step, and the K-steps 8 (c / 2) .. + 7 of every block. It issues no
//     vector-memory instruction inside the K loop. Each A operand read from LDS feeds two MFMAs and each unpacked
//     B operand feeds two: half the LDS reads per MFMA of a 32-row wavefront tile. (Eight compute wavefronts of
//     32 rows x 64 tokens, two per SIMD, were measured slower: the SIMD serves the older wavefront first, the two
//     finish a block 1100 clocks apart and the barrier waits for the second.)
//   * wavefronts 4..7 (one per SIMD) load: per block they bring the activation tile (64 tokens x 512 bytes, two
//     contiguous token rows per instruction) and the raw weight blocks (128 rows x 144 bytes, nine lanes per block,
//     so an instruction touches about 14 cache lines instead of 32 to 64) into one of three LDS stages with
//     direct-to-LDS loads, two blocks ahead, and compute the sub-block sums of the block in work (16 tokens per
//     loader) into the stage's S area while the next block is still landing.
// One barrier per block orders everything: behind barrier i the tile and the weights of block i are complete, the
// sums of block i - 1 too (its Q product runs one block late, like in the tile above), and the tile and weight areas of
// block i - 1's stage are free for block i + 2. The barrier is an LDS-count wait plus s_barrier written by hand:
// the usual workgroup barrier also waits for the wavefront's outstanding global loads, which here are the two blocks
// in flight.
constexpr int L_TOK = 64;
constexpr int L_WROWS = 128;
constexpr int L_COMPUTE = 4;
constexpr int L_LOADERS = 4;
constexpr int L_THREADS = (L_COMPUTE + L_LOADERS) * 64;
constexpr int L_STAGE_A = L_TOK * 512;              // 32,768
constexpr int L_STAGE_W = L_WROWS * Q4_K_BYTES;     // 18,432
constexpr int L_STAGE_S = 2 * 64 * 16;              // sub-block sums operand of the two token sub-tiles
constexpr int L_STAGE = L_STAGE_A + L_STAGE_W + L_STAGE_S;
constexpr int L_STAGES = 3;
constexpr int L_LDS_BYTES = L_STAGES * L_STAGE;     // 159,744 of 163,840
constexpr int L_OUT_PITCH = L_WROWS + 4;            // floats per token of the output tile in LDS
static_assert(L_TOK * L_OUT_PITCH * 4 <= L_LDS_BYTES, "the output tile reuses the stages");

__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__global__ __launch_bounds__(L_THREADS) void k_gemm_q4k_f16_ls(const GemmParams p) {
    warm_kernel_arguments<sizeof(GemmParams)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const size_t tt = blockIdx.y;
    const size_t row0 = (size_t)blockIdx.x * L_WROWS;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nblk = (int)(b1 - b0);

    floatx16 total[2][2];  // [row tile][token tile], compute wavefronts only
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                total[t][a][r] = 0.0f;
            }
        }
    }
    const int kg = (wave >> 1) & 1, rg = wave & 1;
    const int j = lane & 31, kh = lane >> 5;

    if (wave >= L_COMPUTE) {
        // ------------------------------------------------------------------------------------------------ loaders
        const int L = wave - L_COMPUTE;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
        const uint8_t *tile_x = (const uint8_t *)(p.x + tt * L_TOK * p.K);
        const uint32_t row_pitch = (uint32_t)(p.K * 2);
        const uint32_t last_row = (uint32_t)(p.N - 1 - tt * L_TOK);  // token rows beyond it re-read it
        // Activation tile: token t of the tile owns 512 bytes of the stage as 32 chunks of 16 bytes, chunk c stored in
        // slot c ^ (t % 16) (the MFMA operand reads of 16 tokens x one chunk then fall into 16 different bank groups).
        // Loader L brings tokens 16 L .. 16 L + 15, two per instruction.
        uint32_t a_voff[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t t = (uint32_t)(16 * L + 2 * c + (lane >> 5));
            const uint32_t slot = (uint32_t)(lane & 31);
            const uint32_t trow = t < last_row ? t : last_row;
            a_voff[c] = trow * row_pitch + 16u * (slot ^ (t & 15u));
        }
        // Weight blocks: piece q of the stage is 16 bytes q % 9 of tile row q / 9; loader L brings pieces
        // 256 pass + 64 L + lane. Rows beyond M re-read row M - 1 (never stored).
        const size_t row_bytes = p.nb * Q4_K_BYTES;
        const uint32_t last_wrow = (uint32_t)(p.M - 1 - row0);
        uint32_t w_voff[5];
#pragma unroll
        for (int pass = 0; pass < 5; ++pass) {
            const uint32_t q = (uint32_t)(256 * pass + 64 * L + lane);
            const uint32_t r = q / 9u, c9 = q - 9u * r;
            const uint32_t rr = r < last_wrow ? r : last_wrow;
            w_voff[pass] = rr * (uint32_t)row_bytes + 16u * c9;
        }
        const uint8_t *wbase = p.w + row0 * row_bytes;
        const bool fifth = L < 2;  // pieces 1024 .. 1151
        const int per_block = fifth ? 13 : 12;
        auto issue = [&](size_t b, int stage) {
            const uint32_t s0 = lds_base + (uint32_t)(stage * L_STAGE);
            const uint8_t *xb = tile_x + b * 512;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                dma_set_lds_base(s0 + (uint32_t)(8192 * L + 1024 * c));
                dma16_to_lds<0>(xb, a_voff[c]);
            }
            const uint8_t *wb = wbase + b * Q4_K_BYTES;
#pragma unroll
            for (int pass = 0; pass < 4; ++pass) {
                dma_set_lds_base(s0 + (uint32_t)(L_STAGE_A + (256 * pass + 64 * L) * 16));
                dma16_to_lds<0>(wb, w_voff[pass]);
            }
            if (fifth) {
                dma_set_lds_base(s0 + (uint32_t)(L_STAGE_A + (1024 + 64 * L) * 16));
                dma16_to_lds<0>(wb, w_voff[4]);
            }
        };
        // Sub-block sums of this loader's 16 tokens: lane -> token 16 L + lane % 16, sub-blocks 2 (lane / 16) and + 1.
        const int st = 16 * L + (lane & 15), pair = lane >> 4;
        const uint32_t sum_dst = (uint32_t)(L_STAGE_A + L_STAGE_W + (st >> 5) * 1024 + (st & 31) * 16 + 4 * pair);
        auto sums = [&](int stage) {
            uint8_t *sa = lds + (size_t)stage * L_STAGE;
            float s0 = 0.0f, s1 = 0.0f;
            const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint4 v = *(const uint4 *)(sa + st * 512 + 16 * ((8 * pair + c) ^ (st & 15)));
                float acc = c < 4 ? s0 : s1;
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.x), ones, acc, false);
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.y), ones, acc, false);
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.z), ones, acc, false);
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.w), ones, acc, false);
                if (c < 4) {
                    s0 = acc;
                } else {
                    s1 = acc;
                }
            }
            s0 *= 0.03125f;  // exact; keeps the value within fp16 range whatever the activations are
            s1 *= 0.03125f;
            const uint16_t h0 = f2h(s0), h1 = f2h(s1);
            const uint16_t l0 = f2h(s0 - h2f(h0)), l1 = f2h(s1 - h2f(h1));
            // S operand of token sub-tile a: lane i holds the 8 hi parts of token 32 a + i, lane 32 + i the lo parts
            *(uint32_t *)(sa + sum_dst) = (uint32_t)h0 | ((uint32_t)h1 << 16);
            *(uint32_t *)(sa + sum_dst + 512) = (uint32_t)l0 | ((uint32_t)l1 << 16);
        };

        issue(b0, 0);
        if (nblk > 1) {
            issue(b0 + 1, 1);
        }
        wait_vmcnt_at_most(nblk > 1 ? per_block : 0);
        lds_barrier();
        for (int i = 0; i < nblk; ++i) {
            if (i + 2 < nblk) {
                issue(b0 + (size_t)i + 2, (i + 2) % L_STAGES);
            }
            // The sums of block i, whose tile is complete since the barrier that opened this round, while block i + 1
            // is still landing; the compute wavefronts take them one block late (the Q product of block i runs behind
            // the next barrier), so nobody waits for them inside the round.
            compiler_memory_fence();
            sums(i % L_STAGES);
            if (i + 1 < nblk) {
                wait_vmcnt_at_most(i + 2 < nblk ? per_block : 0);
            }
            lds_barrier();
        }
    } else {
        // ------------------------------------------------------------------------------------------------ compute
        // MFMA A operand of K-step 8 kg + i, token sub-tile a, lane (j, kh): token 32 a + j, chunk
        // 16 kg + 4 (i / 2) + 2 kh + i % 2 of the token's 32.
        uint32_t a_off[4][2];
#pragma unroll
        for (int s3 = 0; s3 < 4; ++s3) {
#pragma unroll
            for (int tp = 0; tp < 2; ++tp) {
                a_off[s3][tp] = (uint32_t)(j * 512 + 256 * kg + 16 * ((4 * s3 + 2 * kh + tp) ^ (j & 15)));
            }
        }
        // this lane's two weight rows (row tiles 0 and 1) inside the stage, and the offset of its 16 bytes of 64-value
        // group 2 kg inside a block (+ 32: group 2 kg + 1)
        const uint32_t w_off0 = (uint32_t)(L_STAGE_A + (64 * rg + j) * Q4_K_BYTES);
        const uint32_t q_off = (uint32_t)(16 + 64 * kg + 16 * kh);

        // Q product of a block, all eight sub-blocks: row tile kg by the wavefronts of K half kg, one block late
        uint32_t prev_mn_lo = 0, prev_mn_hi = 0;
        float prev_ndmin = 0.0f;
        auto q_term = [&](const uint8_t *stage_s, floatx16(&tot)[2]) {
            const half8 b2 = mins_operand(prev_mn_lo, prev_mn_hi);
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const half8 a2 = __builtin_bit_cast(half8, *(const uint4 *)(stage_s + ((size_t)a * 64 + lane) * 16));
                const floatx16 zero = {0};
                const floatx16 mq = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b2, zero, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    tot[a][r] = __builtin_fmaf(prev_ndmin, mq[r], tot[a][r]);
                }
            }
        };

        lds_barrier();
        for (int blk = 0; blk < nblk; ++blk) {
            const uint8_t *stage = lds + (size_t)(blk % L_STAGES) * L_STAGE;
            Scales sc[2];
            uint4 wq[2][2];
            uint32_t scw[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint8_t *wr = stage + w_off0 + t * 32 * Q4_K_BYTES;
                const uint4 hdr = *(const uint4 *)wr;
                wq[t][0] = *(const uint4 *)(wr + q_off);
                wq[t][1] = *(const uint4 *)(wr + q_off + 32);
                decode_header(hdr, sc[t]);
                scw[t] = kg ? sc[t].sc_hi : sc[t].sc_lo;
            }
            __half2 scp[2], cp[2];
            uint32_t m0[2] = {0, 0}, m1[2] = {0, 0};
            // piece `piece` of B operand t for this wavefront's K-step i (sub-block 4 kg + i / 2, half i % 2)
            auto b_piece = [&](int t, int i, int piece) -> uint32_t {
                const int s_ = i >> 1, tp = i & 1, gi = i >> 2;
                if (piece == 0) {
                    if (tp == 0) {
                        const uint32_t sel = s_ == 0 ? 0x04000400u : s_ == 1 ? 0x04010401u
                                           : s_ == 2 ? 0x04020402u : 0x04030403u;
                        scp[t] = __hsub2(as_h2(__builtin_amdgcn_perm(0x64646464u, scw[t], sel)), as_h2(0x64006400u));
                        cp[t] = __hmul2(scp[t], as_h2(0xe400e400u));  // -1024 * sc, exact
                    }
                    const uint32_t q0 = tp ? wq[t][gi].z : wq[t][gi].x;
                    const uint32_t q1 = tp ? wq[t][gi].w : wq[t][gi].y;
                    m0[t] = ((s_ & 1) ? (q0 >> 4) : q0) & 0x0f0f0f0fu;
                    m1[t] = ((s_ & 1) ? (q1 >> 4) : q1) & 0x0f0f0f0fu;
                }
                switch (piece) {
                case 0: return dequant_pair<0>(m0[t], scp[t], cp[t]);
                case 1: return dequant_pair<1>(m0[t], scp[t], cp[t]);
                case 2: return dequant_pair<0>(m1[t], scp[t], cp[t]);
                default: return dequant_pair<1>(m1[t], scp[t], cp[t]);
                }
            };
            auto read_a = [&](int i, half8(&aop)[2]) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    aop[a] = __builtin_bit_cast(half8, *(const uint4 *)(stage + a_off[i >> 1][i & 1] + a * 16384));
                }
            };

            floatx16 acc[2][2];
            half8 aop[2][2];       // A operands of the K-step in flight and of the next one
            uint32_t bop[2][2][4];  // B operands likewise
            read_a(0, aop[0]);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int piece = 0; piece < 4; ++piece) {
                    bop[0][t][piece] = b_piece(t, 0, piece);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = i & 1, n = c ^ 1;
                if (i < 7) {
                    read_a(i + 1, aop[n]);  // lands while the MFMAs below run
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const half8 bcur =
                        __builtin_bit_cast(half8, make_uint4(bop[c][t][0], bop[c][t][1], bop[c][t][2], bop[c][t][3]));
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
                        if (i == 0) {
                            const floatx16 zero = {0};
                            acc[t][a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[c][a], bcur, zero, 0, 0, 0);
                        } else {
                            acc[t][a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[c][a], bcur, acc[t][a], 0, 0, 0);
                        }
                        if (i < 7) {  // the next K-step's B operands, two pieces in the shadow of each MFMA
                            bop[n][t][2 * a] = b_piece(t, i + 1, 2 * a);
                            bop[n][t][2 * a + 1] = b_piece(t, i + 1, 2 * a + 1);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            // per-block scale of the P product
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        total[t][a][r] = __builtin_fmaf(sc[t].d, acc[t][a][r], total[t][a][r]);
                    }
                }
            }
            // Q product of the previous block: its sums were written during the previous round and are complete since the
            // barrier that opened this one; its stage's tile and weights are being refilled, its S area is not
            if (blk > 0) {
                const uint8_t *prev_s = lds + (size_t)((blk - 1) % L_STAGES) * L_STAGE + L_STAGE_A + L_STAGE_W;
                if (kg == 0) {
                    q_term(prev_s, total[0]);
                } else {
                    q_term(prev_s, total[1]);
                }
            }
            prev_mn_lo = kg ? sc[1].mn_lo : sc[0].mn_lo;
            prev_mn_hi = kg ? sc[1].mn_hi : sc[0].mn_hi;
            prev_ndmin = -(kg ? sc[1].dmin : sc[0].dmin);
            lds_barrier();
        }
        {   // the last block's Q product: its sums are complete since the loop's last barrier
            const uint8_t *last_s = lds + (size_t)((nblk - 1) % L_STAGES) * L_STAGE + L_STAGE_A + L_STAGE_W;
            if (kg == 0) {
                q_term(last_s, total[0]);
            } else {
                q_term(last_s, total[1]);
            }
        }
    }

    // ---- the two K halves meet in LDS as one [token][weight row] tile, then every thread stores 16 bytes per step.
    // Lane (j, kh) of compute wavefront (kg, rg) holds weight row 64 rg + 32 t + j for tokens
    // 32 a + 8 (r / 4) + 4 kh + r % 4.
    float *tile = (float *)lds;
    if (wave < L_COMPUTE && kg == 1) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    tile[(32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * L_OUT_PITCH + 64 * rg + 32 * t + j] = total[t][a][r];
                }
            }
        }
    }
    lds_barrier();
    if (wave < L_COMPUTE && kg == 0) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float *e = tile + (32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * L_OUT_PITCH + 64 * rg + 32 * t + j;
                    *e = total[t][a][r] + *e;
                }
            }
        }
    }
    lds_barrier();

    const bool partials = p.splits > 1;
    const bool has_bias = !partials && p.bias != nullptr;
    const bool out_f16 = !partials && p.out_is_f16;
    float *const out32 = (float *)p.out + (partials ? (size_t)split * p.N * p.M : 0);
    const bool vec = (p.M & 3) == 0 && (((uintptr_t)p.out) & 15) == 0;
    for (int idx = tid; idx < L_TOK * L_WROWS / 4; idx += L_THREADS) {
        const int t = idx >> 5, q4 = idx & 31;  // rows 4 q4 .. 4 q4 + 3 of token t
        const size_t n = tt * L_TOK + (size_t)t;
        const size_t m4 = row0 + 4 * (size_t)q4;
        if (n >= p.N || m4 >= p.M) {
            continue;
        }
        const float4 v = *(const float4 *)(tile + t * L_OUT_PITCH + 4 * q4);
        const float e4[4] = {v.x, v.y, v.z, v.w};
        float bias4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (has_bias) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (m4 + e < p.M) {
                    bias4[e] = p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[m4 + e]) : ((const float *)p.bias)[m4 + e];
                }
            }
        }
        if (!out_f16) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                o[e] = has_bias ? e4[e] + bias4[e] : e4[e];
            }
            float *dst = out32 + n * p.M + m4;
            if (vec) {  // M % 4 == 0: the four rows exist
                *(float4 *)dst = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (m4 + e < p.M) {
                        dst[e] = o[e];
                    }
                }
            }
        } else {
            uint16_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                h[e] = f2h(e4[e]);  // round to the output type first, then add the bias in it
                if (has_bias) {
                    h[e] = f2h(h2f(h[e]) + bias4[e]);
                }
            }
            uint16_t *dst = (uint16_t *)p.out + n * p.M + m4;
            if (vec) {
                *(uint2 *)dst = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (m4 + e < p.M) {
                        dst[e] = h[e];
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------ 128 tokens x 128 weight rows, loader wavefronts
// The tile above spends most of the SIMD's issue slots on vector instructions that do not depend on the number of
// tokens (the nibble unpack: 200 of 400 per block and wavefront). Here one unpacked weight operand feeds FOUR matrix
// instructions: a compute wavefront owns 64 weight rows x all 128 tokens (2 x 4 tiles) and one K quarter of every
// half-block. 128 accumulator registers per wavefront leave no room for a second set, so the block scale d is not
// applied to a per-block product afterwards; the running tile T is kept in units of the current block's d instead:
//     T <- T * (d_prev / d_b)        once per block, then the block's matrix instructions accumulate sc*q . x onto T,
// and the min term of block b - 1 enters as -(dmin_(b-1) / d_b) * Q. Blocks with d == 0 keep the unit and run with
// zero scales. Against the tile above this costs two more roundings per block and element (the ratio and the rescale),
// the same order as the fp32 accumulation itself.
//   * A round is HALF a block (128 values of K): three LDS stages of 128 tokens x 256 bytes of activations and
//     128 rows x 80 bytes of weights (the 16-byte header and the 64 bytes of quants of this half), two rounds ahead.
//   * wavefronts 4..7 load (32 tokens and a share of the weight pieces each) and compute the sub-block sums of the
//     round in work; the sums of a block sit in one of two 4 KiB areas and are used one block late.
//   * wavefronts 0..3 compute: (rg = rows 64 rg .. + 63, kg = the 64-value group 2 h + kg of the block in round h).
// 512 tokens x 4096 rows are 128 such tiles; K is then split over two workgroups per tile.
constexpr int W_TOK = 128;
constexpr int W_WROWS = 128;
constexpr int W_THREADS = 512;
constexpr int W_STAGE_A = W_TOK * 256;              // 32,768
constexpr int W_ROW = 80;                           // header + the quants of one half
constexpr int W_STAGE_W = W_WROWS * W_ROW;          // 10,240
constexpr int W_STAGE = W_STAGE_A + W_STAGE_W;
constexpr int W_STAGES = 3;
constexpr int W_SUMS = 4 * 64 * 16;                 // sub-block sums operand of the four token sub-tiles of one block
constexpr int W_LDS_BYTES = W_STAGES * W_STAGE + 2 * W_SUMS;   // 137,216
constexpr int W_OUT_PITCH = W_WROWS + 4;
static_assert(W_TOK * W_OUT_PITCH * 4 <= W_STAGES * W_STAGE, "the output tile reuses the stages");

__global__ __launch_bounds__(W_THREADS) void k_gemm_q4k_f16_wide(const GemmParams p) {
    warm_kernel_arguments<sizeof(GemmParams)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const size_t tt = blockIdx.y;
    const size_t row0 = (size_t)blockIdx.x * W_WROWS;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nblk = (int)(b1 - b0);
    const int nr = 2 * nblk;

    floatx16 T[2][4];  // [row tile][token tile], compute wavefronts only
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                T[t][a][r] = 0.0f;
            }
        }
    }
    const int kg = (wave >> 1) & 1, rg = wave & 1;
    const int j = lane & 31, kh = lane >> 5;
    uint8_t *const sums_area = lds + W_STAGES * W_STAGE;

    if (wave >= 4) {
        // ------------------------------------------------------------------------------------------------ loaders
        const int L = wave - 4;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
        const uint8_t *tile_x = (const uint8_t *)(p.x + tt * W_TOK * p.K) + b0 * 512;
        const uint32_t row_pitch = (uint32_t)(p.K * 2);
        const uint32_t last_row = (uint32_t)(p.N - 1 - tt * W_TOK);  // token rows beyond it re-read it
        // Activations: token t of the tile owns 256 bytes of the stage as 16 chunks of 16 bytes, chunk c stored in slot
        // c ^ (t % 16). Loader L brings tokens 32 L .. 32 L + 31, four per instruction.
        uint32_t a_voff[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t t = (uint32_t)(32 * L + 4 * c + (lane >> 4));
            const uint32_t slot = (uint32_t)(lane & 15);
            const uint32_t trow = t < last_row ? t : last_row;
            a_voff[c] = trow * row_pitch + 16u * (slot ^ (t & 15u));
        }
        // Weights: piece q of the stage is 16 bytes q % 5 of tile row q / 5 (0: header, 1..4: the quants of this half);
        // loader L brings pieces 64 (L + 4 pass) + lane. Rows beyond M re-read row M - 1 (never stored).
        const size_t row_bytes = p.nb * Q4_K_BYTES;
        const uint32_t last_wrow = (uint32_t)(p.M - 1 - row0);
        uint32_t w_voff[3], w_half[3];
#pragma unroll
        for (int pass = 0; pass < 3; ++pass) {
            const uint32_t q = (uint32_t)(64 * (L + 4 * pass) + lane);
            const uint32_t r = q / 5u, c5 = q - 5u * r;
            const uint32_t rr = r < last_wrow ? r : last_wrow;
            w_voff[pass] = rr * (uint32_t)row_bytes + (c5 == 0 ? 0u : 16u * c5);
            w_half[pass] = c5 == 0 ? 0u : 64u;
        }
        const uint8_t *wbase = p.w + row0 * row_bytes + b0 * Q4_K_BYTES;
        const bool third = L < 2;  // pieces 512 .. 639
        const int per_round = third ? 11 : 10;
        auto issue = [&](int round, int stage) {
            const uint32_t s0 = lds_base + (uint32_t)(stage * W_STAGE);
            const uint8_t *xb = tile_x + (size_t)round * 256;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                dma_set_lds_base(s0 + (uint32_t)(8192 * L + 1024 * c));
                dma16_to_lds<0>(xb, a_voff[c]);
            }
            const uint8_t *wb = wbase + (size_t)(round >> 1) * Q4_K_BYTES;
            const uint32_t hsel = (round & 1) ? 0xffffffffu : 0u;
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                dma_set_lds_base(s0 + (uint32_t)(W_STAGE_A + 1024 * (L + 4 * pass)));
                dma16_to_lds<0>(wb, w_voff[pass] + (w_half[pass] & hsel));
            }
            if (third) {
                dma_set_lds_base(s0 + (uint32_t)(W_STAGE_A + 1024 * (L + 8)));
                dma16_to_lds<0>(wb, w_voff[2] + (w_half[2] & hsel));
            }
        };
        // Sub-block sums of this loader's 32 tokens: lane -> token 32 L + lane % 32, sub-blocks 2 (lane / 32) and + 1 of
        // the half in work.
        const int st = 32 * L + (lane & 31), pair = lane >> 5;
        const uint32_t sum_dst = (uint32_t)(L * 1024 + (lane & 31) * 16 + 4 * pair);
        auto sums = [&](int round, int stage) {
            const uint8_t *sa = lds + (size_t)stage * W_STAGE;
            float s0 = 0.0f, s1 = 0.0f;
            const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint4 v = *(const uint4 *)(sa + st * 256 + 16 * ((8 * pair + c) ^ (st & 15)));
                float acc = c < 4 ? s0 : s1;
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.x), ones, acc, false);
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.y), ones, acc, false);
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.z), ones, acc, false);
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v.w), ones, acc, false);
                if (c < 4) {
                    s0 = acc;
                } else {
                    s1 = acc;
                }
            }
            s0 *= 0.03125f;  // exact; keeps the value within fp16 range whatever the activations are
            s1 *= 0.03125f;
            const uint16_t h0 = f2h(s0), h1 = f2h(s1);
            const uint16_t l0 = f2h(s0 - h2f(h0)), l1 = f2h(s1 - h2f(h1));
            // S operand of token sub-tile a = L: lane i holds the 8 hi parts of token 32 a + i, lane 32 + i the lo parts
            uint8_t *dst = sums_area + ((round >> 1) & 1) * W_SUMS + sum_dst + 8 * (round & 1);
            *(uint32_t *)dst = (uint32_t)h0 | ((uint32_t)h1 << 16);
            *(uint32_t *)(dst + 512) = (uint32_t)l0 | ((uint32_t)l1 << 16);
        };

        issue(0, 0);
        issue(1, 1);
        wait_vmcnt_at_most(per_round);
        lds_barrier();
        for (int i = 0; i < nr; ++i) {
            if (i + 2 < nr) {
                issue(i + 2, (i + 2) % W_STAGES);
            }
            compiler_memory_fence();
            sums(i, i % W_STAGES);
            if (i + 1 < nr) {
                wait_vmcnt_at_most(i + 2 < nr ? per_round : 0);
            }
            lds_barrier();
        }
    } else {
        // ------------------------------------------------------------------------------------------------ compute
        // MFMA A operand of K-step i4 = 2 s + tp of a round (s: low / high nibbles = sub-block 2 g / 2 g + 1 of the
        // wavefront's 64-value group g), token sub-tile a, lane (j, kh): token 32 a + j, chunk
        // 8 kg + 4 s + 2 kh + tp of the token's 16.
        uint32_t a_off[4];
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            a_off[i4] = (uint32_t)(j * 256 + 16 * ((8 * kg + 4 * (i4 >> 1) + 2 * kh + (i4 & 1)) ^ (j & 15)));
        }
        const uint32_t w_off0 = (uint32_t)(W_STAGE_A + (64 * rg + j) * W_ROW);
        const uint32_t q_off = (uint32_t)(16 + 32 * kg + 16 * kh);

        float d_eff[2] = {1.0f, 1.0f};  // the unit of T[t]
        uint32_t prev_mn_lo = 0, prev_mn_hi = 0;
        float prev_ndmin = 0.0f;
        // Q product of a block, all eight sub-blocks: row tile kg by the wavefronts of K quarter kg, one block late
        auto q_term = [&](const uint8_t *s_area, float coeff, floatx16(&tot)[4]) {
            const half8 b2 = mins_operand(prev_mn_lo, prev_mn_hi);
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const half8 a2 = __builtin_bit_cast(half8, *(const uint4 *)(s_area + ((size_t)a * 64 + lane) * 16));
                const floatx16 zero = {0};
                const floatx16 mq = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b2, zero, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    tot[a][r] = __builtin_fmaf(coeff, mq[r], tot[a][r]);
                }
            }
        };

        auto round_fn = [&](int bb, int h) {
            const int round = 2 * bb + h;
            const uint8_t *stage = lds + (size_t)(round % W_STAGES) * W_STAGE;
            uint4 wq[2];
            uint32_t scw[2];
            uint32_t mn_lo_t[2], mn_hi_t[2];
            float dmin_t[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint8_t *wr = stage + w_off0 + t * 32 * W_ROW;
                const uint4 hdr = *(const uint4 *)wr;
                wq[t] = *(const uint4 *)(wr + q_off);
                Scales sc;
                decode_header(hdr, sc);
                const bool dead = sc.d == 0.0f;
                if (h == 0) {
                    const float dn = dead ? d_eff[t] : sc.d;
                    const float ratio = d_eff[t] / dn;
                    d_eff[t] = dn;
                    if (bb > 0) {
#pragma unroll
                        for (int a = 0; a < 4; ++a) {
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                T[t][a][r] *= ratio;
                            }
                        }
                    }
                }
                const uint32_t word = h ? sc.sc_hi : sc.sc_lo;
                scw[t] = dead ? 0u : (kg ? word >> 16 : word);
                mn_lo_t[t] = sc.mn_lo;
                mn_hi_t[t] = sc.mn_hi;
                dmin_t[t] = sc.dmin;
            }
            if (h == 0 && bb > 0) {
                const uint8_t *prev_s = sums_area + ((bb - 1) & 1) * W_SUMS;
                if (kg == 0) {
                    q_term(prev_s, prev_ndmin / d_eff[0], T[0]);
                } else {
                    q_term(prev_s, prev_ndmin / d_eff[1], T[1]);
                }
            }
            if (h == 1) {
                prev_mn_lo = kg ? mn_lo_t[1] : mn_lo_t[0];
                prev_mn_hi = kg ? mn_hi_t[1] : mn_hi_t[0];
                prev_ndmin = -(kg ? dmin_t[1] : dmin_t[0]);
            }

            __half2 scp[2], cp[2];
            uint32_t m0[2] = {0, 0}, m1[2] = {0, 0};
            // piece `piece` of B operand t for K-step i4 (nibble half s = i4 / 2, byte half tp = i4 % 2)
            auto b_piece = [&](int t, int i4, int piece) -> uint32_t {
                const int s_ = i4 >> 1, tp = i4 & 1;
                if (piece == 0) {
                    if (tp == 0) {
                        const uint32_t sel = s_ == 0 ? 0x04000400u : 0x04010401u;
                        scp[t] = __hsub2(as_h2(__builtin_amdgcn_perm(0x64646464u, scw[t], sel)), as_h2(0x64006400u));
                        cp[t] = __hmul2(scp[t], as_h2(0xe400e400u));  // -1024 * sc, exact
                    }
                    const uint32_t q0 = tp ? wq[t].z : wq[t].x;
                    const uint32_t q1 = tp ? wq[t].w : wq[t].y;
                    m0[t] = (s_ ? (q0 >> 4) : q0) & 0x0f0f0f0fu;
                    m1[t] = (s_ ? (q1 >> 4) : q1) & 0x0f0f0f0fu;
                }
                switch (piece) {
                case 0: return dequant_pair<0>(m0[t], scp[t], cp[t]);
                case 1: return dequant_pair<1>(m0[t], scp[t], cp[t]);
                case 2: return dequant_pair<0>(m1[t], scp[t], cp[t]);
                default: return dequant_pair<1>(m1[t], scp[t], cp[t]);
                }
            };
            auto read_a = [&](int i4, half8(&aop)[4]) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    aop[a] = __builtin_bit_cast(half8, *(const uint4 *)(stage + a_off[i4] + a * 8192));
                }
            };

            half8 aop[2][4];
            uint32_t bop[2][2][4];
            read_a(0, aop[0]);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int piece = 0; piece < 4; ++piece) {
                    bop[0][t][piece] = b_piece(t, 0, piece);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int c = i4 & 1, n = c ^ 1;
                if (i4 < 3) {
                    read_a(i4 + 1, aop[n]);  // lands while the MFMAs below run
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const half8 bcur =
                        __builtin_bit_cast(half8, make_uint4(bop[c][t][0], bop[c][t][1], bop[c][t][2], bop[c][t][3]));
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        T[t][a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[c][a], bcur, T[t][a], 0, 0, 0);
                        if (i4 < 3) {  // the next K-step's B operands, one piece in the shadow of each MFMA
                            bop[n][t][a] = b_piece(t, i4 + 1, a);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        };

        lds_barrier();
        for (int bb = 0; bb < nblk; ++bb) {
            round_fn(bb, 0);
            lds_barrier();
            round_fn(bb, 1);
            lds_barrier();
        }
        // leave the unit: T[t] in plain numbers, then the last block's Q product (its sums are complete since the last
        // barrier)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    T[t][a][r] *= d_eff[t];
                }
            }
        }
        {
            const uint8_t *last_s = sums_area + ((nblk - 1) & 1) * W_SUMS;
            if (kg == 0) {
                q_term(last_s, prev_ndmin, T[0]);
            } else {
                q_term(last_s, prev_ndmin, T[1]);
            }
        }
    }

    // ---- the two K quarters meet in LDS as one [token][weight row] tile, then every thread stores 16 bytes per step.
    // Lane (j, kh) of compute wavefront (kg, rg) holds weight row 64 rg + 32 t + j for tokens
    // 32 a + 8 (r / 4) + 4 kh + r % 4.
    float *tile = (float *)lds;
    if (wave < 4 && kg == 1) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    tile[(32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * W_OUT_PITCH + 64 * rg + 32 * t + j] = T[t][a][r];
                }
            }
        }
    }
    lds_barrier();
    if (wave < 4 && kg == 0) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float *e = tile + (32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * W_OUT_PITCH + 64 * rg + 32 * t + j;
                    *e = T[t][a][r] + *e;
                }
            }
        }
    }
    lds_barrier();

    const bool partials = p.splits > 1;
    const bool has_bias = !partials && p.bias != nullptr;
    const bool out_f16 = !partials && p.out_is_f16;
    float *const out32 = (float *)p.out + (partials ? (size_t)split * p.N * p.M : 0);
    const bool vec = (p.M & 3) == 0 && (((uintptr_t)p.out) & 15) == 0;
    for (int idx = tid; idx < W_TOK * W_WROWS / 4; idx += W_THREADS) {
        const int t = idx >> 5, q4 = idx & 31;  // rows 4 q4 .. 4 q4 + 3 of token t
        const size_t n = tt * W_TOK + (size_t)t;
        const size_t m4 = row0 + 4 * (size_t)q4;
        if (n >= p.N || m4 >= p.M) {
            continue;
        }
        const float4 v = *(const float4 *)(tile + t * W_OUT_PITCH + 4 * q4);
        const float e4[4] = {v.x, v.y, v.z, v.w};
        float bias4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (has_bias) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (m4 + e < p.M) {
                    bias4[e] = p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[m4 + e]) : ((const float *)p.bias)[m4 + e];
                }
            }
        }
        if (!out_f16) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                o[e] = has_bias ? e4[e] + bias4[e] : e4[e];
            }
            float *dst = out32 + n * p.M + m4;
            if (vec) {  // M % 4 == 0: the four rows exist
                *(float4 *)dst = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (m4 + e < p.M) {
                        dst[e] = o[e];
                    }
                }
            }
        } else {
            uint16_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                h[e] = f2h(e4[e]);  // round to the output type first, then add the bias in it
                if (has_bias) {
                    h[e] = f2h(h2f(h[e]) + bias4[e]);
                }
            }
            uint16_t *dst = (uint16_t *)p.out + n * p.M + m4;
            if (vec) {
                *(uint2 *)dst = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (m4 + e < p.M) {
                        dst[e] = h[e];
                    }
                }
            }
        }
    }
}

// sums the K-split partials in split order, then bias / output cast like the single-pass epilogue
template <int V>
__global__ __launch_bounds__(256) void k_gemm_reduce(const float *__restrict__ partial, int splits, size_t N, size_t M,
                                                     const void *bias, int bias_is_f16, void *out, int out_is_f16,
                                                     int bias_first) {
    warm_kernel_arguments<8 * 8 + 4, 8 * 8 + 4>();
    const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
    const size_t total = N * M;
    if (idx >= total) {
        return;
    }
    float v[V];
#pragma unroll
    for (int e = 0; e < V; ++e) {
        v[e] = 0.0f;
    }
    // loads of 4 splits are issued together (one memory latency per 4 splits); the additions stay in split order
    for (int s0 = 0; s0 < splits; s0 += 4) {
        float4 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = s0 + u < splits ? s0 + u : splits - 1;
            const float *src = partial + (size_t)s * total + idx;
            if (V == 4) {
                t[u] = *(const float4 *)src;
            } else {
                t[u] = make_float4(src[0], 0.0f, 0.0f, 0.0f);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (s0 + u < splits) {
                v[0] += t[u].x;
                v[1 % V] += t[u].y;
                v[2 % V] += t[u].z;
                v[3 % V] += t[u].w;
            }
        }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
        const size_t m = (idx + e) % M;
        float bv = 0.0f;
        if (bias != nullptr) {
            bv = bias_is_f16 ? h2f(((const uint16_t *)bias)[m]) : ((const float *)bias)[m];
        }
        if (!out_is_f16) {
            ((float *)out)[idx + e] = bias != nullptr ? v[e] + bv : v[e];
        } else if (bias_first) {
            ((uint16_t *)out)[idx + e] = f2h(bias != nullptr ? v[e] + bv : v[e]);
        } else {
            uint16_t h = f2h(v[e]);
            if (bias != nullptr) {
                h = f2h(h2f(h) + bv);
            }
            ((uint16_t *)out)[idx + e] = h;
        }
    }
}

int launch_splitk_reduce(marmot_hip_device *dev, const float *partial, int splits, size_t N, size_t M,
                         const void *d_bias, int bias_dtype, void *d_out, int out_dtype, bool bias_first) {
    const size_t total = N * M;
    const int bias_is_f16 = bias_dtype == MARMOT_HIP_DTYPE_F16, out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    // small outputs: one wavefront per workgroup, so that the few thousand threads spread over the whole chip
    const bool vec = total % 4 == 0 && M % 4 == 0;
    const size_t threads = vec ? total / 4 : total;
    const unsigned block = threads < 65536 ? 64u : 256u;
    const dim3 grid((unsigned)((threads + block - 1) / block));
    if (vec) {
        hipLaunchKernelGGL(k_gemm_reduce<4>, grid, dim3(block), 0, dev->stream, partial, splits, N, M, d_bias,
                           bias_is_f16, d_out, out_is_f16, bias_first ? 1 : 0);
    } else {
        hipLaunchKernelGGL(k_gemm_reduce<1>, grid, dim3(block), 0, dev->stream, partial, splits, N, M, d_bias,
                           bias_is_f16, d_out, out_is_f16, bias_first ? 1 : 0);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

bool gemm_f16_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M) {
    if (dev->knobs.no_gemm) {
        return false;
    }
    // every token count: a decode step with fp16 activations takes the 64-token tile with one token in it (14336 x
    // 4096 at 1 / 8 rows: 18.0 / 18.4 us; the fp16 matvec, four rows at a time, 70.9 / 175 us)
    return kind == MARMOT_HIP_KIND_Q4_K && N >= 1 && K % QK_K == 0 && M >= 1;
}

template <int TA, int KG>
static int launch_gemm_shape(marmot_hip_device *dev, GemmParams p, size_t N, size_t K, size_t M, const void *d_bias,
                             int bias_dtype, void *d_out, int out_dtype) {
    using S = GemmShape<TA, KG>;
    const size_t nb = K / QK_K;
    const size_t tiles_n = (N + S::TOK - 1) / S::TOK;
    const size_t tiles_m = (M + S::WROWS - 1) / S::WROWS;
    const size_t tiles = tiles_n * tiles_m;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t splits = 1;
    if (tiles * 2 <= cus) {  // fewer tiles than half the chip: split K across workgroups (short prompts)
        splits = cus / tiles;
        const size_t max_splits = nb / (2 * KG) > 0 ? nb / (2 * KG) : 1;  // at least two blocks per K group
        splits = splits > max_splits ? max_splits : splits;
    }
    const size_t blocks_per_split = (nb + splits - 1) / splits;
    splits = (nb + blocks_per_split - 1) / blocks_per_split;
    float *partial = nullptr;
    if (splits > 1) {
        void *ws = nullptr;
        MH_TRY(workspace_reserve(dev, splits * N * M * sizeof(float), &ws));
        partial = (float *)ws;
    }
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q4k_f16<TA, KG>));
    p.out = splits > 1 ? (void *)partial : d_out;
    p.splits = (int)splits;
    p.blocks_per_split = (int)blocks_per_split;
    hipLaunchKernelGGL((k_gemm_q4k_f16<TA, KG>), dim3((unsigned)tiles_m, (unsigned)tiles_n, (unsigned)splits),
                       dim3(G_THREADS), S::LDS_BYTES, dev->stream, p);
    MH_HIP(hipGetLastError());
    if (splits > 1) {
        MH_TRY(launch_splitk_reduce(dev, partial, (int)splits, N, M, d_bias, bias_dtype, d_out, out_dtype));
    }
    return MARMOT_HIP_SUCCESS;
}

static int launch_gemm_ls(marmot_hip_device *dev, GemmParams p, size_t N, size_t K, size_t M, const void *d_bias,
                          int bias_dtype, void *d_out, int out_dtype) {
    const size_t nb = K / QK_K;
    const size_t tiles_n = (N + L_TOK - 1) / L_TOK;
    const size_t tiles_m = (M + L_WROWS - 1) / L_WROWS;
    const size_t tiles = tiles_n * tiles_m;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t splits = 1;
    if (tiles * 2 <= cus) {  // fewer tiles than half the chip: split K across workgroups (short prompts)
        splits = cus / tiles;
        const size_t max_splits = nb / 2 > 0 ? nb / 2 : 1;  // at least two blocks per workgroup
        splits = splits > max_splits ? max_splits : splits;
    }
    const size_t blocks_per_split = (nb + splits - 1) / splits;
    splits = (nb + blocks_per_split - 1) / blocks_per_split;
    float *partial = nullptr;
    if (splits > 1) {
        void *ws = nullptr;
        MH_TRY(workspace_reserve(dev, splits * N * M * sizeof(float), &ws));
        partial = (float *)ws;
    }
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q4k_f16_ls));
    p.out = splits > 1 ? (void *)partial : d_out;
    p.splits = (int)splits;
    p.blocks_per_split = (int)blocks_per_split;
    hipLaunchKernelGGL(k_gemm_q4k_f16_ls, dim3((unsigned)tiles_m, (unsigned)tiles_n, (unsigned)splits),
                       dim3(L_THREADS), L_LDS_BYTES, dev->stream, p);
    MH_HIP(hipGetLastError());
    if (splits > 1) {
        MH_TRY(launch_splitk_reduce(dev, partial, (int)splits, N, M, d_bias, bias_dtype, d_out, out_dtype));
    }
    return MARMOT_HIP_SUCCESS;
}

static int launch_gemm_wide(marmot_hip_device *dev, GemmParams p, size_t N, size_t K, size_t M, const void *d_bias,
                            int bias_dtype, void *d_out, int out_dtype) {
    const size_t nb = K / QK_K;
    const size_t tiles_n = (N + W_TOK - 1) / W_TOK;
    const size_t tiles_m = (M + W_WROWS - 1) / W_WROWS;
    const size_t tiles = tiles_n * tiles_m;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t splits = 1;
    if (tiles * 2 <= cus) {  // fewer tiles than half the chip: split K across workgroups
        splits = cus / tiles;
        splits = splits > nb ? nb : splits;
    }
    const size_t blocks_per_split = (nb + splits - 1) / splits;
    splits = (nb + blocks_per_split - 1) / blocks_per_split;
    float *partial = nullptr;
    if (splits > 1) {
        void *ws = nullptr;
        MH_TRY(workspace_reserve(dev, splits * N * M * sizeof(float), &ws));
        partial = (float *)ws;
    }
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q4k_f16_wide));
    p.out = splits > 1 ? (void *)partial : d_out;
    p.splits = (int)splits;
    p.blocks_per_split = (int)blocks_per_split;
    hipLaunchKernelGGL(k_gemm_q4k_f16_wide, dim3((unsigned)tiles_m, (unsigned)tiles_n, (unsigned)splits),
                       dim3(W_THREADS), W_LDS_BYTES, dev->stream, p);
    MH_HIP(hipGetLastError());
    if (splits > 1) {
        MH_TRY(launch_splitk_reduce(dev, partial, (int)splits, N, M, d_bias, bias_dtype, d_out, out_dtype));
    }
    return MARMOT_HIP_SUCCESS;
}

static int launch_gemm_big(marmot_hip_device *dev, GemmParams p, size_t N, size_t K, size_t M, const void *d_bias,
                           int bias_dtype, void *d_out, int out_dtype) {
    const size_t nb = K / QK_K;
    const size_t tiles_n = (N + B_TOK - 1) / B_TOK;
    const size_t tiles_m = (M + B_WROWS_WG - 1) / B_WROWS_WG;
    const size_t tiles = tiles_n * tiles_m;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t splits = 1;
    if (tiles < cus) {
        splits = cus / tiles;
        splits = splits > nb ? nb : (splits < 1 ? 1 : splits);
    }
    const size_t blocks_per_split = (nb + splits - 1) / splits;
    splits = (nb + blocks_per_split - 1) / blocks_per_split;
    const size_t sums_bytes = tiles_n * nb * B_STAGE_S;
    const size_t partial_bytes = splits > 1 ? splits * N * M * sizeof(float) : 0;
    void *ws = nullptr;
    MH_TRY(workspace_reserve(dev, ((sums_bytes + 255) & ~(size_t)255) + partial_bytes, &ws));
    uint8_t *sums = (uint8_t *)ws;
    float *partial = (float *)((uint8_t *)ws + ((sums_bytes + 255) & ~(size_t)255));
    {
        const size_t total = tiles_n * B_TOK * nb * 8;
        hipLaunchKernelGGL(k_gemm_sums, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dev->stream,
                           (const uint16_t *)p.x, N, K, nb, sums);
        MH_HIP(hipGetLastError());
    }
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q4k_f16_big));
    p.sums = sums;
    p.out = splits > 1 ? (void *)partial : d_out;
    p.splits = (int)splits;
    p.blocks_per_split = (int)blocks_per_split;
    hipLaunchKernelGGL(k_gemm_q4k_f16_big, dim3((unsigned)tiles_m, (unsigned)tiles_n, (unsigned)splits),
                       dim3(G_THREADS), 2 * B_STAGE, dev->stream, p);
    MH_HIP(hipGetLastError());
    if (splits > 1) {
        MH_TRY(launch_splitk_reduce(dev, partial, (int)splits, N, M, d_bias, bias_dtype, d_out, out_dtype));
    }
    return MARMOT_HIP_SUCCESS;
}

int launch_gemm_f16(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K, size_t M,
                    const void *d_bias, int bias_dtype, void *d_out, int out_dtype) {
    if (!gemm_f16_supported(dev, kind, N, K, M)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "prefill GEMM: unsupported kind or shape");
    }
    if ((((uintptr_t)d_x) & 15) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "prefill GEMM: activations must be 16-byte aligned");
    }
    GemmParams p;
    p.w = (const uint8_t *)d_w;
    p.x = (const uint16_t *)d_x;
    p.sums = nullptr;
    p.K = K;
    p.out = d_out;
    p.bias = d_bias;
    p.bias_is_f16 = bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.N = N;
    p.M = M;
    p.nb = K / QK_K;
    p.splits = 1;
    p.blocks_per_split = (int)p.nb;
    // Large tiles when they fill the chip by themselves (long prompts), the 64 x 128 tile with the K split inside the
    // workgroup otherwise.
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    const size_t big_tiles = ((N + 127) / 128) * ((M + 255) / 256);
    const bool big = big_tiles >= cus;
    set_route("gemm_q4_k_f16_mfma");
    if (big) {
        return launch_gemm_big(dev, p, N, K, M, d_bias, bias_dtype, d_out, out_dtype);
    }
    // the loader-wavefront kernel moves 16-byte pieces of the weight blocks; K < 2^22 keeps its 32-bit offsets exact
    if (!dev->knobs.no_gemm_loaders && (((uintptr_t)d_w) & 15) == 0 && K < ((size_t)1 << 22)) {
        // 128 x 128 tiles when one round of them covers most of the chip with the whole K inside each workgroup
        // (513 .. 1024 tokens at 4096 rows): one unpacked weight operand then feeds four matrix instructions
        const size_t wide_tiles = ((N + W_TOK - 1) / W_TOK) * ((M + W_WROWS - 1) / W_WROWS);
        const size_t ls_tiles = ((N + L_TOK - 1) / L_TOK) * ((M + L_WROWS - 1) / L_WROWS);
        const bool wide = wide_tiles <= cus && 8 * wide_tiles >= 5 * cus && ls_tiles > cus;
        if (dev->knobs.gemm_wide || (wide && !dev->knobs.no_gemm_wide)) {
            set_route("gemm_q4_k_f16_mfma_wide");
            return launch_gemm_wide(dev, p, N, K, M, d_bias, bias_dtype, d_out, out_dtype);
        }
        return launch_gemm_ls(dev, p, N, K, M, d_bias, bias_dtype, d_out, out_dtype);
    }
    return launch_gemm_shape<2, 2>(dev, p, N, K, M, d_bias, bias_dtype, d_out, out_dtype);
}

} // namespace mh

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
// Tiling. A workgroup (4 wavefronts) owns 128 tokens x 256 weight rows; each wavefront owns 128 x 64 as 4 x 2 MFMA
// tiles, so one dequantized weight operand feeds 4 MFMAs. The activation tile of the current block (64 KiB, already
// in MFMA operand order) is staged through LDS and shared by the 4 wavefronts, double buffered. Weights are read
// straight from their GGUF blocks into registers, one block ahead, and unpacked with
// (q | 0x6400) as fp16 = 1024 + q, then fma(1024 + q, sc, -1024 * sc) = sc * q exactly.
// K is split across workgroups when there are too few tiles to fill the chip; partial sums meet in a small
// second kernel in a fixed order.
#include "mh_common.h"

#include <stdlib.h>

namespace mh {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int G_TOK = 128;        // tokens per workgroup tile
constexpr int G_WROWS_WAVE = 64;  // weight rows per wavefront
constexpr int G_WROWS_WG = 256;   // weight rows per workgroup
constexpr int STAGE_A = 16 * 4 * 64 * 16;  // 16 K-steps x 4 token sub-tiles x 64 lanes x 16 bytes
constexpr int STAGE_S = 4 * 64 * 16;       // sub-block sums operand: 4 token sub-tiles x 64 lanes x 16 bytes
constexpr int STAGE = STAGE_A + STAGE_S;   // 69,632 bytes per (token tile, block)
constexpr int STAGE_CHUNKS = STAGE / 16;   // 4352 = 17 per thread

// slot e of an operand's 8 halves holds the value whose byte index within the lane's 8-byte piece is PERM[e]:
// the nibble extraction below yields (byte0, byte2), (byte1, byte3), ...
__device__ __forceinline__ uint32_t half_bits(float f) {
    return (uint32_t)f2h(f);
}

// ------------------------------------------------------------------ activation packing
// X fp16 [N, K] -> per (token tile tt, block b): operands in MFMA order.
//   A operand (ks, a), lane (i = lane % 32, kh = lane / 32), slot e:
//       X[128*tt + 32*a + i][256*b + 32*(ks/2) + 16*kh + 8*(ks%2) + PERM[e]],  PERM = {0,2,1,3,4,6,5,7}
//   S operand a, lane (i, kh), slot e: kh == 0 ? hi : lo of (sum of X over sub-block e) / 32
// Tokens beyond N are zero.
__global__ __launch_bounds__(256) void k_gemm_pack_x(const uint16_t *__restrict__ x, size_t N, size_t K, size_t nb,
                                                     uint8_t *__restrict__ packed) {
    const size_t chunk = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // one 16-byte operand piece
    const size_t tiles = (N + G_TOK - 1) / G_TOK;
    const size_t total = tiles * nb * (STAGE_A / 16);
    if (chunk >= total) {
        return;
    }
    const size_t stage = chunk / (STAGE_A / 16);
    const int within = (int)(chunk % (STAGE_A / 16));
    const int lane = within & 63;
    const int a = (within >> 6) & 3;
    const int ks = within >> 8;
    const size_t tt = stage / nb, b = stage % nb;
    const int i = lane & 31, kh = lane >> 5;
    const size_t token = tt * G_TOK + 32 * a + i;
    uint4 out = make_uint4(0, 0, 0, 0);
    if (token < N) {
        const size_t k0 = b * 256 + 32 * (ks >> 1) + 16 * kh + 8 * (ks & 1);
        const uint4 v = *(const uint4 *)(x + token * K + k0);
        out.x = (v.x & 0xffffu) | (v.y << 16);
        out.y = (v.x >> 16) | (v.y & 0xffff0000u);
        out.z = (v.z & 0xffffu) | (v.w << 16);
        out.w = (v.z >> 16) | (v.w & 0xffff0000u);
    }
    *(uint4 *)(packed + stage * STAGE + (size_t)within * 16) = out;
}

__global__ __launch_bounds__(256) void k_gemm_pack_s(const uint16_t *__restrict__ x, size_t N, size_t K, size_t nb,
                                                     uint8_t *__restrict__ packed) {
    // one thread per (stage, a, i, e): sums one 32-value sub-block of one token
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t tiles = (N + G_TOK - 1) / G_TOK;
    const size_t total = tiles * nb * 4 * 32 * 8;
    if (idx >= total) {
        return;
    }
    const int e = (int)(idx & 7);
    const int i = (int)((idx >> 3) & 31);
    const int a = (int)((idx >> 8) & 3);
    const size_t stage = idx >> 10;
    const size_t tt = stage / nb, b = stage % nb;
    const size_t token = tt * G_TOK + 32 * a + i;
    float s = 0.0f;
    if (token < N) {
        const uint16_t *p = x + token * K + b * 256 + 32 * e;
        for (int t = 0; t < 32; ++t) {
            s += h2f(p[t]);
        }
    }
    s *= 0.03125f;  // exact; keeps the value within fp16 range whatever the activations are
    const uint16_t hi = f2h(s);
    const uint16_t lo = f2h(s - h2f(hi));
    uint16_t *base = (uint16_t *)(packed + stage * STAGE + STAGE_A + (size_t)a * 64 * 16);
    base[(size_t)i * 8 + e] = hi;          // lane i       (kh = 0)
    base[(size_t)(32 + i) * 8 + e] = lo;   // lane 32 + i  (kh = 1)
}

// ------------------------------------------------------------------ main kernel
struct GemmParams {
    const uint8_t *w;       // Q4_K blocks, M rows of nb blocks
    const uint8_t *packed;  // packed activations
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
    s.sc_lo = hdr.y & 0x3f3f3f3fu;
    s.mn_lo = hdr.z & 0x3f3f3f3fu;
    s.sc_hi = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
    s.mn_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
}

// (v, v) as fp16 pair for an integer 0 <= v < 1024
__device__ __forceinline__ __half2 int_pair(uint32_t v) {
    const __half2 magic = as_h2(0x64006400u | v | (v << 16));  // (1024 + v, 1024 + v)
    return __hsub2(magic, as_h2(0x64006400u));
}

// 8 weights of one K-step as fp16 sc*q, from the two dwords (q0, q1) of the lane's 8-byte piece
template <int NIB>
__device__ __forceinline__ half8 dequant_kstep(uint32_t q0, uint32_t q1, __half2 sc, __half2 c) {
    uint32_t t[4];
    if (NIB == 0) {
        t[0] = (q0 & 0x000f000fu) | 0x64006400u;
        t[1] = ((q0 >> 8) & 0x000f000fu) | 0x64006400u;
        t[2] = (q1 & 0x000f000fu) | 0x64006400u;
        t[3] = ((q1 >> 8) & 0x000f000fu) | 0x64006400u;
    } else {
        t[0] = ((q0 >> 4) & 0x000f000fu) | 0x64006400u;
        t[1] = ((q0 >> 12) & 0x000f000fu) | 0x64006400u;
        t[2] = ((q1 >> 4) & 0x000f000fu) | 0x64006400u;
        t[3] = ((q1 >> 12) & 0x000f000fu) | 0x64006400u;
    }
    uint4 r;
    r.x = as_u32(__hfma2(as_h2(t[0]), sc, c));  // (1024 + q) * sc - 1024 * sc = sc * q, one rounding of an exact value
    r.y = as_u32(__hfma2(as_h2(t[1]), sc, c));
    r.z = as_u32(__hfma2(as_h2(t[2]), sc, c));
    r.w = as_u32(__hfma2(as_h2(t[3]), sc, c));
    return __builtin_bit_cast(half8, r);
}

__global__ __launch_bounds__(256) void k_gemm_q4k_f16(const GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // 2 stages
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int j = lane & 31, kh = lane >> 5;
    const size_t tt = blockIdx.y;
    const size_t wrow0 = (size_t)blockIdx.x * G_WROWS_WG + (size_t)wave * G_WROWS_WAVE;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }

    const uint8_t *wrow[2];
#pragma unroll
    for (int wt = 0; wt < 2; ++wt) {
        size_t r = wrow0 + 32 * wt + j;
        if (r >= p.M) {
            r = p.M - 1;  // harmless re-read; never stored
        }
        wrow[wt] = p.w + r * p.nb * Q4_K_BYTES;
    }

    floatx16 total[4][2];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int wt = 0; wt < 2; ++wt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                total[a][wt][r] = 0.0f;
            }
        }
    }

    if (b0 < b1) {
        // stage the first activation block
        const uint8_t *src = p.packed + (tt * p.nb + b0) * STAGE;
#pragma unroll
        for (int c = 0; c < 17; ++c) {
            const int chunk = tid + 256 * c;
            *(uint4 *)(lds + (size_t)chunk * 16) = *(const uint4 *)(src + (size_t)chunk * 16);
        }
    }
    WeightRegs wnext[2];
    if (b0 < b1) {
#pragma unroll
        for (int wt = 0; wt < 2; ++wt) {
            load_weights(wnext[wt], wrow[wt] + b0 * Q4_K_BYTES, kh);
        }
    }
    __syncthreads();

    for (size_t b = b0; b < b1; ++b) {
        const int cur = (int)((b - b0) & 1);
        const uint8_t *stage = lds + (size_t)cur * STAGE;
        uint8_t *stage_next = lds + (size_t)(cur ^ 1) * STAGE;
        const bool more = b + 1 < b1;
        const uint8_t *src_next = p.packed + (tt * p.nb + b + 1) * STAGE;

        WeightRegs wcur[2];
        Scales sc[2];
#pragma unroll
        for (int wt = 0; wt < 2; ++wt) {
            wcur[wt] = wnext[wt];
            decode_header(wcur[wt].hdr, sc[wt]);
        }
        if (more) {
#pragma unroll
            for (int wt = 0; wt < 2; ++wt) {
                load_weights(wnext[wt], wrow[wt] + (b + 1) * Q4_K_BYTES, kh);
            }
        }

        floatx16 acc[4][2];
        uint4 stg[5];  // activation staging for the next block, moved in 4 groups across the K-steps
#pragma unroll
        for (int ks = 0; ks < 16; ++ks) {
            const int s = ks >> 1, tp = ks & 1, g = s >> 1;
            // next block's activations: global -> registers at K-steps 0,4,8,12; registers -> LDS at 3,7,11,15
            if ((ks & 3) == 0 && more) {
                const int grp = ks >> 2;
#pragma unroll
                for (int c = 0; c < 5; ++c) {
                    const int cc = grp * 5 + c;  // 0..19, chunks 17..19 do not exist
                    if (cc < 17) {
                        stg[c] = *(const uint4 *)(src_next + (size_t)(tid + 256 * cc) * 16);
                    }
                }
            }
            half8 bop[2];
#pragma unroll
            for (int wt = 0; wt < 2; ++wt) {
                const uint32_t scw = s < 4 ? sc[wt].sc_lo : sc[wt].sc_hi;
                const __half2 scp = int_pair((scw >> (8 * (s & 3))) & 0xffu);
                const __half2 cp = __hmul2(scp, as_h2(0xe400e400u));  // -1024 * sc, exact
                const uint32_t q0 = tp ? wcur[wt].q[g].z : wcur[wt].q[g].x;
                const uint32_t q1 = tp ? wcur[wt].q[g].w : wcur[wt].q[g].y;
                bop[wt] = (s & 1) ? dequant_kstep<1>(q0, q1, scp, cp) : dequant_kstep<0>(q0, q1, scp, cp);
            }
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const half8 aop = __builtin_bit_cast(half8, *(const uint4 *)(stage + ((size_t)(ks * 4 + a) * 64 + lane) * 16));
#pragma unroll
                for (int wt = 0; wt < 2; ++wt) {
                    if (ks == 0) {
                        const floatx16 zero = {0};
                        acc[a][wt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop, bop[wt], zero, 0, 0, 0);
                    } else {
                        acc[a][wt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop, bop[wt], acc[a][wt], 0, 0, 0);
                    }
                }
            }
            if ((ks & 3) == 3 && more) {
                const int grp = ks >> 2;
#pragma unroll
                for (int c = 0; c < 5; ++c) {
                    const int cc = grp * 5 + c;
                    if (cc < 17) {
                        *(uint4 *)(stage_next + (size_t)(tid + 256 * cc) * 16) = stg[c];
                    }
                }
            }
        }
        // min term and the per-block scales
        half8 b2[2];
#pragma unroll
        for (int wt = 0; wt < 2; ++wt) {
            uint4 r;
            const uint32_t lo = sc[wt].mn_lo, hi = sc[wt].mn_hi;
            const __half2 k32 = as_h2(0x50005000u);  // (32, 32)
            const __half2 m1024 = as_h2(0x64006400u);
            r.x = as_u32(__hmul2(__hsub2(as_h2(0x64006400u | (lo & 0xffu) | ((lo & 0xff00u) << 8)), m1024), k32));
            r.y = as_u32(__hmul2(__hsub2(as_h2(0x64006400u | ((lo >> 16) & 0xffu) | ((lo >> 8) & 0xff0000u)), m1024), k32));
            r.z = as_u32(__hmul2(__hsub2(as_h2(0x64006400u | (hi & 0xffu) | ((hi & 0xff00u) << 8)), m1024), k32));
            r.w = as_u32(__hmul2(__hsub2(as_h2(0x64006400u | ((hi >> 16) & 0xffu) | ((hi >> 8) & 0xff0000u)), m1024), k32));
            b2[wt] = __builtin_bit_cast(half8, r);
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const half8 a2 = __builtin_bit_cast(half8, *(const uint4 *)(stage + STAGE_A + ((size_t)a * 64 + lane) * 16));
#pragma unroll
            for (int wt = 0; wt < 2; ++wt) {
                const floatx16 zero = {0};
                const floatx16 mq = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b2[wt], zero, 0, 0, 0);
                const float d = sc[wt].d, nd = -sc[wt].dmin;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    total[a][wt][r] = __builtin_fmaf(d, acc[a][wt][r], total[a][wt][r]);
                    total[a][wt][r] = __builtin_fmaf(nd, mq[r], total[a][wt][r]);
                }
            }
        }
        __syncthreads();
    }

    // epilogue
#pragma unroll
    for (int wt = 0; wt < 2; ++wt) {
        const size_t m = wrow0 + 32 * wt + j;
        if (m >= p.M) {
            continue;
        }
        float bias = 0.0f;
        if (p.splits == 1 && p.bias != nullptr && !p.out_is_f16) {
            bias = ((const float *)p.bias)[m];
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t n = tt * G_TOK + 32 * a + 8 * (r >> 2) + 4 * kh + (r & 3);
                if (n >= p.N) {
                    continue;
                }
                const float v = total[a][wt][r];
                if (p.splits > 1) {
                    ((float *)p.out)[((size_t)split * p.N + n) * p.M + m] = v;
                } else if (!p.out_is_f16) {
                    ((float *)p.out)[n * p.M + m] = v + bias;
                } else {
                    uint16_t h = f2h(v);
                    if (p.bias != nullptr) {
                        const float bv =
                            p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[m]) : ((const float *)p.bias)[m];
                        h = f2h(h2f(h) + bv);
                    }
                    ((uint16_t *)p.out)[n * p.M + m] = h;
                }
            }
        }
    }
}

// sums the K-split partials in split order, then bias / output cast like the single-pass epilogue
__global__ __launch_bounds__(256) void k_gemm_reduce(const float *__restrict__ partial, int splits, size_t N, size_t M,
                                                     const void *bias, int bias_is_f16, void *out, int out_is_f16) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N * M) {
        return;
    }
    float v = 0.0f;
    for (int s = 0; s < splits; ++s) {
        v += partial[(size_t)s * N * M + idx];
    }
    const size_t m = idx % M;
    if (!out_is_f16) {
        if (bias != nullptr) {
            v += ((const float *)bias)[m];
        }
        ((float *)out)[idx] = v;
    } else {
        uint16_t h = f2h(v);
        if (bias != nullptr) {
            const float bv = bias_is_f16 ? h2f(((const uint16_t *)bias)[m]) : ((const float *)bias)[m];
            h = f2h(h2f(h) + bv);
        }
        ((uint16_t *)out)[idx] = h;
    }
}

bool gemm_f16_supported(int kind, size_t N, size_t K, size_t M) {
    if (getenv("MARMOT_HIP_NO_GEMM") != nullptr) {
        return false;
    }
    return kind == MARMOT_HIP_KIND_Q4_K && N > 8 && K % QK_K == 0 && M >= 1;
}

int launch_gemm_f16(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K, size_t M,
                    const void *d_bias, int bias_dtype, void *d_out, int out_dtype) {
    if (!gemm_f16_supported(kind, N, K, M)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "prefill GEMM: unsupported kind or shape");
    }
    if ((((uintptr_t)d_x) & 15) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "prefill GEMM: activations must be 16-byte aligned");
    }
    const size_t nb = K / QK_K;
    const size_t tiles_n = (N + G_TOK - 1) / G_TOK;
    const size_t tiles_m = (M + G_WROWS_WG - 1) / G_WROWS_WG;
    const size_t tiles = tiles_n * tiles_m;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t splits = 1;
    if (tiles < cus) {
        splits = cus / tiles;
        if (splits > nb) {
            splits = nb;
        }
        if (splits < 1) {
            splits = 1;
        }
    }
    if (const char *e = getenv("MH_GEMM_SPLITS")) {
        splits = (size_t)atoi(e);
        if (splits < 1) {
            splits = 1;
        }
        if (splits > nb) {
            splits = nb;
        }
    }
    const size_t blocks_per_split = (nb + splits - 1) / splits;
    splits = (nb + blocks_per_split - 1) / blocks_per_split;

    const size_t packed_bytes = tiles_n * nb * STAGE;
    const size_t partial_bytes = splits > 1 ? splits * N * M * sizeof(float) : 0;
    void *ws = nullptr;
    int st = workspace_reserve(dev, ((packed_bytes + 255) & ~(size_t)255) + partial_bytes, &ws);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    uint8_t *packed = (uint8_t *)ws;
    float *partial = (float *)((uint8_t *)ws + ((packed_bytes + 255) & ~(size_t)255));

    {
        const size_t total = tiles_n * nb * (STAGE_A / 16);
        hipLaunchKernelGGL(k_gemm_pack_x, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dev->stream,
                           (const uint16_t *)d_x, N, K, nb, packed);
        const size_t total_s = tiles_n * nb * 4 * 32 * 8;
        hipLaunchKernelGGL(k_gemm_pack_s, dim3((unsigned)((total_s + 255) / 256)), dim3(256), 0, dev->stream,
                           (const uint16_t *)d_x, N, K, nb, packed);
        MH_HIP(hipGetLastError());
    }

    static bool attr_set = false;
    if (!attr_set) {
        MH_HIP(hipFuncSetAttribute((const void *)k_gemm_q4k_f16, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * STAGE));
        attr_set = true;
    }
    GemmParams p;
    p.w = (const uint8_t *)d_w;
    p.packed = packed;
    p.out = splits > 1 ? (void *)partial : d_out;
    p.bias = d_bias;
    p.bias_is_f16 = bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.N = N;
    p.M = M;
    p.nb = nb;
    p.splits = (int)splits;
    p.blocks_per_split = (int)blocks_per_split;
    hipLaunchKernelGGL(k_gemm_q4k_f16, dim3((unsigned)tiles_m, (unsigned)tiles_n, (unsigned)splits), dim3(256),
                       2 * STAGE, dev->stream, p);
    MH_HIP(hipGetLastError());
    if (splits > 1) {
        const size_t total = N * M;
        hipLaunchKernelGGL(k_gemm_reduce, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dev->stream, partial,
                           (int)splits, N, M, d_bias, p.bias_is_f16, d_out, p.out_is_f16);
        MH_HIP(hipGetLastError());
    }
    set_route("gemm_q4_k_f16_mfma");
    return MARMOT_HIP_SUCCESS;
}

} // namespace mh

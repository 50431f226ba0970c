// Prefill GEMM for fp16 activations and EVERY weight format but Q4_K (which has the kernels of mh_gemm.hip), on
// v_mfma_f32_32x32x16_f16 with fp32 accumulation.
//
// Arithmetic. The reference's direct fp16 dots (cpu_vec_dot_*_f16, vec_dot_impl.h:240-450 for the 32-value formats,
// :866-1128 for the K-quants) decode a weight to fp32 and add w * (float)x in fp32, element by element. Here a weight is
// decoded by the same function as in the fp16 matvec (direct_f16_weight<KIND>, mh_dequant.h: the reference's own index
// patterns, which for Q2_K / Q3_K / Q5_K / Q6_K differ from its dequantizers), then written as the sum of two fp16
// numbers, w = hi + lo with |w - hi - lo| <= 2^-22 |w|; hi * x and lo * x are exact in fp32, so the result differs from
// exact arithmetic by 2^-22 per weight and by the fp32 accumulation, less than the reference's own sequential sum.
// Weights must be below the fp16 maximum in magnitude (65504; any trained model's are below 100).
//
// Tiling. A workgroup of four wavefronts owns 128 weight rows x 64 tokens and walks K in rounds of 32 values (one block
// of the 32-value formats, an eighth of a K-quant block). Per round every thread decodes 16 weights of one row (the
// same 16-value half of the round for all rows; for Q8_0, Q4_0 and Q6_K the bytes are requested a round earlier),
// splits them and stores them into one of two LDS stages in MFMA operand order; wavefront c then multiplies its 32 rows with the 64 tokens: two K-steps x two parts x two token tiles = eight
// matrix instructions, activations straight from memory (16 bytes per lane, K-step and token tile). One barrier per
// round. K is split across workgroups when the tiles do not fill the chip; the partial sums meet in k_gemm_reduce.
#include "mh_common.h"
#include "mh_dequant.h"

namespace mh {

typedef _Float16 fa_half8 __attribute__((ext_vector_type(8)));
typedef float fa_floatx16 __attribute__((ext_vector_type(16)));

constexpr int FA_TOK = 64;
constexpr int FA_WROWS = 128;
constexpr int FA_THREADS = 256;
constexpr int FA_ROUND = 32;                          // values of K per round
constexpr int FA_STAGE = 2 * 2 * 4 * 2 * 32 * 16;     // K-step x part x wavefront x k half x row x 16 bytes = 16,384
constexpr int FA_MIN_TOKENS = 9;

struct GemmAnyParams {
    const uint8_t *w;
    const uint16_t *x;   // fp16 activations [N, K]
    void *out;           // [N, M] of the output type, or fp32 partials [splits, N, M]
    const void *bias;
    int bias_is_f16;
    int out_is_f16;
    size_t N, K, M;
    size_t row_bytes;
    int splits;
    int rounds_per_split;
};

// The 16 weights a thread decodes per round, in two steps so that the bytes can be requested a round before they are
// needed: fetch() issues the loads, decode() turns them into the fp32 weights of direct_f16_weight<KIND> (same
// expressions, same bits). Formats without a form of their own keep the pointer and load inside decode().
template <int KIND>
struct AnyRaw {
    const uint8_t *blk;
    int v0;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        blk = b;
        v0 = v;
    }
    __device__ __forceinline__ void decode(float (&w)[16]) const {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            w[i] = direct_f16_weight<KIND>(blk, v0 + i);
        }
    }
};
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q8_0> {
    uint4 q;
    uint16_t s;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        __builtin_memcpy(&s, b, 2);
        __builtin_memcpy(&q, b + 2 + v, 16);
    }
    __device__ __forceinline__ void decode(float (&w)[16]) const {
        const float d = h2f(s);
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            w[i] = (float)(int8_t)(qw[i >> 2] >> (8 * (i & 3))) * d;  // dequant_value_q8_0
        }
    }
};
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q4_0> {
    uint4 q;
    uint16_t s;
    int high;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        __builtin_memcpy(&s, b, 2);
        __builtin_memcpy(&q, b + 2, 16);
        high = v >= 16;
    }
    __device__ __forceinline__ void decode(float (&w)[16]) const {
        const float d = h2f(s);
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t byte = (qw[i >> 2] >> (8 * (i & 3))) & 0xffu;
            const int nib = (int)(high ? byte >> 4 : byte & 0xfu);
            w[i] = (float)(nib - 8) * d;  // dequant_value_q4_0
        }
    }
};
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q6_K> {
    uint2 ql;
    uint32_t qh;
    int8_t sc;
    uint16_t d;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {  // v: a multiple of 16
        __builtin_memcpy(&ql, b + (v >> 1), 8);
        __builtin_memcpy(&qh, b + 128 + (v >> 2), 4);
        sc = (int8_t)b[192 + (v >> 7)];
        __builtin_memcpy(&d, b + 208, 2);
    }
    __device__ __forceinline__ void decode(float (&w)[16]) const {  // direct_f16_weight_q6_k for v .. v + 15
        const float scale = h2f(d) * (float)sc;
        const uint32_t lw[2] = {ql.x, ql.y};
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t byte = (lw[i >> 3] >> (8 * ((i >> 1) & 3))) & 0xffu;
            const uint32_t nib = (i & 1) ? byte >> 4 : byte & 0xfu;
            const uint32_t hi2 = (qh >> (8 * (i >> 2) + 2 * (i & 3))) & 3u;
            const int qv = (int)(int8_t)(nib | (hi2 << 4)) - 32;
            w[i] = scale * (float)qv;
        }
    }
};

template <int KIND>
__global__ __launch_bounds__(FA_THREADS) void k_gemm_any_f16(const GemmAnyParams p) {
    using KT = KindTraits<KIND>;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * FA_STAGE];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, kh = lane >> 5;
    const size_t row0 = (size_t)blockIdx.x * FA_WROWS;
    const size_t tok0 = (size_t)blockIdx.y * FA_TOK;
    const int split = blockIdx.z;
    const size_t rounds = p.K / FA_ROUND;
    const size_t r0 = (size_t)split * p.rounds_per_split;
    size_t r1 = r0 + p.rounds_per_split;
    if (r1 > rounds) {
        r1 = rounds;
    }

    // decode role: row tid / 2 of the tile, values 16 (tid % 2) .. + 15 of the round = K-step tid % 2
    const int drow = tid >> 1, dks = tid & 1;
    size_t wr = row0 + (size_t)drow;
    wr = wr < p.M ? wr : p.M - 1;  // rows beyond M re-read the last row (never stored)
    const uint8_t *const wrow = p.w + wr * p.row_bytes;
    // LDS slot of (K-step ks, part, wavefront c, k half, row j): 16 bytes
    auto slot = [](int ks, int part, int c, int half, int row) -> uint32_t {
        return (uint32_t)(((((ks * 2 + part) * 4 + c) * 2 + half) * 32 + row) * 16);
    };
    auto fetch = [&](size_t round, AnyRaw<KIND> &raw) {
        const size_t k0 = round * FA_ROUND + (size_t)(16 * dks);
        const size_t b = k0 / KT::BV;
        raw.fetch(wrow + b * KT::BB, (int)(k0 - b * KT::BV));
    };
    auto decode = [&](const AnyRaw<KIND> &raw, int stage) {
        float w[16];
        raw.decode(w);
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint16_t h[2], l[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                h[e] = f2h(w[2 * i + e]);
                l[e] = f2h(w[2 * i + e] - h2f(h[e]));
            }
            hi[i] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
            lo[i] = (uint32_t)l[0] | ((uint32_t)l[1] << 16);
        }
        uint8_t *st = lds + (size_t)stage * FA_STAGE;
        const int c = drow >> 5, row = drow & 31;
        *(uint4 *)(st + slot(dks, 0, c, 0, row)) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        *(uint4 *)(st + slot(dks, 0, c, 1, row)) = make_uint4(hi[4], hi[5], hi[6], hi[7]);
        *(uint4 *)(st + slot(dks, 1, c, 0, row)) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        *(uint4 *)(st + slot(dks, 1, c, 1, row)) = make_uint4(lo[4], lo[5], lo[6], lo[7]);
    };

    // activations: token tile a, lane (j, kh) -> token 32 a + j (tokens beyond N re-read the last one), 8 values
    const uint16_t *xrow[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        size_t t = tok0 + (size_t)(32 * a + j);
        t = t < p.N ? t : p.N - 1;
        xrow[a] = p.x + t * p.K + (size_t)(8 * kh);
    }

    fa_floatx16 acc[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            acc[a][r] = 0.0f;
        }
    }

    // rounds in flight: the weights of round + 2 and the activations of round + 1 are requested while round is
    // multiplied and round + 1 is decoded
    auto load_x = [&](size_t round, uint4 (&xa)[2][2]) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                xa[ks][a] = *(const uint4 *)(xrow[a] + round * FA_ROUND + (size_t)(16 * ks));
            }
        }
    };
    AnyRaw<KIND> raw;
    uint4 xa[2][2];  // [K-step][token tile]
    if (r0 < r1) {
        fetch(r0, raw);
        load_x(r0, xa);
        decode(raw, 0);
        if (r0 + 1 < r1) {
            fetch(r0 + 1, raw);
        }
    }
    __syncthreads();
    for (size_t round = r0; round < r1; ++round) {
        const int stage = (int)((round - r0) & 1);
        AnyRaw<KIND> raw_next = raw;
        uint4 xa_next[2][2];
        if (round + 2 < r1) {
            fetch(round + 2, raw_next);
        }
        if (round + 1 < r1) {
            load_x(round + 1, xa_next);
            decode(raw, stage ^ 1);  // the other stage: the barrier that closed the previous round released it
        }
        const uint8_t *st = lds + (size_t)stage * FA_STAGE;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int part = 0; part < 2; ++part) {
                const fa_half8 wb = __builtin_bit_cast(fa_half8, *(const uint4 *)(st + slot(ks, part, wave, kh, j)));
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(fa_half8, xa[ks][a]), wb, acc[a],
                                                                    0, 0, 0);
                }
            }
        }
        raw = raw_next;
        if (round + 1 < r1) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    xa[ks][a] = xa_next[ks][a];
                }
            }
        }
        __syncthreads();
    }

    // lane (j, kh) of wavefront c holds weight row 32 c + j for tokens 32 a + 8 (r / 4) + 4 kh + r % 4
    const size_t m = row0 + (size_t)(32 * wave + j);
    if (m >= p.M) {
        return;
    }
    const bool partials = p.splits > 1;
    float bias = 0.0f;
    const bool has_bias = !partials && p.bias != nullptr;
    if (has_bias) {
        bias = p.bias_is_f16 ? h2f(((const uint16_t *)p.bias)[m]) : ((const float *)p.bias)[m];
    }
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const size_t n = tok0 + (size_t)(32 * a + 8 * (r >> 2) + 4 * kh + (r & 3));
            if (n >= p.N) {
                continue;
            }
            const float v = acc[a][r];
            if (partials) {
                ((float *)p.out)[((size_t)split * p.N + n) * p.M + m] = v;
            } else if (!p.out_is_f16) {
                ((float *)p.out)[n * p.M + m] = has_bias ? v + bias : v;
            } else {
                uint16_t h = f2h(v);  // round to the output type first, then add the bias in it
                if (has_bias) {
                    h = f2h(h2f(h) + bias);
                }
                ((uint16_t *)p.out)[n * p.M + m] = h;
            }
        }
    }
}

bool gemm_f16_any_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M) {
    if (dev->knobs.no_gemm || kind == MARMOT_HIP_KIND_Q4_K || kind == MARMOT_HIP_KIND_Q8_K) {
        return false;
    }
    return N >= FA_MIN_TOKENS && K % FA_ROUND == 0 && K % block_values(kind) == 0 && M >= 1;
}

template <int KIND>
static int launch_any_kind(marmot_hip_device *dev, GemmAnyParams p, const dim3 grid) {
    hipLaunchKernelGGL((k_gemm_any_f16<KIND>), grid, dim3(FA_THREADS), 0, dev->stream, p);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int launch_gemm_f16_any(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K,
                        size_t M, const void *d_bias, int bias_dtype, void *d_out, int out_dtype) {
    if (!gemm_f16_any_supported(dev, kind, N, K, M)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "fp16 GEMM: unsupported kind or shape");
    }
    if ((((uintptr_t)d_x) & 15) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "fp16 GEMM: activations must be 16-byte aligned");
    }
    const size_t rounds = K / FA_ROUND;
    const size_t tiles_n = (N + FA_TOK - 1) / FA_TOK, tiles_m = (M + FA_WROWS - 1) / FA_WROWS;
    const size_t tiles = tiles_n * tiles_m;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    // two workgroups per compute unit overlap each other's barriers; fewer tiles than that: split K (at least 16 rounds
    // per workgroup)
    size_t splits = 1;
    if (tiles < 2 * cus) {
        splits = (2 * cus) / tiles;
        const size_t max_splits = rounds / 16 > 0 ? rounds / 16 : 1;
        splits = splits > max_splits ? max_splits : splits;
        splits = splits > 16 ? 16 : splits;
    }
    const size_t rps = (rounds + splits - 1) / splits;
    splits = (rounds + rps - 1) / rps;
    float *partial = nullptr;
    if (splits > 1) {
        void *ws = nullptr;
        MH_TRY(workspace_reserve(dev, splits * N * M * sizeof(float), &ws));
        partial = (float *)ws;
    }
    GemmAnyParams p;
    p.w = (const uint8_t *)d_w;
    p.x = (const uint16_t *)d_x;
    p.out = splits > 1 ? (void *)partial : d_out;
    p.bias = d_bias;
    p.bias_is_f16 = bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.N = N;
    p.K = K;
    p.M = M;
    p.row_bytes = (K / block_values(kind)) * block_bytes(kind);
    p.splits = (int)splits;
    p.rounds_per_split = (int)rps;
    const dim3 grid((unsigned)tiles_m, (unsigned)tiles_n, (unsigned)splits);
    int st;
    switch (kind) {
    case MARMOT_HIP_KIND_Q8_0:
        set_route("gemm_q8_0_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q8_0>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q4_0:
        set_route("gemm_q4_0_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q4_0>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q8_1:
        set_route("gemm_q8_1_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q8_1>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q4_1:
        set_route("gemm_q4_1_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q4_1>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q5_0:
        set_route("gemm_q5_0_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q5_0>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q5_1:
        set_route("gemm_q5_1_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q5_1>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q2_K:
        set_route("gemm_q2_k_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q2_K>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q3_K:
        set_route("gemm_q3_k_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q3_K>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q5_K:
        set_route("gemm_q5_k_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q5_K>(dev, p, grid);
        break;
    case MARMOT_HIP_KIND_Q6_K:
        set_route("gemm_q6_k_f16_mfma");
        st = launch_any_kind<MARMOT_HIP_KIND_Q6_K>(dev, p, grid);
        break;
    default:
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "fp16 GEMM: unsupported kind");
    }
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    if (splits > 1) {
        MH_TRY(launch_splitk_reduce(dev, partial, (int)splits, N, M, d_bias, bias_dtype, d_out, out_dtype));
    }
    return MARMOT_HIP_SUCCESS;
}

} // namespace mh

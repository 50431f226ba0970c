// Prefill with fp32 activations: Q4_K weights x Q8_K activations as a tiled GEMM on the int8 matrix cores.
//
// Same integer arithmetic as cpu_vec_dot_q4_k_q8_k (src/backends/cpu/ops/matmul/quantized/vec_dot_impl.h:689-732):
// per 256-value block
//     isum = sum_j sc_j * (q_j . a_j),   msum = sum_j mn_j * (sum of a over sub-block j),
//     y += a.d * (w.d * isum - w.dmin * msum)
// A workgroup computes 128 weight rows x 64 tokens over a range of blocks. The 6-bit scale is folded into the
// matrix-core operand, so that the eight sub-block products of a block chain through the accumulators and the fp32
// work per output happens once per block instead of once per sub-block: sc = 8 * (sc >> 3) + (sc & 7), and both
// q * (sc & 7) and q * (sc >> 3) are at most 15 * 7 = 105, i.e. int8. Per sub-block and 32 x 32 output tile that is
//     X += A . (q * (sc & 7)),   Y += A . (q * (sc >> 3)),   T += A . mn        (v_mfma_i32_32x32x32_i8, exact)
// and per block isum = X + 8 Y, msum = T. All integer results are exact (|isum| < 2^25); only the fp32 accumulation
// over blocks is ordered differently from the CPU.
//
// Eight wavefronts, two per SIMD: wavefront (rg, kg) owns weight rows 32 rg .. 32 rg + 31 of the tile and all 64 tokens
// (two 32 x 32 tiles) and works on every second block of the workgroup's K range (K group kg), so a round consumes two
// consecutive blocks; the two K groups' sums meet in LDS at the end. There are no loader wavefronts: at the start of a
// round every wavefront issues its quarter of its K group's next block (int8 activation tile 64 tokens x 256 bytes
// with the chunks XOR-swizzled by token, raw weight blocks 128 rows x 144 bytes, 64 activation scales) as
// direct-to-LDS loads into the other round buffer, then computes, then waits for its own loads; one barrier per round.
// On this chip a wavefront's instruction stream costs about 5.6 clocks per vector instruction and 16 per
// matrix-core or LDS instruction whatever else the SIMD does, so the kernel is bound by its instruction count
// (per block and wavefront: 378 vector, 48 matrix-core, 29 LDS); the operand preparation of sub-block s + 1 is placed
// between the matrix-core instructions of sub-block s so that the matrix cores never wait for it.
#include "mh_rows.h"

namespace mh {

typedef int i8_intx4 __attribute__((ext_vector_type(4)));
typedef int i8_intx16 __attribute__((ext_vector_type(16)));
typedef unsigned short i8_u16x2 __attribute__((ext_vector_type(2)));

struct GemmI8Params {
    const uint8_t *w;   // Q4_K blocks, M rows of nb blocks
    const int8_t *qs;   // quantized activations, rows of kp bytes
    const float *ad;    // activation block scales [N][nb]
    const int16_t *sums = nullptr;  // Q8_0 activations: sum of a block's codes [N][8 nb] (formats with a minimum)
    size_t kp;
    size_t N, M, nb;
    void *out;          // [N][M] of the output type, or fp32 partials [splits][N][M] when splits > 1
    int splits;
    int blocks_per_split;
    const void *bias;
    int bias_is_f16;
    int bias_first;     // fp16 output: f16(dot + bias) instead of f16(f16(dot) + bias)
    int out_is_f16;
};

constexpr int I8_TOK = 64;
constexpr int I8_WROWS = 128;
constexpr int I8_WAVES = 8;
constexpr int I8_THREADS = I8_WAVES * 64;
constexpr int I8_STAGE_A = I8_TOK * QK_K;             // 16,384
constexpr int I8_STAGE_W = I8_WROWS * Q4_K_BYTES;     // 18,432
constexpr int I8_STAGE_D = I8_TOK * 4;                // 256
constexpr int I8_STAGE = I8_STAGE_A + I8_STAGE_W + I8_STAGE_D;   // one block of the tile: 35,072 bytes
constexpr int I8_ROUND = 2 * I8_STAGE;                // a round is two consecutive blocks, one per K group
constexpr int I8_LDS_BYTES = 2 * I8_ROUND;            // the round in work and the round in flight: 140,288
constexpr int I8_OUT_PITCH = I8_WROWS + 4;            // floats per token of the output tile in LDS
constexpr int I8_OUT_TILE_BYTES = I8_TOK * I8_OUT_PITCH * 4;   // the output tile, which reuses the stages
static_assert(I8_OUT_TILE_BYTES <= I8_LDS_BYTES, "the output tile reuses the stages");
static_assert(I8_STAGE % 16 == 0, "stages keep 16-byte alignment");

__device__ __forceinline__ void i8_lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One direct-to-LDS load of 64 x 4 bytes (see dma16_to_lds): lane l's dword lands at LDS address M0 + 4 l.
__device__ __forceinline__ void dma4_to_lds(const uint8_t *base, uint32_t voff) {
    asm volatile("global_load_lds_dword %0, %1" : : "v"(voff), "s"(base) : "memory");
}

// the four bytes of `nib` (each 0..15) times the scalar in both 16-bit halves of `s16` (0..7): no byte overflows
__device__ __forceinline__ int i8_scale_bytes(uint32_t nib, uint32_t s16) {
    const i8_u16x2 r = __builtin_bit_cast(i8_u16x2, nib) * __builtin_bit_cast(i8_u16x2, s16);
    return __builtin_bit_cast(int, r);
}

// The two K groups of a workgroup meet in LDS as one [token][weight row] tile, then every thread stores 16 bytes per
// step. Lane (j, kh) of wavefront (rg, kg) holds weight row 32 rg + j for tokens 32 a + 8 (r / 4) + 4 kh + r % 4. Every
// wavefront of the workgroup calls this after its last read of the stages (the function contains barriers).
// NA: token tiles of 32 per workgroup (2, or 1 in the kernels that have a form for at most 32 activation rows).
template <int NA>
__device__ __forceinline__ void i8_merge_and_store(const GemmI8Params &p, uint8_t *lds, const float (&total)[NA][16],
                                                   int tid, int rg, int kg, int j, int kh, size_t tt, size_t row0,
                                                   int split) {
    float *tile = (float *)lds;
    if (kg == 1) {
#pragma unroll
        for (int a = 0; a < NA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                tile[(32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * I8_OUT_PITCH + 32 * rg + j] = total[a][r];
            }
        }
    }
    i8_lds_barrier();
    if (kg == 0) {
#pragma unroll
        for (int a = 0; a < NA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float *e = tile + (32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * I8_OUT_PITCH + 32 * rg + j;
                *e = total[a][r] + *e;
            }
        }
    }
    i8_lds_barrier();

    const bool partials = p.splits > 1;
    const bool has_bias = !partials && p.bias != nullptr;
    const bool out_f16 = !partials && p.out_is_f16;
    float *const out32 = (float *)p.out + (partials ? (size_t)split * p.N * p.M : 0);
    const bool vec = (p.M & 3) == 0 && (((uintptr_t)p.out) & 15) == 0;
    for (int idx = tid; idx < 32 * NA * I8_WROWS / 4; idx += I8_THREADS) {
        const int t = idx >> 5, q4 = idx & 31;  // rows 4 q4 .. 4 q4 + 3 of token t
        const size_t n = tt * (32 * NA) + (size_t)t;
        const size_t m4 = row0 + 4 * (size_t)q4;
        if (n >= p.N || m4 >= p.M) {
            continue;
        }
        const float4 v = *(const float4 *)(tile + t * I8_OUT_PITCH + 4 * q4);
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
                if (p.bias_first) {
                    h[e] = f2h(has_bias ? e4[e] + bias4[e] : e4[e]);
                } else {
                    h[e] = f2h(e4[e]);  // round to the output type first, then add the bias in it
                    if (has_bias) {
                        h[e] = f2h(h2f(h[e]) + bias4[e]);
                    }
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

__global__ __launch_bounds__(I8_THREADS) void k_gemm_q4k_q8k_tile(const GemmI8Params p) {
    warm_kernel_arguments<sizeof(GemmI8Params)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = wave & 3;   // weight rows 32 rg .. + 31 of the tile; also this wavefront's share of the loads
    const int kg = wave >> 2;  // K group: blocks b0 + kg, b0 + kg + 2, ...
    const size_t tt = blockIdx.y;
    const size_t row0 = (size_t)blockIdx.x * I8_WROWS;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nblk = (int)(b1 - b0);
    const int rounds = (nblk + 1) / 2;
    const int j = lane & 31, kh = lane >> 5;

    float total[2][16];  // [token tile][register]
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            total[a][r] = 0.0f;
        }
    }

    // ---- loads: the four wavefronts of a K group bring that group's block of every round, a quarter each
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    const uint32_t last_tok = (uint32_t)(p.N - 1 - tt * I8_TOK);  // token rows beyond it re-read it
    const uint8_t *tile_q = (const uint8_t *)p.qs + tt * I8_TOK * p.kp;
    // Activation tile: token t owns 256 bytes of the stage as 16 chunks of 16 bytes, chunk c stored in slot
    // c ^ (t % 16) (the MFMA operand reads of 32 tokens x one chunk then spread over the bank groups). One
    // instruction moves four token rows; wavefront rg brings tokens 16 rg .. 16 rg + 15.
    uint32_t a_voff[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t t = (uint32_t)(16 * rg + 4 * c + (lane >> 4));
        const uint32_t slot = (uint32_t)(lane & 15);
        const uint32_t trow = t < last_tok ? t : last_tok;
        a_voff[c] = trow * (uint32_t)p.kp + 16u * (slot ^ (t & 15u));
    }
    // Weight blocks: piece q of the stage is 16 bytes q % 9 of tile row q / 9; wavefront rg brings pieces
    // 256 pass + 64 rg + lane. Rows beyond M re-read row M - 1 (never stored).
    const size_t row_bytes = p.nb * Q4_K_BYTES;
    const uint32_t last_wrow = (uint32_t)(p.M - 1 - row0);
    uint32_t w_voff[5];
#pragma unroll
    for (int pass = 0; pass < 5; ++pass) {
        const uint32_t q = (uint32_t)(256 * pass + 64 * rg + lane);
        const uint32_t r = q / 9u, c9 = q - 9u * r;
        const uint32_t rr = r < last_wrow ? r : last_wrow;
        w_voff[pass] = rr * (uint32_t)row_bytes + 16u * c9;
    }
    const uint8_t *wbase = p.w + row0 * row_bytes;
    const bool fifth = rg < 2;    // pieces 1024 .. 1151
    const bool scales = rg == 3;  // the 64 activation scales of the block
    uint32_t d_voff;
    {
        const uint32_t t = (uint32_t)lane;
        const uint32_t trow = t < last_tok ? t : last_tok;
        d_voff = (uint32_t)((trow * p.nb) * 4);
    }
    const uint8_t *tile_d = (const uint8_t *)(p.ad + tt * I8_TOK * p.nb);
    // block b0 + 2 round + kg into the K group's half of round buffer round % 2 (nothing when the block does not exist)
    auto issue = [&](int round) {
        const int bi = 2 * round + kg;
        if (bi >= nblk) {
            return;
        }
        const size_t b = b0 + (size_t)bi;
        const uint32_t s0 = lds_base + (uint32_t)((round & 1) * I8_ROUND + kg * I8_STAGE);
        const uint8_t *qb = tile_q + b * QK_K;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            dma_set_lds_base(s0 + (uint32_t)(4096 * rg + 1024 * c));
            dma16_to_lds<0>(qb, a_voff[c]);
        }
        const uint8_t *wb = wbase + b * Q4_K_BYTES;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            dma_set_lds_base(s0 + (uint32_t)(I8_STAGE_A + (256 * pass + 64 * rg) * 16));
            dma16_to_lds<0>(wb, w_voff[pass]);
        }
        if (fifth) {
            dma_set_lds_base(s0 + (uint32_t)(I8_STAGE_A + (1024 + 64 * rg) * 16));
            dma16_to_lds<0>(wb, w_voff[4]);
        }
        if (scales) {
            dma_set_lds_base(s0 + (uint32_t)(I8_STAGE_A + I8_STAGE_W));
            dma4_to_lds(tile_d + b * 4, d_voff);
        }
    };

    // ---- compute: this wavefront's weight row 32 rg + j of its K group's block, all 64 tokens
    const uint32_t w_off = (uint32_t)(kg * I8_STAGE + I8_STAGE_A + (32 * rg + j) * Q4_K_BYTES);
    // A operand of sub-block sb, token tile a, lane (j, kh): token 32 a + j, chunk 2 sb + kh at slot chunk ^ (j % 16)
    uint32_t a_off[8];
#pragma unroll
    for (int sb = 0; sb < 8; ++sb) {
        a_off[sb] = (uint32_t)(kg * I8_STAGE + j * QK_K + 16 * ((2 * sb + kh) ^ (j & 15)));
    }
    const uint32_t d_off = (uint32_t)(kg * I8_STAGE + I8_STAGE_A + I8_STAGE_W + 16 * kh);

    issue(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    i8_lds_barrier();
    for (int round = 0; round < rounds; ++round) {
        // the next round's blocks land in the other buffer while this round computes: the barrier that closed the
        // previous round guarantees that nobody reads that buffer any more
        if (round + 1 < rounds) {
            issue(round + 1);
        }
        if (2 * round + kg < nblk) {
            const uint8_t *stage = lds + (size_t)(round & 1) * I8_ROUND;
            const uint8_t *wr = stage + w_off;
            const uint4 hdr = *(const uint4 *)wr;
            uint4 wq[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                wq[g] = *(const uint4 *)(wr + 16 + 32 * g + 16 * kh);
            }
            auto read_a = [&](int sb, i8_intx4(&aop)[2]) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const uint4 av = *(const uint4 *)(stage + a_off[sb] + a * (32 * QK_K));
                    aop[a] = i8_intx4{(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                }
            };
            i8_intx4 aop[3][2];  // A operands of the sub-block in work and of the next two
            read_a(0, aop[0]);
            read_a(1, aop[1]);
            // 6-bit scales and mins as bytes (get_scale_min_k4, kquant_common.h:29-37)
            float d = h2f((uint16_t)(hdr.x & 0xffffu));
            float dmin = h2f((uint16_t)(hdr.x >> 16));
            asm volatile("" : "+v"(d), "+v"(dmin));  // plain fp32 values: no mixed-precision multiply-adds below
            const uint32_t sc_lo = hdr.y & 0x3f3f3f3fu;
            const uint32_t mn_lo = hdr.z & 0x3f3f3f3fu;
            const uint32_t sc_hi = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
            const uint32_t mn_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
            const uint32_t s3_lo[2] = {sc_lo & 0x07070707u, sc_hi & 0x07070707u};                // sc & 7
            const uint32_t s3_hi[2] = {(sc_lo >> 3) & 0x07070707u, (sc_hi >> 3) & 0x07070707u};  // sc >> 3

            i8_intx16 X[2], Y[2], T[2];
            float4 da4[2][4];
            // B operands of sub-block sb: the nibbles times (sc & 7), times (sc >> 3), and the min in every byte. Built
            // in six pieces, one behind each matrix-core instruction of the previous sub-block.
            uint32_t nib[4], lo16 = 0, hi16 = 0;
            i8_intx4 bx[2], by[2];
            int bt[2];
            auto prep = [&](int sb, int piece) {
                const int n = sb & 1;
                const uint4 src = wq[sb >> 1];
                switch (piece) {
                case 0:
                    if (sb & 1) {
                        nib[0] = (src.x >> 4) & 0x0f0f0f0fu;
                        nib[1] = (src.y >> 4) & 0x0f0f0f0fu;
                    } else {
                        nib[0] = src.x & 0x0f0f0f0fu;
                        nib[1] = src.y & 0x0f0f0f0fu;
                    }
                    break;
                case 1:
                    if (sb & 1) {
                        nib[2] = (src.z >> 4) & 0x0f0f0f0fu;
                        nib[3] = (src.w >> 4) & 0x0f0f0f0fu;
                    } else {
                        nib[2] = src.z & 0x0f0f0f0fu;
                        nib[3] = src.w & 0x0f0f0f0fu;
                    }
                    break;
                case 2: {
                    // byte sb % 4 of the packed 3-bit halves in both 16-bit lanes; of the packed mins in all four bytes
                    const uint32_t sel16 = 0x0c000c00u | (uint32_t)(sb & 3) | ((uint32_t)(sb & 3) << 16);
                    lo16 = __builtin_amdgcn_perm(0u, s3_lo[sb >> 2], sel16);
                    hi16 = __builtin_amdgcn_perm(0u, s3_hi[sb >> 2], sel16);
                    bt[n] = (int)__builtin_amdgcn_perm(0u, sb < 4 ? mn_lo : mn_hi, 0x01010101u * (sb & 3));
                    break;
                }
                case 3:
                    bx[n][0] = i8_scale_bytes(nib[0], lo16);
                    bx[n][1] = i8_scale_bytes(nib[1], lo16);
                    bx[n][2] = i8_scale_bytes(nib[2], lo16);
                    break;
                case 4:
                    bx[n][3] = i8_scale_bytes(nib[3], lo16);
                    by[n][0] = i8_scale_bytes(nib[0], hi16);
                    by[n][1] = i8_scale_bytes(nib[1], hi16);
                    break;
                default:
                    by[n][2] = i8_scale_bytes(nib[2], hi16);
                    by[n][3] = i8_scale_bytes(nib[3], hi16);
                    break;
                }
            };
#pragma unroll
            for (int piece = 0; piece < 6; ++piece) {
                prep(0, piece);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                const int c = sb & 1;
                if (sb < 6) {
                    read_a(sb + 2, aop[(sb + 2) % 3]);  // lands while the MFMAs of this and the next sub-block run
                }
                if (sb == 6) {
                    // activation scales: registers 4 g .. 4 g + 3 of token tile a are tokens 32 a + 8 g + 4 kh .. + 3
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            da4[a][g] = *(const float4 *)(stage + d_off + 4 * (32 * a + 8 * g));
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                const i8_intx4 btv = {bt[c], bt[c], bt[c], bt[c]};
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const i8_intx4 av = aop[sb % 3][a];
                    const i8_intx16 zero = {0};
                    X[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bx[c], sb == 0 ? zero : X[a], 0, 0, 0);
                    if (sb < 7) {
                        prep(sb + 1, 3 * a);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    Y[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, by[c], sb == 0 ? zero : Y[a], 0, 0, 0);
                    if (sb < 7) {
                        prep(sb + 1, 3 * a + 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    T[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, btv, sb == 0 ? zero : T[a], 0, 0, 0);
                    if (sb < 7) {
                        prep(sb + 1, 3 * a + 2);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // once per block and output: y += a.d * (w.d * isum - w.dmin * msum)
            const float ndmin = -dmin;
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float da[4] = {da4[a][g].x, da4[a][g].y, da4[a][g].z, da4[a][g].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = 4 * g + e;
                        const int isum = X[a][r] + (Y[a][r] << 3);
                        const float v = __builtin_fmaf(ndmin, (float)T[a][r], d * (float)isum);
                        total[a][r] = __builtin_fmaf(da[e], v, total[a][r]);
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's share of the next round has landed
        i8_lds_barrier();
    }

    i8_merge_and_store<2>(p, lds, total, tid, rg, kg, j, kh, tt, row0, split);
}

// ------------------------------------------------------------------ Q5_K x Q8_K
// The Q4_K kernel with the fifth bit (cpu_vec_dot_q5_k_q8_k, vec_dot_impl.h:734-781): q5 = q4 + 16 bit, so
// isum = sum_j sc_j * (q4_j . a_j) + 16 * sum_j sc_j * (bit_j . a_j); the second sum is one more scale plane,
// bit * sc <= 63. Blocks are 176 bytes (11 chunks of 16 per row): two round buffers of 2 x 39,168 bytes.
constexpr int I5_STAGE_W = I8_WROWS * Q5_K_BYTES;                  // 22,528
constexpr int I5_STAGE = I8_STAGE_A + I5_STAGE_W + I8_STAGE_D;     // 39,168
constexpr int I5_ROUND = 2 * I5_STAGE;
constexpr int I5_LDS_BYTES = 2 * I5_ROUND;                         // 156,672 of 163,840
static_assert(I5_STAGE % 16 == 0, "stages keep 16-byte alignment");

__global__ __launch_bounds__(I8_THREADS) void k_gemm_q5k_q8k_tile(const GemmI8Params p) {
    warm_kernel_arguments<sizeof(GemmI8Params)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = wave & 3;   // weight rows 32 rg .. + 31 of the tile; also this wavefront's share of the loads
    const int kg = wave >> 2;  // K group: blocks b0 + kg, b0 + kg + 2, ...
    const size_t tt = blockIdx.y;
    const size_t row0 = (size_t)blockIdx.x * I8_WROWS;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nblk = (int)(b1 - b0);
    const int rounds = (nblk + 1) / 2;
    const int j = lane & 31, kh = lane >> 5;

    float total[2][16];  // [token tile][register]
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            total[a][r] = 0.0f;
        }
    }

    // ---- loads: the four wavefronts of a K group bring that group's block of every round, a quarter each
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    const uint32_t last_tok = (uint32_t)(p.N - 1 - tt * I8_TOK);  // token rows beyond it re-read it
    const uint8_t *tile_q = (const uint8_t *)p.qs + tt * I8_TOK * p.kp;
    // Activation tile: token t owns 256 bytes of the stage as 16 chunks of 16 bytes, chunk c stored in slot
    // c ^ (t % 16) (the MFMA operand reads of 32 tokens x one chunk then spread over the bank groups). One
    // instruction moves four token rows; wavefront rg brings tokens 16 rg .. 16 rg + 15.
    uint32_t a_voff[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t t = (uint32_t)(16 * rg + 4 * c + (lane >> 4));
        const uint32_t slot = (uint32_t)(lane & 15);
        const uint32_t trow = t < last_tok ? t : last_tok;
        a_voff[c] = trow * (uint32_t)p.kp + 16u * (slot ^ (t & 15u));
    }
    // Weight blocks: piece q of the stage is 16 bytes q % 11 of tile row q / 11; wavefront rg brings pieces
    // 256 pass + 64 rg + lane. Rows beyond M re-read row M - 1 (never stored).
    const size_t row_bytes = p.nb * Q5_K_BYTES;
    const uint32_t last_wrow = (uint32_t)(p.M - 1 - row0);
    uint32_t w_voff[6];
#pragma unroll
    for (int pass = 0; pass < 6; ++pass) {
        const uint32_t q = (uint32_t)(256 * pass + 64 * rg + lane);
        const uint32_t r = q / 11u, c11 = q - 11u * r;
        const uint32_t rr = r < last_wrow ? r : last_wrow;
        w_voff[pass] = rr * (uint32_t)row_bytes + 16u * c11;
    }
    const uint8_t *wbase = p.w + row0 * row_bytes;
    const bool sixth = rg < 2;    // pieces 1280 .. 1407
    const bool scales = rg == 3;  // the 64 activation scales of the block
    uint32_t d_voff;
    {
        const uint32_t t = (uint32_t)lane;
        const uint32_t trow = t < last_tok ? t : last_tok;
        d_voff = (uint32_t)((trow * p.nb) * 4);
    }
    const uint8_t *tile_d = (const uint8_t *)(p.ad + tt * I8_TOK * p.nb);
    // block b0 + 2 round + kg into the K group's half of round buffer round % 2 (nothing when the block does not exist)
    auto issue = [&](int round) {
        const int bi = 2 * round + kg;
        if (bi >= nblk) {
            return;
        }
        const size_t b = b0 + (size_t)bi;
        const uint32_t s0 = lds_base + (uint32_t)((round & 1) * I5_ROUND + kg * I5_STAGE);
        const uint8_t *qb = tile_q + b * QK_K;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            dma_set_lds_base(s0 + (uint32_t)(4096 * rg + 1024 * c));
            dma16_to_lds<0>(qb, a_voff[c]);
        }
        const uint8_t *wb = wbase + b * Q5_K_BYTES;
#pragma unroll
        for (int pass = 0; pass < 5; ++pass) {
            dma_set_lds_base(s0 + (uint32_t)(I8_STAGE_A + (256 * pass + 64 * rg) * 16));
            dma16_to_lds<0>(wb, w_voff[pass]);
        }
        if (sixth) {
            dma_set_lds_base(s0 + (uint32_t)(I8_STAGE_A + (1280 + 64 * rg) * 16));
            dma16_to_lds<0>(wb, w_voff[5]);
        }
        if (scales) {
            dma_set_lds_base(s0 + (uint32_t)(I8_STAGE_A + I5_STAGE_W));
            dma4_to_lds(tile_d + b * 4, d_voff);
        }
    };

    // ---- compute: this wavefront's weight row 32 rg + j of its K group's block, all 64 tokens
    const uint32_t w_off = (uint32_t)(kg * I5_STAGE + I8_STAGE_A + (32 * rg + j) * Q5_K_BYTES);
    // A operand of sub-block sb, token tile a, lane (j, kh): token 32 a + j, chunk 2 sb + kh at slot chunk ^ (j % 16)
    uint32_t a_off[8];
#pragma unroll
    for (int sb = 0; sb < 8; ++sb) {
        a_off[sb] = (uint32_t)(kg * I5_STAGE + j * QK_K + 16 * ((2 * sb + kh) ^ (j & 15)));
    }
    const uint32_t d_off = (uint32_t)(kg * I5_STAGE + I8_STAGE_A + I5_STAGE_W + 16 * kh);

    issue(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    i8_lds_barrier();
    for (int round = 0; round < rounds; ++round) {
        // the next round's blocks land in the other buffer while this round computes: the barrier that closed the
        // previous round guarantees that nobody reads that buffer any more
        if (round + 1 < rounds) {
            issue(round + 1);
        }
        if (2 * round + kg < nblk) {
            const uint8_t *stage = lds + (size_t)(round & 1) * I5_ROUND;
            const uint8_t *wr = stage + w_off;
            const uint4 hdr = *(const uint4 *)wr;
            uint4 wq[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                wq[g] = *(const uint4 *)(wr + 48 + 32 * g + 16 * kh);
            }
            // fifth bits of this lane's 16 positions: bit sb of byte l belongs to sub-block sb (q5k_gguf.c:162-198)
            const uint4 wqh = *(const uint4 *)(wr + 16 + 16 * kh);
            auto read_a = [&](int sb, i8_intx4(&aop)[2]) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const uint4 av = *(const uint4 *)(stage + a_off[sb] + a * (32 * QK_K));
                    aop[a] = i8_intx4{(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                }
            };
            i8_intx4 aop[2][2];  // A operands of the sub-block in work and of the next one
            read_a(0, aop[0]);
            // 6-bit scales and mins as bytes (get_scale_min_k4, kquant_common.h:29-37)
            float d = h2f((uint16_t)(hdr.x & 0xffffu));
            float dmin = h2f((uint16_t)(hdr.x >> 16));
            asm volatile("" : "+v"(d), "+v"(dmin));  // plain fp32 values: no mixed-precision multiply-adds below
            const uint32_t sc_lo = hdr.y & 0x3f3f3f3fu;
            const uint32_t mn_lo = hdr.z & 0x3f3f3f3fu;
            const uint32_t sc_hi = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
            const uint32_t mn_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
            const uint32_t s3_lo[2] = {sc_lo & 0x07070707u, sc_hi & 0x07070707u};                // sc & 7
            const uint32_t s3_hi[2] = {(sc_lo >> 3) & 0x07070707u, (sc_hi >> 3) & 0x07070707u};  // sc >> 3

            // Two sweeps over the eight sub-blocks, so that three accumulator chains are never live together with the
            // partial sums of the other two. First the Q4_K part, X += A . (q4 * (sc & 7)), Y += A . (q4 * (sc >> 3)),
            // folded into P = X + 8 Y; then Z += A . (bit * sc) (the fifth bit times the whole 6-bit scale is at most
            // 63) and T += A . mn, which read the activation operands a second time. isum = P + 16 Z, msum = T.
            i8_intx16 X[2], Y[2];
            float4 da4[2][4];
            uint32_t nib[4], lo16 = 0, hi16 = 0;
            i8_intx4 bx[2], by[2];
            auto prep1 = [&](int sb, int piece) {
                const int n = sb & 1;
                const uint4 src = wq[sb >> 1];
                switch (piece) {
                case 0:
                    if (sb & 1) {
                        nib[0] = (src.x >> 4) & 0x0f0f0f0fu;
                        nib[1] = (src.y >> 4) & 0x0f0f0f0fu;
                        nib[2] = (src.z >> 4) & 0x0f0f0f0fu;
                        nib[3] = (src.w >> 4) & 0x0f0f0f0fu;
                    } else {
                        nib[0] = src.x & 0x0f0f0f0fu;
                        nib[1] = src.y & 0x0f0f0f0fu;
                        nib[2] = src.z & 0x0f0f0f0fu;
                        nib[3] = src.w & 0x0f0f0f0fu;
                    }
                    break;
                case 1: {
                    const uint32_t sel16 = 0x0c000c00u | (uint32_t)(sb & 3) | ((uint32_t)(sb & 3) << 16);
                    lo16 = __builtin_amdgcn_perm(0u, s3_lo[sb >> 2], sel16);
                    hi16 = __builtin_amdgcn_perm(0u, s3_hi[sb >> 2], sel16);
                    bx[n][0] = i8_scale_bytes(nib[0], lo16);
                    bx[n][1] = i8_scale_bytes(nib[1], lo16);
                    break;
                }
                case 2:
                    bx[n][2] = i8_scale_bytes(nib[2], lo16);
                    bx[n][3] = i8_scale_bytes(nib[3], lo16);
                    by[n][0] = i8_scale_bytes(nib[0], hi16);
                    break;
                default:
                    by[n][1] = i8_scale_bytes(nib[1], hi16);
                    by[n][2] = i8_scale_bytes(nib[2], hi16);
                    by[n][3] = i8_scale_bytes(nib[3], hi16);
                    break;
                }
            };
#pragma unroll
            for (int piece = 0; piece < 4; ++piece) {
                prep1(0, piece);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                const int c = sb & 1;
                read_a(sb < 7 ? sb + 1 : 0, aop[c ^ 1]);  // the next sub-block's operands; at the end, the second sweep's first
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const i8_intx4 av = aop[c][a];
                    const i8_intx16 zero = {0};
                    X[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bx[c], sb == 0 ? zero : X[a], 0, 0, 0);
                    if (sb < 7) {
                        prep1(sb + 1, 2 * a);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    Y[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, by[c], sb == 0 ? zero : Y[a], 0, 0, 0);
                    if (sb < 7) {
                        prep1(sb + 1, 2 * a + 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // second sweep: bz = fifth bits times the 6-bit scale, bt = the min in every byte
            i8_intx4 bz[2];
            int bt[2];
            uint32_t bits[4], sc16 = 0;
            auto prep2 = [&](int sb, int piece) {
                const int n = sb & 1;
                switch (piece) {
                case 0:
                    bits[0] = (wqh.x >> sb) & 0x01010101u;
                    bits[1] = (wqh.y >> sb) & 0x01010101u;
                    break;
                case 1:
                    bits[2] = (wqh.z >> sb) & 0x01010101u;
                    bits[3] = (wqh.w >> sb) & 0x01010101u;
                    break;
                case 2: {
                    const uint32_t sel16 = 0x0c000c00u | (uint32_t)(sb & 3) | ((uint32_t)(sb & 3) << 16);
                    sc16 = __builtin_amdgcn_perm(0u, sb < 4 ? sc_lo : sc_hi, sel16);
                    bt[n] = (int)__builtin_amdgcn_perm(0u, sb < 4 ? mn_lo : mn_hi, 0x01010101u * (sb & 3));
                    bz[n][0] = i8_scale_bytes(bits[0], sc16);
                    break;
                }
                default:
                    bz[n][1] = i8_scale_bytes(bits[1], sc16);
                    bz[n][2] = i8_scale_bytes(bits[2], sc16);
                    bz[n][3] = i8_scale_bytes(bits[3], sc16);
                    break;
                }
            };
#pragma unroll
            for (int piece = 0; piece < 4; ++piece) {
                prep2(0, piece);
            }
            // P = X + 8 Y takes X's registers; Y's become free for the second sweep
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    X[a][r] = X[a][r] + (Y[a][r] << 3);
                }
            }
            i8_intx16 Z[2], T[2];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                const int c = sb & 1;  // sweep 1 ended with sub-block 0's operands in aop[0]
                if (sb < 7) {
                    read_a(sb + 1, aop[c ^ 1]);
                }
                if (sb == 6) {
                    // activation scales: registers 4 g .. 4 g + 3 of token tile a are tokens 32 a + 8 g + 4 kh .. + 3
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            da4[a][g] = *(const float4 *)(stage + d_off + 4 * (32 * a + 8 * g));
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                const i8_intx4 btv = {bt[c], bt[c], bt[c], bt[c]};
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const i8_intx4 av = aop[c][a];
                    const i8_intx16 zero = {0};
                    Z[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bz[c], sb == 0 ? zero : Z[a], 0, 0, 0);
                    if (sb < 7) {
                        prep2(sb + 1, 2 * a);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    T[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, btv, sb == 0 ? zero : T[a], 0, 0, 0);
                    if (sb < 7) {
                        prep2(sb + 1, 2 * a + 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // once per block and output: y += a.d * (w.d * isum - w.dmin * msum)
            const float ndmin = -dmin;
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float da[4] = {da4[a][g].x, da4[a][g].y, da4[a][g].z, da4[a][g].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = 4 * g + e;
                        const int isum = X[a][r] + (Z[a][r] << 4);
                        const float v = __builtin_fmaf(ndmin, (float)T[a][r], d * (float)isum);
                        total[a][r] = __builtin_fmaf(da[e], v, total[a][r]);
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's share of the next round has landed
        i8_lds_barrier();
    }

    i8_merge_and_store<2>(p, lds, total, tid, rg, kg, j, kh, tt, row0, split);
}

// ------------------------------------------------------------------ Q6_K x Q8_K
// cpu_vec_dot_q6_k_q8_k (vec_dot_impl.h:783-828): per block y += a.d * w.d * sum_g sc_g * ((u_g - 32) . a_g) over 16
// groups of 16 values, u the unsigned 6-bit values, sc signed bytes. The scale cannot be folded into an int8 operand
// here (63 * 127), so every group is one v_mfma_i32_32x32x16_i8 per 32 x 32 tile whose result takes the scale with
// one integer multiply-add per output, and the offset is taken out as 32 * sum_g sc_g * (sum of a over group g): a
// second MFMA per group with the scale byte broadcast as the column operand, chained over the groups (exact, like the
// CPU's use of the stored sums). Same tile and wavefront roles as the Q4_K kernel, except that the two K groups share
// every block: K group kg takes the block's half kg (128 values = groups 8 kg .. 8 kg + 7, which have their own
// 64 + 32 bytes of low and high bits), so a round is one block and both groups apply the per-block scales to their
// partial sums. Blocks are 210 bytes, so a block (and, unless a row is a multiple of 8 blocks, a row) starts at any even
// address: the stage holds for each of the 128 rows the 14 chunks of 16 bytes from the one that contains the block start,
// at a stride of 240 bytes (the 15th chunk slot is not loaded), and a lane reads its row's block at that row's own offset
// (row start + 210 b) % 16 inside the row slot.
constexpr int I6_ROWB = 240;
constexpr int I6_STAGE_W = I8_WROWS * I6_ROWB;                     // 30,720
constexpr int I6_STAGE = I6_STAGE_W + I8_STAGE_A + I8_STAGE_D;     // 47,360
constexpr int I6_LDS_BYTES = 2 * I6_STAGE;                         // 94,720
static_assert(I8_OUT_TILE_BYTES <= I6_LDS_BYTES, "the output tile reuses the stages");
static_assert(I6_STAGE % 16 == 0, "stages keep 16-byte alignment");

__global__ __launch_bounds__(I8_THREADS) void k_gemm_q6k_q8k_tile(const GemmI8Params p) {
    warm_kernel_arguments<sizeof(GemmI8Params)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = wave & 3;   // weight rows 32 rg .. + 31 of the tile
    const int kg = wave >> 2;  // half of every block
    const size_t tt = blockIdx.y;
    const size_t row0 = (size_t)blockIdx.x * I8_WROWS;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nblk = (int)(b1 - b0);
    const int j = lane & 31, kh = lane >> 5;

    float total[2][16];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            total[a][r] = 0.0f;
        }
    }

    // ---- loads: 16 activation instructions (two per wavefront), 30 weight instructions of 64 chunk slots (128 rows x
    // 15 slots; wavefront w takes instructions w, w + 8, w + 16, w + 24), the activation scales by wavefront 7
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    const uint32_t last_tok = (uint32_t)(p.N - 1 - tt * I8_TOK);
    const uint8_t *tile_q = (const uint8_t *)p.qs + tt * I8_TOK * p.kp;
    uint32_t a_voff[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const uint32_t t = (uint32_t)(8 * wave + 4 * c + (lane >> 4));
        const uint32_t slot = (uint32_t)(lane & 15);
        const uint32_t trow = t < last_tok ? t : last_tok;
        a_voff[c] = trow * (uint32_t)p.kp + 16u * (slot ^ (t & 15u));
    }
    const size_t row_bytes = p.nb * Q6_K_BYTES;
    const uint32_t last_wrow = (uint32_t)(p.M - 1 - row0);
    // Rows need not start on a 16-byte boundary (210-byte blocks: they do only when a row is a multiple of 8 blocks):
    // every row's 14 chunks start at ITS OWN boundary below the block start, w_row[m] + 210 b rounded down; the tile's
    // first row is addressed from the 16-byte boundary below it (`lead` bytes before it).
    const uint32_t lead = (uint32_t)((row0 * row_bytes) & 15);
    uint32_t w_row[4], w_pc[4];
    bool w_on[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const uint32_t q = (uint32_t)(64 * (wave + 8 * m) + lane);  // chunk slot: row q / 15, chunk q % 15
        const uint32_t r = q / 15u, pc = q - 15u * r;
        const uint32_t rr = r < last_wrow ? r : last_wrow;  // rows beyond M re-read row M - 1 (never stored)
        w_row[m] = lead + rr * (uint32_t)row_bytes;
        w_pc[m] = 16u * pc;
        w_on[m] = wave + 8 * m < 30 && r < (uint32_t)I8_WROWS && pc < 14u;
    }
    const uint8_t *wbase = p.w + ((row0 * row_bytes) & ~(size_t)15);
    const size_t w_end64 = (size_t)lead + (p.M - row0) * row_bytes;  // the tensor's end, from wbase
    const uint32_t w_end = w_end64 > 0xffffffffull ? 0xffffffffu : (uint32_t)w_end64;
    uint32_t d_voff;
    {
        const uint32_t t = (uint32_t)lane;
        const uint32_t trow = t < last_tok ? t : last_tok;
        d_voff = (uint32_t)((trow * p.nb) * 4);
    }
    const uint8_t *tile_d = (const uint8_t *)(p.ad + tt * I8_TOK * p.nb);
    auto issue = [&](int bi) {
        const size_t b = b0 + (size_t)bi;
        const uint32_t s0 = lds_base + (uint32_t)((bi & 1) * I6_STAGE);
        const uint8_t *qb = tile_q + b * QK_K;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            dma_set_lds_base(s0 + (uint32_t)(I6_STAGE_W + 2048 * wave + 1024 * c));
            dma16_to_lds<0>(qb, a_voff[c]);
        }
        const uint32_t boff = (uint32_t)(b * Q6_K_BYTES);
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            if (wave + 8 * m < 30) {  // uniform over the wavefront
                dma_set_lds_base(s0 + (uint32_t)(1024 * (wave + 8 * m)));
                const uint32_t voff = ((w_row[m] + boff) & ~15u) + w_pc[m];  // from the chunk that holds the block start
                // The last chunk of the tensor's last block ends up to 14 bytes behind the tensor when its size is not
                // a multiple of 16: those bytes may not exist. Such a chunk (rows beyond M repeat it) is brought two
                // bytes at a time, only the bytes that exist, by plain loads and LDS stores; the barrier that ends
                // the round waits for both.
                const bool past = voff + 16u > w_end;
                if (w_on[m] && !past) {
                    dma16_to_lds<0>(wbase, voff);
                }
                if (w_on[m] && past) {
                    const uint32_t slot = (uint32_t)((bi & 1) * I6_STAGE + 1024 * (wave + 8 * m) + 16 * lane);
                    for (uint32_t e = 0; e < 16u && voff + e < w_end; e += 2u) {
                        *(uint16_t *)(lds + slot + e) = *(const uint16_t *)(wbase + voff + e);
                    }
                }
            }
        }
        if (wave == 7) {
            dma_set_lds_base(s0 + (uint32_t)(I6_STAGE_W + I8_STAGE_A));
            dma4_to_lds(tile_d + b * 4, d_voff);
        }
    };

    // ---- compute: weight row 32 rg + j, half kg of the block, all 64 tokens
    const uint32_t w_off = (uint32_t)((32 * rg + j) * I6_ROWB);
    uint32_t w_own;  // byte offset of this lane's weight row from wbase (the clamped row, like the loads)
    {
        const uint32_t r = (uint32_t)(32 * rg + j);
        w_own = lead + (r < last_wrow ? r : last_wrow) * (uint32_t)row_bytes;
    }
    const uint32_t a_base = (uint32_t)(I6_STAGE_W + j * QK_K + 8 * kh);
    const uint32_t d_off = (uint32_t)(I6_STAGE_W + I8_STAGE_A + 16 * kh);

    issue(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    i8_lds_barrier();
    for (int blk = 0; blk < nblk; ++blk) {
        if (blk + 1 < nblk) {
            issue(blk + 1);  // into the other buffer, which the barrier that closed the previous block has released
        }
        {
            const uint8_t *stage = lds + (size_t)(blk & 1) * I6_STAGE;
            const uint32_t o = (w_own + (uint32_t)((b0 + (size_t)blk) * Q6_K_BYTES)) & 15u;  // this lane's row
            const uint8_t *wrow = stage + w_off + o;
            uint2 scv;  // the eight scale bytes of this half
            __builtin_memcpy(&scv, wrow + 192 + 8 * kg, 8);
            uint16_t dh;
            __builtin_memcpy(&dh, wrow + 208, 2);
            float d = h2f(dh);
            asm volatile("" : "+v"(d));
            uint2 ql[2][2], qh[2];  // [second 32][second 16], [second 16]: this lane's 8 bytes each
#pragma unroll
            for (int s16 = 0; s16 < 2; ++s16) {
                __builtin_memcpy(&qh[s16], wrow + 128 + 32 * kg + 16 * s16 + 8 * kh, 8);
#pragma unroll
                for (int h32 = 0; h32 < 2; ++h32) {
                    __builtin_memcpy(&ql[h32][s16], wrow + 64 * kg + 32 * h32 + 16 * s16 + 8 * kh, 8);
                }
            }
            const uint32_t scw[2] = {scv.x, scv.y};
            // group g of this half (block group 8 kg + g): token tile a's 8 bytes of chunk 8 kg + g, swizzled by token
            auto acts_of = [&](int g, int a) {
                const uint2 v = *(const uint2 *)(stage + a_base + a * (32 * QK_K) + 16 * ((8 * kg + g) ^ (j & 15)));
                return (long)(((unsigned long)v.y << 32) | v.x);
            };
            auto weights_of = [&](int g) {
                const int q = (g >> 1) & 3, s16 = g & 1;
                const uint2 l = ql[q & 1][s16], hh = qh[s16];
                uint32_t x = (q >> 1) ? ((l.x >> 4) & 0x0f0f0f0fu) : (l.x & 0x0f0f0f0fu);
                uint32_t y = (q >> 1) ? ((l.y >> 4) & 0x0f0f0f0fu) : (l.y & 0x0f0f0f0fu);
                x |= ((hh.x >> (2 * q)) & 0x03030303u) << 4;
                y |= ((hh.y >> (2 * q)) & 0x03030303u) << 4;
                return (long)(((unsigned long)y << 32) | x);
            };
            int bsum[2][16];
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    bsum[a][r] = 0;
                }
            }
            const i8_intx16 zero = {0};
            i8_intx16 ds[2] = {zero, zero};
            i8_intx16 dq[2][2];  // [token tile][group parity]
            long av[2][2];
            float4 da4[2][4];
            long wv = weights_of(0);
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                av[a][0] = acts_of(0, a);
                dq[a][0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[a][0], wv, zero, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                const int c = g & 1;
                const uint32_t scb = (scw[g >> 2] >> (8 * (g & 3))) & 0xffu;
                const int sc = (int)(int8_t)scb;
                const uint32_t sc4 = __builtin_amdgcn_perm(0u, scw[g >> 2], 0x01010101u * (g & 3));  // byte broadcast
                const long scl = (long)(((unsigned long)sc4 << 32) | sc4);
                if (g < 7) {
                    wv = weights_of(g + 1);
                }
                if (g == 5) {
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4) {
                            da4[a][q4] = *(const float4 *)(stage + d_off + 4 * (32 * a + 8 * q4));
                        }
                    }
                }
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    ds[a] = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[a][c], scl, ds[a], 0, 0, 0);
                    if (g < 7) {
                        av[a][c ^ 1] = acts_of(g + 1, a);
                        dq[a][c ^ 1] = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[a][c ^ 1], wv, zero, 0, 0, 0);
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        bsum[a][r] += __mul24(dq[a][c][r], sc);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // once per block, output and K group: y += (a.d * w.d) * (isum - 32 * ssum)
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const float da[4] = {da4[a][q4].x, da4[a][q4].y, da4[a][q4].z, da4[a][q4].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = 4 * q4 + e;
                        const int isum = bsum[a][r] + __mul24(ds[a][r], -32);  // one multiply-add; |ds| < 2^22
                        total[a][r] = __builtin_fmaf(da[e] * d, (float)isum, total[a][r]);
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's share of the next block has landed
        i8_lds_barrier();
    }
    i8_merge_and_store<2>(p, lds, total, tid, rg, kg, j, kh, tt, row0, split);
}

// ------------------------------------------------------------------ the 32-value formats x Q8_0
// cpu_vec_dot_q8_0_q8_0 / cpu_vec_dot_q4_0_q8_0 (vec_dot_impl.h:452-479 and its Q4_0 sibling): per 32-value block
//     y += (float)(q . a) * (w.d * a.d),
// Q5_0 likewise with q = (nibble | fifth bit << 4) - 16; Q4_1 and Q5_1 (vec_dot_impl.h:186-217, 288-349) keep q
// unsigned and add w.min * a.d * sum(a) per block: a.d * sum(a) depends on the token alone and is formed once per
// round and token into LDS ([block][token], beside the scales), so the term costs one more multiply-add per output.
// integer dot exact, one fp32 multiply-add per block in block order. Here a block of 32 weight rows x 32 tokens is one
// v_mfma_i32_32x32x32_i8, and every output takes its block's product of the two scales with three vector
// instructions (convert, scale product, multiply-add): the formats have one scale per 32 values and nothing to fold,
// so the kernel is bound by these, at about an eighth of the int8 peak.
// Same tile and wavefront roles as the Q6_K kernel: a round is 256 values of K (eight blocks), K group kg takes blocks
// 4 kg .. 4 kg + 3 of every round. Weight rows must be a multiple of eight blocks (K % 256 == 0: rows and rounds start
// on 16-byte boundaries); the stage holds each row's 272 (Q8_0) / 144 (Q4_0) bytes of the round at a pitch of 304 / 144
// bytes (lanes 0..15 of a read then fall into different banks), the activation tile as in the kernels above, and the
// 8 x 64 activation scales of the round as [block][token] (one dword gather per block and round).
template <int KIND>
struct Q80Tile {
    static constexpr bool HAS_MIN = KIND == MARMOT_HIP_KIND_Q4_1 || KIND == MARMOT_HIP_KIND_Q5_1;
    static constexpr bool FIFTH = KIND == MARMOT_HIP_KIND_Q5_0 || KIND == MARMOT_HIP_KIND_Q5_1;
    static constexpr int BLK = KIND == MARMOT_HIP_KIND_Q8_0 ? 34 : 18 + (HAS_MIN ? 2 : 0) + (FIFTH ? 4 : 0);
    static constexpr int QS_AT = BLK - (KIND == MARMOT_HIP_KIND_Q8_0 ? 32 : 16);  // the values behind the header
    static constexpr int CHUNK = 8 * BLK;
    static constexpr int PIECES = CHUNK / 16;
    // an odd number of 16-byte pieces: 16 rows start in 16 different bank groups (Q8_0: 19, so that the second group a
    // read at byte 2 of a block touches is not another row's first)
    static constexpr int PITCH_P = KIND == MARMOT_HIP_KIND_Q8_0 ? 19 : (PIECES | 1);
    static constexpr int ROWB = PITCH_P * 16;
    static constexpr int STAGE_W = I8_WROWS * ROWB;
    static constexpr int STAGE_D = 8 * I8_TOK * 4;
    static constexpr int STAGE_S = HAS_MIN ? I8_TOK * 16 : 0;       // the round's 8 code sums of every token
    static constexpr int STAGE_M = HAS_MIN ? 8 * I8_TOK * 4 : 0;    // scale x sum as [block][token]
    static constexpr int STAGE = STAGE_W + I8_STAGE_A + STAGE_D + STAGE_S + STAGE_M;
    static constexpr int LDS_BYTES = 2 * STAGE;
    static constexpr int W_INSTR = (I8_WROWS * PITCH_P + 63) / 64;
    static constexpr int W_PER_WAVE = (W_INSTR + I8_WAVES - 1) / I8_WAVES;
    static_assert(CHUNK % 16 == 0 && STAGE % 16 == 0, "16-byte pieces");
    static_assert(PITCH_P >= PIECES, "a row's pieces fit its pitch");
    static_assert(I8_OUT_TILE_BYTES <= LDS_BYTES, "the output tile reuses the stages");
};

// p.nb counts rounds (K / 256); p.ad holds 8 p.nb scales per token
template <int KIND, int NA>
__global__ __launch_bounds__(I8_THREADS) void k_gemm_q80_tile(const GemmI8Params p) {
    using T = Q80Tile<KIND>;
    constexpr int TOK = 32 * NA;  // tokens per workgroup: 64, or 32 for at most 32 activation rows
    warm_kernel_arguments<sizeof(GemmI8Params)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = wave & 3;   // weight rows 32 rg .. + 31 of the tile
    const int kg = wave >> 2;  // blocks 4 kg .. 4 kg + 3 of every round
    const size_t tt = blockIdx.y;
    const size_t row0 = (size_t)blockIdx.x * I8_WROWS;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nrounds = (int)(b1 - b0);
    const int j = lane & 31, kh = lane >> 5;

    float total[NA][16];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            total[a][r] = 0.0f;
        }
    }

    // ---- loads per round: 16 activation instructions (two per wavefront), W_INSTR weight instructions of 64 piece
    // slots (wavefront w takes instructions w, w + 8, ...), one gather of 64 activation scales per wavefront
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    const uint32_t last_tok = (uint32_t)(p.N - 1 - tt * TOK);
    const uint8_t *tile_q = (const uint8_t *)p.qs + tt * TOK * p.kp;
    uint32_t a_voff[NA];
#pragma unroll
    for (int c = 0; c < NA; ++c) {
        const uint32_t t = (uint32_t)(4 * NA * wave + 4 * c + (lane >> 4));
        const uint32_t slot = (uint32_t)(lane & 15);
        const uint32_t trow = t < last_tok ? t : last_tok;
        a_voff[c] = trow * (uint32_t)p.kp + 16u * (slot ^ (t & 15u));
    }
    const size_t row_bytes = p.nb * T::CHUNK;
    const uint32_t last_wrow = (uint32_t)(p.M - 1 - row0);
    uint32_t w_voff[T::W_PER_WAVE];
    bool w_on[T::W_PER_WAVE];
#pragma unroll
    for (int m = 0; m < T::W_PER_WAVE; ++m) {
        const uint32_t q = (uint32_t)(64 * (wave + 8 * m) + lane);  // piece slot: row q / PITCH_P, piece q % PITCH_P
        const uint32_t r = q / (uint32_t)T::PITCH_P, pc = q - (uint32_t)T::PITCH_P * r;
        const uint32_t rr = r < last_wrow ? r : last_wrow;  // rows beyond M re-read row M - 1 (never stored)
        w_voff[m] = rr * (uint32_t)row_bytes + 16u * pc;
        w_on[m] = wave + 8 * m < T::W_INSTR && r < (uint32_t)I8_WROWS && pc < (uint32_t)T::PIECES;
    }
    const uint8_t *wbase = p.w + row0 * row_bytes;
    uint32_t d_voff;
    {
        const uint32_t t = (uint32_t)lane;
        const uint32_t trow = t < last_tok ? t : last_tok;
        d_voff = (uint32_t)((trow * 8u * p.nb + (uint32_t)wave) * 4u);  // block `wave` of the round, token `lane`
    }
    const uint8_t *tile_d = (const uint8_t *)(p.ad + tt * TOK * 8u * p.nb);
    const uint8_t *tile_s = (const uint8_t *)(p.sums + tt * TOK * 8u * p.nb);
    const uint32_t s_voff = (uint32_t)(((uint32_t)lane < last_tok ? (uint32_t)lane : last_tok) * 16u * p.nb);
    auto issue = [&](int ri) {
        const size_t b = b0 + (size_t)ri;
        const uint32_t s0 = lds_base + (uint32_t)((ri & 1) * T::STAGE);
        const uint8_t *qb = tile_q + b * QK_K;
#pragma unroll
        for (int c = 0; c < NA; ++c) {
            dma_set_lds_base(s0 + (uint32_t)(T::STAGE_W + 1024 * NA * wave + 1024 * c));
            dma16_to_lds<0>(qb, a_voff[c]);
        }
        const uint8_t *wb = wbase + b * T::CHUNK;
#pragma unroll
        for (int m = 0; m < T::W_PER_WAVE; ++m) {
            if (wave + 8 * m < T::W_INSTR) {  // uniform over the wavefront
                dma_set_lds_base(s0 + (uint32_t)(1024 * (wave + 8 * m)));
                if (w_on[m]) {
                    dma16_to_lds<0>(wb, w_voff[m]);
                }
            }
        }
        dma_set_lds_base(s0 + (uint32_t)(T::STAGE_W + I8_STAGE_A + 256 * wave));
        dma4_to_lds(tile_d + b * 32, d_voff);
        if constexpr (T::HAS_MIN) {
            if (wave == 7) {  // 16 bytes per token: the round's eight sums
                dma_set_lds_base(s0 + (uint32_t)(T::STAGE_W + I8_STAGE_A + T::STAGE_D));
                dma16_to_lds<0>(tile_s + b * 16, s_voff);
            }
        }
    };
    // scale x sum of a landed round, one (block, token) per thread
    auto fold_sums = [&](int ri) {
        if constexpr (T::HAS_MIN) {
            uint8_t *stage = lds + (size_t)(ri & 1) * T::STAGE;
            const int blk = tid >> 6, tok = tid & 63;
            const float da = *(const float *)(stage + T::STAGE_W + I8_STAGE_A + 4 * tid);
            const int16_t sum = *(const int16_t *)(stage + T::STAGE_W + I8_STAGE_A + T::STAGE_D + 16 * tok + 2 * blk);
            *(float *)(stage + T::STAGE_W + I8_STAGE_A + T::STAGE_D + T::STAGE_S + 4 * tid) = da * (float)sum;
            i8_lds_barrier();
        }
    };

    // ---- compute: weight row 32 rg + j, the lane's 16 values (16 kh .. + 15) of each of its four blocks, all 64 tokens
    const uint32_t w_off = (uint32_t)((32 * rg + j) * T::ROWB);
    const uint32_t a_base = (uint32_t)(T::STAGE_W + j * QK_K);
    const uint32_t d_off = (uint32_t)(T::STAGE_W + I8_STAGE_A + 16 * kh);

    issue(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    i8_lds_barrier();
    fold_sums(0);
    for (int ri = 0; ri < nrounds; ++ri) {
        if (ri + 1 < nrounds) {
            issue(ri + 1);  // into the other buffer, which the barrier that closed the previous round has released
        }
        {
            const uint8_t *stage = lds + (size_t)(ri & 1) * T::STAGE;
            const uint8_t *wrow = stage + w_off;
            const i8_intx16 zero = {0};
#pragma unroll
            for (int bi = 0; bi < 4; ++bi) {
                const int blk = 4 * kg + bi;
                uint16_t dh;
                __builtin_memcpy(&dh, wrow + T::BLK * blk, 2);
                float dw = h2f(dh);
                asm volatile("" : "+v"(dw));  // a conversion of its own (not folded into mixed-precision multiplies)
                float mw = 0.0f;
                if constexpr (T::HAS_MIN) {
                    uint16_t mh;
                    __builtin_memcpy(&mh, wrow + T::BLK * blk + 2, 2);
                    mw = h2f(mh);
                    asm volatile("" : "+v"(mw));
                }
                i8_intx4 wv;
                if constexpr (KIND == MARMOT_HIP_KIND_Q8_0) {
                    __builtin_memcpy(&wv, wrow + T::BLK * blk + 2 + 16 * kh, 16);
                } else {
                    // byte i of the block: value i in the low nibble, value 16 + i in the high nibble; Q5_0 / Q5_1: bit
                    // i (16 + i) of the 32-bit word before them is the value's fifth bit. Q4_0: (n + 0x78) ^ 0x80 is
                    // n - 8 as a signed byte, Q5_0: (v + 0x70) ^ 0x80 is v - 16, both without carries between bytes.
                    uint4 raw;
                    __builtin_memcpy(&raw, wrow + T::BLK * blk + T::QS_AT, 16);
                    const uint32_t rw[4] = {raw.x, raw.y, raw.z, raw.w};
                    uint32_t qh = 0u;
                    if constexpr (T::FIFTH) {
                        __builtin_memcpy(&qh, wrow + T::BLK * blk + T::QS_AT - 4, 4);
                        qh = kh ? qh >> 16 : qh;
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        uint32_t v = (kh ? (rw[e] >> 4) : rw[e]) & 0x0f0f0f0fu;
                        if constexpr (T::FIFTH) {  // bits 4 e .. 4 e + 3 to bit 4 of bytes 0 .. 3
                            v |= ((((qh >> (4 * e)) & 0xfu) * 0x00204081u) & 0x01010101u) << 4;
                        }
                        if constexpr (KIND == MARMOT_HIP_KIND_Q4_0) {
                            v = (v + 0x78787878u) ^ 0x80808080u;
                        } else if constexpr (KIND == MARMOT_HIP_KIND_Q5_0) {
                            v = (v + 0x70707070u) ^ 0x80808080u;
                        }
                        wv[e] = (int)v;
                    }
                }
#pragma unroll
                for (int a = 0; a < NA; ++a) {
                    const i8_intx4 av = *(const i8_intx4 *)(stage + a_base + a * (32 * QK_K) +
                                                           16 * ((2 * blk + kh) ^ (j & 15)));
                    const i8_intx16 dq = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, wv, zero, 0, 0, 0);
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        const float4 d4 = *(const float4 *)(stage + d_off + 256 * blk + 4 * (32 * a + 8 * q4));
                        const float da[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int r = 4 * q4 + e;
                            total[a][r] = __builtin_fmaf((float)dq[r], dw * da[e], total[a][r]);
                        }
                        if constexpr (T::HAS_MIN) {
                            const float4 m4 = *(const float4 *)(stage + d_off + T::STAGE_D + T::STAGE_S + 256 * blk +
                                                                4 * (32 * a + 8 * q4));
                            const float ms[4] = {m4.x, m4.y, m4.z, m4.w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int r = 4 * q4 + e;
                                total[a][r] = __builtin_fmaf(mw, ms[e], total[a][r]);
                            }
                        }
                    }
                    if constexpr (T::HAS_MIN) {
                        // one matrix product and its 16 outputs at a time (left alone, the compiler forms all eight
                        // products of the round first and spills their 128 results)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            asm volatile("" : "+v"(total[a][r]));
                        }
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's share of the next round has landed
        i8_lds_barrier();
        if (ri + 1 < nrounds) {
            fold_sums(ri + 1);
        }
    }
    i8_merge_and_store<NA>(p, lds, total, tid, rg, kg, j, kh, tt, row0, split);
}

// ------------------------------------------------------------------ Q2_K / Q3_K x Q8_K
// cpu_vec_dot_q2_k_q8_k (vec_dot_impl.h:560-618): per block y += (a.d * w.d) * isum - (a.d * w.dmin) * summs with
//     isum = sum over the 16 groups of 16 values of (group scale) * (q2 . a),   summs = sum (group min) * (sum of a),
// cpu_vec_dot_q3_k_q8_k (:620-687): y += (a.d * w.d) * sum over groups of (six-bit scale - 32) * (q3 . a), q3 the
// two-bit value minus 4 unless its mask bit is set. Groups of 16 values carry their own scale, and a matrix instruction
// spans two of them, so the scale is multiplied into the int8 operand (both kh halves of a product then differ only in
// the operand bytes), and what would not fit a signed byte goes into a second chain of products:
//   Q2_K: chain 1 = q2 * scale (0 .. 45), chain 2 = the group's min in every byte (its product is min * sum of a);
//   Q3_K: q3 = 2 vh + vb with vh in -2 .. 1 and vb in 0 .. 1: chain 1 = vh * scale (-64 .. 64), chain 2 = vb * scale,
//         isum = 2 * chain 1 + chain 2 (q3 * scale itself reaches +128).
// Four packed bytes are multiplied by one small factor in a single 32-bit multiply where no byte's product reaches 256.
// Same tile and wavefront roles as the kernels above (a round is one block; K group kg takes its steps 4 kg .. + 3), but
// the weights do not pass through LDS: lane (j, kh) is the only reader of its row's bytes for its half of every step
// (16 + 8 + 4 bytes per block for Q2_K, 16 + 16 + 12 + 2 for Q3_K), requested a round ahead into registers; rows of
// 84 / 110 bytes need only 4- / 2-byte alignment.
constexpr int I23_STAGE = I8_STAGE_A + I8_STAGE_D;  // 64 tokens x 256 codes + 64 block scales: 16,640 bytes
constexpr int I23_LDS_BYTES = (I8_OUT_TILE_BYTES > 2 * I23_STAGE) ? I8_OUT_TILE_BYTES : 2 * I23_STAGE;

template <int KIND>
struct Q23Raw;
template <>
struct Q23Raw<MARMOT_HIP_KIND_Q2_K> {
    uint4 q;        // qs[32 kg + 16 kh ..]: the lane's 16 values of steps 4 kg .. 4 kg + 3, two bits per step
    uint2 sc;       // scales[8 kg ..]: group 8 kg + 2 bi + kh belongs to step bi
    uint32_t dd;    // d, dmin
    __device__ __forceinline__ void fetch(const uint8_t *b, int kg, int kh) {
        __builtin_memcpy(&sc, b + 8 * kg, 8);
        __builtin_memcpy(&q, b + 16 + 32 * kg + 16 * kh, 16);
        __builtin_memcpy(&dd, b + 80, 4);
    }
};
template <>
struct Q23Raw<MARMOT_HIP_KIND_Q3_K> {
    uint4 q, hm;    // qs[32 kg + 16 kh ..], hmask[16 kh ..] (bit s of a mask byte belongs to step s)
    uint32_t t0, t1, t2;
    uint16_t d;
    __device__ __forceinline__ void fetch(const uint8_t *b, int kg, int kh) {
        __builtin_memcpy(&hm, b + 16 * kh, 16);
        __builtin_memcpy(&q, b + 32 + 32 * kg + 16 * kh, 16);
        __builtin_memcpy(&t0, b + 96, 4);
        __builtin_memcpy(&t1, b + 100, 4);
        __builtin_memcpy(&t2, b + 104, 4);
        __builtin_memcpy(&d, b + 108, 2);
    }
};

template <int KIND, int NA>
__global__ __launch_bounds__(I8_THREADS) void k_gemm_q23k_tile(const GemmI8Params p) {
    constexpr int TOK = 32 * NA;  // tokens per workgroup: 64, or 32 for at most 32 activation rows
    constexpr bool Q2 = KIND == MARMOT_HIP_KIND_Q2_K;
    constexpr int BB = Q2 ? Q2_K_BYTES : Q3_K_BYTES;
    warm_kernel_arguments<sizeof(GemmI8Params)>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = wave & 3;   // weight rows 32 rg .. + 31 of the tile
    const int kg = wave >> 2;  // steps 4 kg .. 4 kg + 3 of every block
    const size_t tt = blockIdx.y;
    const size_t row0 = (size_t)blockIdx.x * I8_WROWS;
    const int split = blockIdx.z;
    const size_t b0 = (size_t)split * p.blocks_per_split;
    size_t b1 = b0 + p.blocks_per_split;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nrounds = (int)(b1 - b0);
    const int j = lane & 31, kh = lane >> 5;

    float total[NA][16];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            total[a][r] = 0.0f;
        }
    }

    // ---- loads per round: 16 activation instructions (two per wavefront), one gather of the 64 block scales
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    const uint32_t last_tok = (uint32_t)(p.N - 1 - tt * TOK);
    const uint8_t *tile_q = (const uint8_t *)p.qs + tt * TOK * p.kp;
    uint32_t a_voff[NA];
#pragma unroll
    for (int c = 0; c < NA; ++c) {
        const uint32_t t = (uint32_t)(4 * NA * wave + 4 * c + (lane >> 4));
        const uint32_t slot = (uint32_t)(lane & 15);
        const uint32_t trow = t < last_tok ? t : last_tok;
        a_voff[c] = trow * (uint32_t)p.kp + 16u * (slot ^ (t & 15u));
    }
    const uint32_t d_voff = (uint32_t)(((uint32_t)lane < last_tok ? (uint32_t)lane : last_tok) * 4u * p.nb);
    const uint8_t *tile_d = (const uint8_t *)(p.ad + tt * TOK * p.nb);
    size_t wr = row0 + (size_t)(32 * rg + j);
    wr = wr < p.M ? wr : p.M - 1;  // rows beyond M re-read row M - 1 (never stored)
    const uint8_t *wrow = p.w + wr * (p.nb * BB) + b0 * BB;
    auto issue = [&](int ri, Q23Raw<KIND> &raw) {
        const size_t b = b0 + (size_t)ri;
        const uint32_t s0 = lds_base + (uint32_t)((ri & 1) * I23_STAGE);
        const uint8_t *qb = tile_q + b * QK_K;
#pragma unroll
        for (int c = 0; c < NA; ++c) {
            dma_set_lds_base(s0 + (uint32_t)(1024 * NA * wave + 1024 * c));
            dma16_to_lds<0>(qb, a_voff[c]);
        }
        if (wave == 0) {
            dma_set_lds_base(s0 + (uint32_t)I8_STAGE_A);
            dma4_to_lds(tile_d + b * 4, d_voff);
        }
        raw.fetch(wrow + (size_t)ri * BB, kg, kh);
    };

    const uint32_t a_base = (uint32_t)(j * QK_K);
    const uint32_t d_off = (uint32_t)(I8_STAGE_A + 16 * kh);
    Q23Raw<KIND> cur, nxt;
    issue(0, cur);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    i8_lds_barrier();
    for (int ri = 0; ri < nrounds; ++ri) {
        if (ri + 1 < nrounds) {
            issue(ri + 1, nxt);  // into the other buffer, which the barrier that closed the previous round has released
        }
        {
            const uint8_t *stage = lds + (size_t)(ri & 1) * I23_STAGE;
            i8_intx16 c1[NA], c2[NA];
#pragma unroll
            for (int a = 0; a < NA; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    c1[a][r] = 0;
                    c2[a][r] = 0;
                }
            }
            const uint32_t qw[4] = {cur.q.x, cur.q.y, cur.q.z, cur.q.w};
#pragma unroll
            for (int bi = 0; bi < 4; ++bi) {
                const int step = 4 * kg + bi;
                i8_intx4 w1, w2;
                if constexpr (Q2) {
                    const uint32_t scb = ((bi < 2 ? cur.sc.x : cur.sc.y) >> (8 * (2 * (bi & 1) + kh))) & 0xffu;
                    const uint32_t dsc = scb & 0xfu, mn = scb >> 4;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        w1[e] = (int)(((qw[e] >> (2 * bi)) & 0x03030303u) * dsc);
                        w2[e] = (int)(mn * 0x01010101u);
                    }
                } else {
                    // q3k_group_scale(scales, is) for group is = 2 step + kh, plus 32: low nibble from scales[is]
                    // (is < 8) or the high nibble of scales[is - 8], two more bits from scales[8 + is % 4]
                    const int is = 2 * step + kh;
                    const uint64_t low8 = (uint64_t)cur.t0 | ((uint64_t)cur.t1 << 32);
                    const uint32_t low = (uint32_t)(low8 >> (8 * (is & 7) + (is < 8 ? 0 : 4))) & 0xfu;
                    const uint32_t high = (cur.t2 >> (8 * (is & 3) + 2 * (is >> 2))) & 3u;
                    const uint32_t sp = low | (high << 4);              // scale + 32: 0 .. 63
                    const uint32_t sbyte = (sp - 32u) & 0xffu;          // the scale as a signed byte
                    const uint32_t bias = (uint32_t)((96 - 2 * (int)sp) * 0x01010101);
                    const uint32_t hw[4] = {cur.hm.x, cur.hm.y, cur.hm.z, cur.hm.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t q2 = (qw[e] >> (2 * bi)) & 0x03030303u;
                        const uint32_t hb = (hw[e] >> step) & 0x01010101u;
                        const uint32_t uh = ((q2 >> 1) & 0x01010101u) | (hb << 1);  // (q3 + 4) / 2: 0 .. 3
                        // vh * s + 128 = uh * sp + 32 (3 - uh) + 96 - 2 sp with vh = uh - 2, s = sp - 32: every partial
                        // sum stays inside 0 .. 255 in every byte
                        const uint32_t biased = uh * sp + ((uh ^ 0x03030303u) << 5) + bias;
                        w1[e] = (int)(biased ^ 0x80808080u);
                        w2[e] = (int)((q2 & 0x01010101u) * sbyte);
                    }
                }
#pragma unroll
                for (int a = 0; a < NA; ++a) {
                    const i8_intx4 av = *(const i8_intx4 *)(stage + a_base + a * (32 * QK_K) +
                                                           16 * ((2 * step + kh) ^ (j & 15)));
                    c1[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, w1, c1[a], 0, 0, 0);
                    c2[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, w2, c2[a], 0, 0, 0);
                }
            }
            float dw, dmw = 0.0f;
            if constexpr (Q2) {
                dw = h2f((uint16_t)(cur.dd & 0xffffu));
                dmw = h2f((uint16_t)(cur.dd >> 16));
                asm volatile("" : "+v"(dmw));
            } else {
                dw = h2f(cur.d);
            }
            asm volatile("" : "+v"(dw));  // conversions of their own (not folded into mixed-precision multiplies)
#pragma unroll
            for (int a = 0; a < NA; ++a) {
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const float4 d4 = *(const float4 *)(stage + d_off + 4 * (32 * a + 8 * q4));
                    const float da[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = 4 * q4 + e;
                        if constexpr (Q2) {
                            float t = __builtin_fmaf(da[e] * dw, (float)c1[a][r], total[a][r]);
                            total[a][r] = __builtin_fmaf(-(da[e] * dmw), (float)c2[a][r], t);
                        } else {
                            total[a][r] = __builtin_fmaf(da[e] * dw, (float)(2 * c1[a][r] + c2[a][r]), total[a][r]);
                        }
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the next round's activations and this lane's weights are here
        i8_lds_barrier();
        if (ri + 1 < nrounds) {
            cur = nxt;
        }
    }
    i8_merge_and_store<NA>(p, lds, total, tid, rg, kg, j, kh, tt, row0, split);
}

// ------------------------------------------------------------------ host side
// From this many activation rows on (more than one 32-row pass of the streaming small-batch kernel) the tile kernel
// is the faster one on every shape measured (4096 x 4096, 14336 x 4096, 4096 x 14336; e.g. 4096 x 14336 at 48 rows
// 24.8 us against 58.8 us, at 512 rows 113 us against 186 us).
constexpr size_t I8_MIN_ROWS = 33;

static size_t gemm_i8_splits(const marmot_hip_device *dev, size_t N, size_t M, size_t nb, size_t *blocks_per_split) {
    const size_t tiles = ((N + I8_TOK - 1) / I8_TOK) * ((M + I8_WROWS - 1) / I8_WROWS);
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    size_t splits = 1;
    if (tiles * 2 <= cus) {  // fewer tiles than half the chip: split K across workgroups (short prompts)
        splits = cus / tiles;
        const size_t max_splits = nb / 2 > 0 ? nb / 2 : 1;  // at least two blocks per workgroup
        splits = splits > max_splits ? max_splits : splits;
    }
    const size_t bps = (nb + splits - 1) / splits;
    *blocks_per_split = bps;
    return (nb + bps - 1) / bps;
}

bool gemm_i8_applies(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *const *weights, int count,
                     const ActScratch &act) {
    // Q6_K: the small-batch kernel holds 16 rows per pass, and from the second pass on the tile is faster (14336 x 4096
    // at 17 .. 32 rows: 48 us in two passes, the tile 41 us at 33 rows; 18944 x 3584: 87 - 94 against 63 us)
    const size_t min_rows = kind == MARMOT_HIP_KIND_Q6_K ? 17 : I8_MIN_ROWS;
    if (dev->knobs.no_gemm_i8 || N < min_rows || K % QK_K != 0) {
        return false;
    }
    size_t block_bytes = Q4_K_BYTES;
    if (kind == MARMOT_HIP_KIND_Q5_K) {
        block_bytes = Q5_K_BYTES;
    } else if (kind == MARMOT_HIP_KIND_Q6_K) {
        block_bytes = Q6_K_BYTES;  // (rows of 210-byte blocks need not be 16-byte aligned: the kernel rounds down per row)
    } else if (kind != MARMOT_HIP_KIND_Q4_K) {
        return false;
    }
    if ((((uintptr_t)act.qs) & 15) != 0 || act.kp % 16 != 0 || N * act.kp >= ((size_t)1 << 32) ||
        N * (K / QK_K) * 4 >= ((size_t)1 << 32) || I8_WROWS * (K / QK_K) * block_bytes >= ((size_t)1 << 32)) {
        return false;  // 16-byte direct-to-LDS loads with 32-bit lane offsets
    }
    for (int i = 0; i < count; ++i) {
        if ((((uintptr_t)weights[i]) & 15) != 0) {
            return false;
        }
    }
    return true;
}

size_t gemm_i8_scratch_bytes(const marmot_hip_device *dev, size_t N, size_t K, size_t M, int weights) {
    size_t bps = 0;
    const size_t splits = gemm_i8_splits(dev, N, M, K / QK_K, &bps);
    return splits > 1 ? splits * N * M * sizeof(float) * (size_t)weights : 0;
}

int launch_gemm_i8(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                   size_t M, int out_dtype, void *scratch) {
    const bool q6 = kind == MARMOT_HIP_KIND_Q6_K, q5 = kind == MARMOT_HIP_KIND_Q5_K;
    const size_t nb = K / QK_K;
    size_t bps = 0;
    const size_t splits = gemm_i8_splits(dev, N, M, nb, &bps);
    float *partial = (float *)scratch;
    if (splits > 1 && partial == nullptr) {
        void *wsp = nullptr;
        MH_TRY(workspace_reserve(dev, gemm_i8_scratch_bytes(dev, N, K, M, ws.count), &wsp));
        partial = (float *)wsp;
    }
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q4k_q8k_tile));
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q6k_q8k_tile));
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q5k_q8k_tile));
    const dim3 grid((unsigned)((M + I8_WROWS - 1) / I8_WROWS), (unsigned)((N + I8_TOK - 1) / I8_TOK), (unsigned)splits);
    for (int which = 0; which < ws.count; ++which) {
        GemmI8Params p;
        p.w = (const uint8_t *)ws.w[which];
        p.qs = act.qs;
        p.ad = act.d;
        p.kp = act.kp;
        p.N = N;
        p.M = M;
        p.nb = nb;
        float *part = splits > 1 ? partial + (size_t)which * splits * N * M : nullptr;
        p.out = splits > 1 ? (void *)part : ws.out[which];
        p.splits = (int)splits;
        p.blocks_per_split = (int)bps;
        p.bias = ws.bias[which];
        p.bias_is_f16 = ws.bias_dtype == MARMOT_HIP_DTYPE_F16;
        p.bias_first = ws.bias_first ? 1 : 0;
        p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
        if (q6) {
            hipLaunchKernelGGL(k_gemm_q6k_q8k_tile, grid, dim3(I8_THREADS), I6_LDS_BYTES, dev->stream, p);
        } else if (q5) {
            hipLaunchKernelGGL(k_gemm_q5k_q8k_tile, grid, dim3(I8_THREADS), I5_LDS_BYTES, dev->stream, p);
        } else {
            hipLaunchKernelGGL(k_gemm_q4k_q8k_tile, grid, dim3(I8_THREADS), I8_LDS_BYTES, dev->stream, p);
        }
        MH_HIP(hipGetLastError());
        if (splits > 1) {
            MH_TRY(launch_splitk_reduce(dev, part, (int)splits, N, M, ws.bias[which], ws.bias_dtype, ws.out[which],
                                        out_dtype, ws.bias_first));
        }
    }
    set_route(q6 ? "mmq_q6_k_q8_k_mfma_tile" : q5 ? "mmq_q5_k_q8_k_mfma_tile" : "mmq_q4_k_q8_k_mfma_tile");
    return MARMOT_HIP_SUCCESS;
}

// Q8_0 / Q4_0 weights on Q8_0 activations: rows of whole rounds (K % 256 == 0), nine activation rows and more (up to
// eight the packed matvec streams the weights once; measured at 4096 x 4096 / 14336 x 4096: the matvec takes 16.6 /
// 33 us at 9 rows and 34 / 74 us at 32, this kernel 16 / 30 us at 33)
constexpr size_t Q80_MIN_ROWS = 9;
// Q2_K / Q3_K: the packed matvec is bound by the unpacking of its many values per byte and pays it once per activation
// row (14336 x 4096: 10 / 20 / 23 us (Q2_K), 13 / 23 / 34 us (Q3_K) at 1 / 4 / 8 rows; the tile 20 / 24 us at 16 rows)
constexpr size_t Q23K_MIN_ROWS = 5;
size_t gemm_q80_min_rows(int kind) {
    return (kind == MARMOT_HIP_KIND_Q2_K || kind == MARMOT_HIP_KIND_Q3_K) ? Q23K_MIN_ROWS : Q80_MIN_ROWS;
}
static bool q80_format(int kind) {
    return kind == MARMOT_HIP_KIND_Q8_0 || kind == MARMOT_HIP_KIND_Q4_0 || kind == MARMOT_HIP_KIND_Q4_1 ||
           kind == MARMOT_HIP_KIND_Q5_0 || kind == MARMOT_HIP_KIND_Q5_1;
}
static bool q23k_format(int kind) {
    return kind == MARMOT_HIP_KIND_Q2_K || kind == MARMOT_HIP_KIND_Q3_K;
}
bool gemm_q80_kind(int kind) {
    return q80_format(kind) || q23k_format(kind);
}

bool gemm_q80_applies(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *const *weights, int count,
                      const ActScratch &act) {
    if (q23k_format(kind)) {
        return gemm_q23k_applies(dev, kind, N, K, weights, count, act);
    }
    if (dev->knobs.no_gemm_i8 || N < Q80_MIN_ROWS || K % QK_K != 0 || !q80_format(kind)) {
        return false;
    }
    const size_t chunk = 8 * block_bytes(kind);
    if ((((uintptr_t)act.qs) & 15) != 0 || act.kp % 16 != 0 || N * act.kp >= ((size_t)1 << 32) ||
        N * (K / 32) * 4 >= ((size_t)1 << 32) || I8_WROWS * (K / QK_K) * chunk >= ((size_t)1 << 32) ||
        (((uintptr_t)act.sums) & 15) != 0) {
        return false;  // 16-byte direct-to-LDS loads with 32-bit lane offsets
    }
    for (int i = 0; i < count; ++i) {
        if ((((uintptr_t)weights[i]) & 15) != 0) {
            return false;
        }
    }
    return true;
}

// at most 32 activation rows: the form with one token tile of 32 per workgroup (half the matrix instructions and
// epilogue of the 64-token form, whose second tile would hold no token)
template <int KIND>
static int launch_gemm_q80_kind(marmot_hip_device *dev, const GemmI8Params &p, dim3 grid) {
    if (p.N <= 32) {
        MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q80_tile<KIND, 1>));
        hipLaunchKernelGGL((k_gemm_q80_tile<KIND, 1>), grid, dim3(I8_THREADS), Q80Tile<KIND>::LDS_BYTES, dev->stream, p);
    } else {
        MH_TRY(allow_large_lds(dev, (const void *)k_gemm_q80_tile<KIND, 2>));
        hipLaunchKernelGGL((k_gemm_q80_tile<KIND, 2>), grid, dim3(I8_THREADS), Q80Tile<KIND>::LDS_BYTES, dev->stream, p);
    }
    return MARMOT_HIP_SUCCESS;
}

int launch_gemm_q80(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                    size_t M, int out_dtype, void *scratch) {
    if (q23k_format(kind)) {
        return launch_gemm_q23k(dev, kind, ws, act, N, K, M, out_dtype, scratch);
    }
    const size_t nb = K / QK_K;
    size_t bps = 0;
    const size_t splits = gemm_i8_splits(dev, N, M, nb, &bps);
    float *partial = (float *)scratch;
    if (splits > 1 && partial == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "tiled Q8_0 GEMM: no room for the K-split partial sums");
    }
    const dim3 grid((unsigned)((M + I8_WROWS - 1) / I8_WROWS), (unsigned)((N + I8_TOK - 1) / I8_TOK), (unsigned)splits);
    for (int which = 0; which < ws.count; ++which) {
        GemmI8Params p;
        p.w = (const uint8_t *)ws.w[which];
        p.qs = act.qs;
        p.ad = act.d;
        p.sums = act.sums;
        p.kp = act.kp;
        p.N = N;
        p.M = M;
        p.nb = nb;
        float *part = splits > 1 ? partial + (size_t)which * splits * N * M : nullptr;
        p.out = splits > 1 ? (void *)part : ws.out[which];
        p.splits = (int)splits;
        p.blocks_per_split = (int)bps;
        p.bias = ws.bias[which];
        p.bias_is_f16 = ws.bias_dtype == MARMOT_HIP_DTYPE_F16;
        p.bias_first = ws.bias_first ? 1 : 0;
        p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
        switch (kind) {
        case MARMOT_HIP_KIND_Q8_0:
            MH_TRY(launch_gemm_q80_kind<MARMOT_HIP_KIND_Q8_0>(dev, p, grid));
            break;
        case MARMOT_HIP_KIND_Q4_0:
            MH_TRY(launch_gemm_q80_kind<MARMOT_HIP_KIND_Q4_0>(dev, p, grid));
            break;
        case MARMOT_HIP_KIND_Q4_1:
            MH_TRY(launch_gemm_q80_kind<MARMOT_HIP_KIND_Q4_1>(dev, p, grid));
            break;
        case MARMOT_HIP_KIND_Q5_0:
            MH_TRY(launch_gemm_q80_kind<MARMOT_HIP_KIND_Q5_0>(dev, p, grid));
            break;
        default:
            MH_TRY(launch_gemm_q80_kind<MARMOT_HIP_KIND_Q5_1>(dev, p, grid));
            break;
        }
        MH_HIP(hipGetLastError());
        if (splits > 1) {
            MH_TRY(launch_splitk_reduce(dev, part, (int)splits, N, M, ws.bias[which], ws.bias_dtype, ws.out[which],
                                        out_dtype, ws.bias_first));
        }
    }
    static const char *const routes[] = {"gemm_q8_0_q8_0_mfma_tile", "gemm_q4_0_q8_0_mfma_tile", "gemm_q4_1_q8_0_mfma_tile",
                                         "gemm_q5_0_q8_0_mfma_tile", "gemm_q5_1_q8_0_mfma_tile"};
    set_route(routes[kind == MARMOT_HIP_KIND_Q8_0   ? 0
                     : kind == MARMOT_HIP_KIND_Q4_0 ? 1
                     : kind == MARMOT_HIP_KIND_Q4_1 ? 2
                     : kind == MARMOT_HIP_KIND_Q5_0 ? 3
                                                    : 4]);
    return MARMOT_HIP_SUCCESS;
}

// Q2_K / Q3_K weights on Q8_K activations, nine activation rows and more (up to eight the packed matvec streams the
// weights once)
bool gemm_q23k_applies(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *const *weights, int count,
                       const ActScratch &act) {
    if (dev->knobs.no_gemm_i8 || N < Q23K_MIN_ROWS || K % QK_K != 0 ||
        (kind != MARMOT_HIP_KIND_Q2_K && kind != MARMOT_HIP_KIND_Q3_K)) {
        return false;
    }
    if ((((uintptr_t)act.qs) & 15) != 0 || act.kp % 16 != 0 || N * act.kp >= ((size_t)1 << 32) ||
        N * (K / QK_K) * 4 >= ((size_t)1 << 32)) {
        return false;  // 16-byte direct-to-LDS loads with 32-bit lane offsets
    }
    for (int i = 0; i < count; ++i) {
        if ((((uintptr_t)weights[i]) & 3) != 0) {
            return false;
        }
    }
    return true;
}

int launch_gemm_q23k(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                     size_t M, int out_dtype, void *scratch) {
    const bool q2 = kind == MARMOT_HIP_KIND_Q2_K;
    const size_t nb = K / QK_K;
    size_t bps = 0;
    const size_t splits = gemm_i8_splits(dev, N, M, nb, &bps);
    float *partial = (float *)scratch;
    if (splits > 1 && partial == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "tiled Q2_K / Q3_K GEMM: no room for the K-split partial sums");
    }
    const dim3 grid((unsigned)((M + I8_WROWS - 1) / I8_WROWS), (unsigned)((N + I8_TOK - 1) / I8_TOK), (unsigned)splits);
    for (int which = 0; which < ws.count; ++which) {
        GemmI8Params p;
        p.w = (const uint8_t *)ws.w[which];
        p.qs = act.qs;
        p.ad = act.d;
        p.kp = act.kp;
        p.N = N;
        p.M = M;
        p.nb = nb;
        float *part = splits > 1 ? partial + (size_t)which * splits * N * M : nullptr;
        p.out = splits > 1 ? (void *)part : ws.out[which];
        p.splits = (int)splits;
        p.blocks_per_split = (int)bps;
        p.bias = ws.bias[which];
        p.bias_is_f16 = ws.bias_dtype == MARMOT_HIP_DTYPE_F16;
        p.bias_first = ws.bias_first ? 1 : 0;
        p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
        if (N <= 32) {  // one token tile of 32 per workgroup
            if (q2) {
                hipLaunchKernelGGL((k_gemm_q23k_tile<MARMOT_HIP_KIND_Q2_K, 1>), grid, dim3(I8_THREADS), I23_LDS_BYTES,
                                   dev->stream, p);
            } else {
                hipLaunchKernelGGL((k_gemm_q23k_tile<MARMOT_HIP_KIND_Q3_K, 1>), grid, dim3(I8_THREADS), I23_LDS_BYTES,
                                   dev->stream, p);
            }
        } else if (q2) {
            hipLaunchKernelGGL((k_gemm_q23k_tile<MARMOT_HIP_KIND_Q2_K, 2>), grid, dim3(I8_THREADS), I23_LDS_BYTES,
                               dev->stream, p);
        } else {
            hipLaunchKernelGGL((k_gemm_q23k_tile<MARMOT_HIP_KIND_Q3_K, 2>), grid, dim3(I8_THREADS), I23_LDS_BYTES,
                               dev->stream, p);
        }
        MH_HIP(hipGetLastError());
        if (splits > 1) {
            MH_TRY(launch_splitk_reduce(dev, part, (int)splits, N, M, ws.bias[which], ws.bias_dtype, ws.out[which],
                                        out_dtype, ws.bias_first));
        }
    }
    set_route(q2 ? "gemm_q2_k_q8_k_mfma_tile" : "gemm_q3_k_q8_k_mfma_tile");
    return MARMOT_HIP_SUCCESS;
}

} // namespace mh

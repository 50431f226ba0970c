// Small-batch quantized matmul on the int8 matrix cores: Q4_K / Q6_K weights x Q8_K activations for 3..16 activation rows
// per pass (continuous-batching decode, the layer stack at 16 sequences, MoE expert segments).
//
// Same integer arithmetic as cpu_vec_dot_q4_k_q8_k (vec_dot_impl.h:689-732): per 256-value block
//     bsum = sum_j sc_j * (q_j . a_j),   msum = sum_j mn_j * (sum of a over sub-block j),
//     y += (a.d * w.d) * bsum - (a.d * w.dmin) * msum
// but the 32-value sub-block dots of 32 weight rows x up to 32 activation rows are one v_mfma_i32_32x32x32_i8:
// activations are the row operand (token i = lane % 32), unpacked nibbles of weight row j = lane % 32 the column
// operand, so every lane ends up with the int32 dots of ITS weight row against 16 tokens and applies its own 6-bit
// scale with one integer multiply-add per token. The min term needs sum_k mn_j(k) * a_k, which is a second MFMA per
// sub-block with the byte mn_j broadcast as the column operand, chained through the accumulator over the 8
// sub-blocks. All integer results are exact; only the fp32 accumulation over blocks is ordered differently from the
// CPU (per wavefront sequential, then across the K-split in a fixed order).
//
// A consumer wavefront owns 32 weight rows and a contiguous range of blocks; W of them per workgroup and S workgroups
// split K so that the chip is filled even when M / 32 is small. Weights stream from HBM exactly once per pass, as
// direct-to-LDS loads; activations (int8, L2-resident) take the same way into the same stage.
#include "mh_common.h"

#include <stdlib.h>

namespace mh {

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));

struct MmqParams {
    const uint8_t *w[3];   // blocks, M rows of nb blocks: nw weights of one shape sharing the activations
    void *out[3];          // [N][M] of out dtype, or fp32 partials [splits][N][M] when splits > 1
    int nw;                // weights in this launch: blockIdx.y = split * nw + weight
    const int8_t *qs;      // quantized activations, rows of kp bytes
    const float *ad;       // activation block scales [rows][nb]
    size_t kp;
    size_t N, M, nb;
    size_t n0;             // first activation row of this pass
    int ncols;             // activation rows of this pass (<= 32)
    int bpw;               // blocks per wavefront
    int splits;            // workgroups along K
    const void *bias[3];
    int bias_is_f16;
    int bias_first;        // fp16 output: f16(dot + bias) instead of f16(f16(dot) + bias)
    int out_is_f16;
    // grouped (MoE) mode: blockIdx.z selects a work item = up to 8 consecutive routes of one expert
    const int4 *items;
    const int *n_items;
    const uint32_t *act_index;
    size_t expert_stride;
};

typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef const __attribute__((address_space(1))) uint8_t glb_u8;

constexpr int MMQ_TOK = 16;                // activation rows per pass
// one block of 32 weight rows is 32 * 144 = 4608 bytes of Q4_K, 32 * 176 = 5632 bytes of Q5_K
constexpr int MMQ_ABLK = MMQ_TOK * QK_K;   // one block of 16 activation rows: 4096 bytes
constexpr int MMQ_STAGES = 2;              // Q6_K: blocks in flight per wavefront

// ---- shared epilogue pieces of the small-batch kernels
// K-split within the workgroup: the consumers' partial sums meet in LDS and wavefront 0 adds them in wavefront order
// (all of them requested before the first addition: W <= 4). Every wavefront of the workgroup calls this (it contains
// a barrier); returns true for the wavefront that goes on to store.
template <int NR>
__device__ __forceinline__ bool mmq_reduce_consumers(float *red, int W, int wave, int lane, bool is_consumer,
                                                     float (&acc)[NR]) {
    if (is_consumer) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            red[(wave * NR + r) * 64 + lane] = acc[r];
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    if (wave != 0) {
        return false;
    }
    float part[4][NR];
#pragma unroll
    for (int w2 = 0; w2 < 4; ++w2) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            part[w2][r] = w2 < W ? red[(w2 * NR + r) * 64 + lane] : 0.0f;
        }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        float sum = part[0][r];
#pragma unroll
        for (int w2 = 1; w2 < 4; ++w2) {
            if (w2 < W) {
                sum += part[w2][r];
            }
        }
        acc[r] = sum;
    }
    return true;
}

// Stores the sums of weight row mm for the tokens of this lane: fp32 partials of this K split, or the final values
// with bias in the reference's order (fp16 output: round the dot first, then add the bias to the stored value).
template <int NR>
__device__ __forceinline__ void mmq_store(const MmqParams &p, int which, int split, size_t mm, size_t n0, int ncols,
                                          const int (&tok)[NR], const float (&acc)[NR]) {
    if (mm >= p.M) {
        return;
    }
    void *out = p.out[which];
    // The bias of this weight row is fetched once, before the stores: a load (and the wait for it) between two stores
    // would also wait for the earlier store, the memory counter being in order.
    const void *bias = p.bias[which];
    const bool has_bias = p.splits == 1 && bias != nullptr;
    float bv = 0.0f;
    if (has_bias) {
        bv = p.bias_is_f16 ? h2f(((const uint16_t *)bias)[mm]) : ((const float *)bias)[mm];
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        if (tok[r] >= ncols) {
            continue;
        }
        const size_t n = n0 + tok[r];
        if (p.splits > 1) {
            ((float *)out)[((size_t)split * p.N + n) * p.M + mm] = acc[r];
        } else if (!p.out_is_f16) {
            ((float *)out)[n * p.M + mm] = has_bias ? acc[r] + bv : acc[r];
        } else if (p.bias_first) {
            ((uint16_t *)out)[n * p.M + mm] = f2h(has_bias ? acc[r] + bv : acc[r]);
        } else {
            uint16_t h = f2h(acc[r]);
            if (has_bias) {
                h = f2h(h2f(h) + bv);
            }
            ((uint16_t *)out)[n * p.M + mm] = h;
        }
    }
}

// ------------------------------------------------------------------ Q4_K x Q8_K
// Work decomposition. All consumer wavefronts of a workgroup work on the SAME 32 weight rows; consumer w walks its own
// contiguous range of blocks, so the workgroup as a whole streams whole weight rows (a decomposition in which a
// workgroup covers many rows and a narrow K range measured 2.7x slower in HBM time for the same bytes). Every consumer
// has a private ring of stages in LDS, filled by direct-to-LDS loads: weights [32 rows][144 B] (9 chunks per row:
// 16-byte reads of consecutive rows fall into different bank groups), activations [tokens][256 B] with the 16-byte
// chunks XOR-swizzled by token, and the activation scales of the block.
//
// The wavefronts of a workgroup are specialised: W consumers only read LDS and run the matrix cores, one loader
// issues every direct-to-LDS load of the workgroup. A wavefront that issues loads is held at the issue stage whenever
// the memory queues of its CU are full, which under a saturated HBM is most of the time; with every wavefront loading
// AND computing, the computation only ran in the gaps (measured with the cycle counter: the load phases and the
// compute phases of a wavefront added up instead of overlapping). Here the loader absorbs those stalls. Steps are
// separated by a bare s_barrier (no implied memory wait): in step t the loader issues block t of every consumer into
// stage t % STAGES and waits until block t - (STAGES - 2) has landed, the consumers work on block t - (STAGES - 1).
//
// NR: live accumulator registers per lane: 4 for up to 8 activation rows (8 rows staged per block), 8 for up to 16
// (token of register r: 8 * (r / 4) + 4 * kh + r % 4, the row layout of the 32x32 MFMA result).
//
// Q5: Q5_K weights. The block is the Q4_K block with 32 bytes of fifth bits between the scales and the nibbles
// (176 bytes = 11 chunks, still an odd number of 16-byte chunks per row); sub-block sb takes bit sb of qh[l]
// (q5k_gguf.c:162-198, vec_dot_impl.h:734-781). Everything else is shared.
template <int NR, int STAGES, bool Q5 = false>
__global__ __launch_bounds__(320) void k_mmq_q4k(const MmqParams p) {
    constexpr int TOK = 2 * NR;
    constexpr int WBYTES = Q5 ? Q5_K_BYTES : Q4_K_BYTES;  // bytes per block
    constexpr int PIECES = WBYTES / 16;                   // 16-byte chunks per block: 9 or 11
    constexpr int QS_OFF = Q5 ? 48 : 16;                  // nibbles behind the header (and the fifth bits)
    constexpr int W_CHUNKS = 32 * PIECES;                 // chunks of one stage of weights: 288 or 352
    constexpr int W_LOADS = (W_CHUNKS + 63) / 64;         // 5 or 6, the last one by the first 32 lanes
    static_assert(W_CHUNKS % 64 == 32, "the last weight load is issued by half a wavefront");
    constexpr int A_OFF = 32 * WBYTES, D_OFF = A_OFF + TOK * QK_K, STAGE = D_OFF + TOK * 4;
    constexpr int A_LOADS = TOK / 4;              // 16-byte chunks of the activation tile / 64 lanes
    constexpr int LOADS = W_LOADS + A_LOADS + 1;  // memory instructions per stage
    constexpr int AHEAD = STAGES - 1;          // blocks the loader runs ahead of the consumers
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = (int)(blockDim.x >> 6) - 1;
    const bool loader = wave == W;
    warm_kernel_arguments<sizeof(MmqParams), sizeof(MmqParams)>();
    const int j = lane & 31, kh = lane >> 5;
    const int split = (int)blockIdx.y / p.nw;
    const int which = (int)blockIdx.y - split * p.nw;
    const uint8_t *wbase = p.w[which];
    size_t n0 = p.n0;
    int ncols = p.ncols;
    if (p.items != nullptr) {
        if ((int)blockIdx.z >= *p.n_items) {
            return;  // uniform for the whole workgroup, before any barrier
        }
        const int4 it = p.items[blockIdx.z];
        wbase += (size_t)it.x * p.expert_stride;
        n0 = (size_t)it.y;
        ncols = it.z;
    } else if (gridDim.z > 1) {
        // dense call with several passes in one launch: blockIdx.z selects the pass of TOK activation rows
        n0 = p.n0 + (size_t)blockIdx.z * TOK;
        const size_t left = p.N - n0;
        ncols = left < (size_t)TOK ? (int)left : TOK;
    }
    const size_t row0 = (size_t)blockIdx.x * 32;
    const int steps = p.bpw + AHEAD;  // the same for every wavefront of the workgroup
    // blocks [b0, b0 + nblk) of consumer w
    auto first_block = [&](int w) { return ((size_t)split * W + w) * p.bpw; };
    auto block_count = [&](int w) {
        const size_t b0 = first_block(w);
        size_t b1 = b0 + p.bpw;
        if (b1 > p.nb) {
            b1 = p.nb;
        }
        return b1 > b0 ? (int)(b1 - b0) : 0;
    };

    float acc[NR];
    int tok[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        acc[r] = 0.0f;
        tok[r] = 8 * (r >> 2) + 4 * kh + (r & 3);
    }

    if (loader) {
        // ---- per-lane source offsets (block-independent)
        uint32_t w_off[W_LOADS];  // weights: chunks of 16 bytes in row order (PIECES per row)
#pragma unroll
        for (int c = 0; c < W_LOADS; ++c) {
            const int chunk = c * 64 + lane;
            int row = chunk / PIECES;
            const int piece = chunk - row * PIECES;
            if (row > 31) {
                row = 31;
            }
            size_t m = row0 + row;
            if (m >= p.M) {
                m = p.M - 1;  // harmless re-read; never stored
            }
            w_off[c] = (uint32_t)((m - row0) * p.nb * WBYTES + 16 * piece);
        }
        const uint8_t *wgroup = wbase + row0 * p.nb * WBYTES;
        uint32_t a_off[A_LOADS];  // activations: chunk (token, slot) holds source chunk slot ^ (token % 16)
#pragma unroll
        for (int c = 0; c < A_LOADS; ++c) {
            const int chunk = c * 64 + lane;
            const int slot = chunk & 15, tk = chunk >> 4;
            const int tt = tk < ncols ? tk : 0;  // rows beyond ncols re-read the first row; never stored
            const size_t arow = p.act_index != nullptr ? (size_t)p.act_index[n0 + tt] : n0 + tt;
            a_off[c] = (uint32_t)(arow * p.kp + 16 * (slot ^ (tk & 15)));
        }
        uint32_t ad_off;
        {
            const int tk = lane & (TOK - 1);
            const int tt = tk < ncols ? tk : 0;
            const size_t arow = p.act_index != nullptr ? (size_t)p.act_index[n0 + tt] : n0 + tt;
            ad_off = (uint32_t)(arow * p.nb);
        }
        for (int t = 0; t < steps; ++t) {
            if (t < p.bpw) {
                for (int w = 0; w < W; ++w) {
                    // a consumer with fewer blocks gets its last block again (never used): the number of loads per
                    // step stays the same for the counted wait below
                    const int nb_w = block_count(w);
                    size_t b = first_block(w) + (t < nb_w ? t : (nb_w > 0 ? nb_w - 1 : 0));
                    if (b >= p.nb) {
                        b = p.nb - 1;
                    }
                    uint8_t *dst = lds + ((size_t)w * STAGES + (t % STAGES)) * STAGE;
#pragma unroll
                    for (int c = 0; c < W_LOADS; ++c) {
                        if (c < W_LOADS - 1 || lane < 32) {  // 288 = 4 * 64 + 32, 352 = 5 * 64 + 32 chunks
                            __builtin_amdgcn_global_load_lds((glb_u8 *)(wgroup + w_off[c] + b * WBYTES),
                                                             (lds_u8 *)(dst + c * 1024), 16, 0, 0);
                        }
                    }
#pragma unroll
                    for (int c = 0; c < A_LOADS; ++c) {
                        __builtin_amdgcn_global_load_lds((glb_u8 *)(p.qs + a_off[c] + b * QK_K),
                                                         (lds_u8 *)(dst + A_OFF + c * 1024), 16, 0, 0);
                    }
                    if (lane < TOK) {
                        __builtin_amdgcn_global_load_lds((glb_u8 *)(p.ad + ad_off + b), (lds_u8 *)(dst + D_OFF), 4, 0,
                                                         0);
                    }
                }
            }
            // loads complete in order: block t - (AHEAD - 1) has landed once at most the loads of the AHEAD - 1 newer
            // steps are outstanding
            const int newer = t < p.bpw ? (AHEAD - 1) : (AHEAD - 1) - (t - p.bpw + 1);
            wait_vmcnt_at_most(newer > 0 ? newer * W * LOADS : 0);
            __builtin_amdgcn_s_barrier();
        }
    } else {
        const int nblk = block_count(wave);
        const uint8_t *ring = lds + (size_t)wave * STAGES * STAGE;
        // MFMA row operand of this lane: token j % TOK (the other rows of the product repeat them and are ignored),
        // chunk 2 * sb + kh of the block, stored at slot chunk ^ token
        const int ti = j & (TOK - 1);
        for (int t = 0; t < steps; ++t) {
            const int blk = t - AHEAD;
            if (blk >= 0 && blk < nblk) {
                const uint8_t *stage = ring + (blk % STAGES) * STAGE;
                const uint8_t *wcur = stage + j * WBYTES;
                const uint8_t *a_blk = stage + A_OFF + ti * QK_K;
                const float *ad_blk = (const float *)(stage + D_OFF);
                const uint4 hdr = *(const uint4 *)wcur;
                uint4 aq[8], wq4[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    wq4[g] = *(const uint4 *)(wcur + QS_OFF + 32 * g + 16 * kh);
                }
                uint4 wqh = make_uint4(0, 0, 0, 0);  // fifth bits of this lane's 16 positions, one bit per sub-block
                if constexpr (Q5) {
                    wqh = *(const uint4 *)(wcur + 16 + 16 * kh);
                }
#pragma unroll
                for (int sb = 0; sb < 8; ++sb) {
                    aq[sb] = *(const uint4 *)(a_blk + 16 * ((2 * sb + kh) ^ (ti & 15)));
                }
                float adr[NR];
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    adr[r] = ad_blk[tok[r] & (TOK - 1)];
                }
                // 6-bit scales and mins as bytes (get_scale_min_k4, kquant_common.h:29-37)
                const float d = h2f((uint16_t)(hdr.x & 0xffffu));
                const float dmin = h2f((uint16_t)(hdr.x >> 16));
                const uint32_t sc_lo = hdr.y & 0x3f3f3f3fu;
                const uint32_t mn_lo = hdr.z & 0x3f3f3f3fu;
                const uint32_t sc_hi = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
                const uint32_t mn_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
                int bsum[NR];
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    bsum[r] = 0;
                }
                auto acts_of = [&](int sb) {
                    return intx4{(int)aq[sb].x, (int)aq[sb].y, (int)aq[sb].z, (int)aq[sb].w};
                };
                auto weights_of = [&](int sb) {
                    const uint4 wq = wq4[sb >> 1];
                    uint4 v;
                    if (sb & 1) {
                        v = make_uint4((wq.x >> 4) & 0x0f0f0f0fu, (wq.y >> 4) & 0x0f0f0f0fu, (wq.z >> 4) & 0x0f0f0f0fu,
                                       (wq.w >> 4) & 0x0f0f0f0fu);
                    } else {
                        v = make_uint4(wq.x & 0x0f0f0f0fu, wq.y & 0x0f0f0f0fu, wq.z & 0x0f0f0f0fu, wq.w & 0x0f0f0f0fu);
                    }
                    if constexpr (Q5) {
                        // bit sb of every byte to bit 4 (sb is a compile-time constant after unrolling)
                        const int sh = 4 - sb;
                        v.x |= (sh >= 0 ? wqh.x << (sh & 31) : wqh.x >> (-sh & 31)) & 0x10101010u;
                        v.y |= (sh >= 0 ? wqh.y << (sh & 31) : wqh.y >> (-sh & 31)) & 0x10101010u;
                        v.z |= (sh >= 0 ? wqh.z << (sh & 31) : wqh.z >> (-sh & 31)) & 0x10101010u;
                        v.w |= (sh >= 0 ? wqh.w << (sh & 31) : wqh.w >> (-sh & 31)) & 0x10101010u;
                    }
                    return intx4{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                };
                const intx16 zero = {0};
                intx16 dm = {0};
                intx16 dq[2];
                dq[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(acts_of(0), weights_of(0), zero, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int sb = 0; sb < 8; ++sb) {
                    const int sc = (int)(((sb < 4 ? sc_lo : sc_hi) >> (8 * (sb & 3))) & 0xffu);
                    // byte sb & 3 of the packed mins in all four bytes (v_perm_b32: one full-rate instruction where
                    // extract + multiply by 0x01010101 would be a quarter-rate multiply)
                    const int mn4 = (int)__builtin_amdgcn_perm(0u, sb < 4 ? mn_lo : mn_hi, 0x01010101u * (sb & 3));
                    dm = __builtin_amdgcn_mfma_i32_32x32x32_i8(acts_of(sb), intx4{mn4, mn4, mn4, mn4}, dm, 0, 0, 0);
                    if (sb < 7) {
                        dq[(sb + 1) & 1] =
                            __builtin_amdgcn_mfma_i32_32x32x32_i8(acts_of(sb + 1), weights_of(sb + 1), zero, 0, 0, 0);
                    }
#pragma unroll
                    for (int r = 0; r < NR; ++r) {
                        bsum[r] += __mul24(dq[sb & 1][r], sc);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    acc[r] += (adr[r] * d) * (float)bsum[r] - (adr[r] * dmin) * (float)dm[r];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this step's LDS reads are done before the stage is reused
            __builtin_amdgcn_s_barrier();
        }
    }

    // ---- K-split within the workgroup: partial sums meet in LDS and are added in wavefront order. The last barrier
    // of the loop guarantees that every stage has been read.
    if (W > 1) {
        if (!mmq_reduce_consumers<NR>((float *)lds, W, wave, lane, !loader, acc)) {
            return;
        }
    } else if (loader) {
        return;
    }
    mmq_store<NR>(p, which, split, row0 + j, n0, ncols, tok, acc);
}

// ------------------------------------------------------------------ Q6_K x Q8_K
// Same decomposition; the differences follow from the format (q6k_gguf.c:63-99, vec_dot_impl.h:783-828):
//   * 16 scale groups of 16 values per block -> 16 MFMAs of K = 16 (v_mfma_i32_32x32x16_i8), signed int8 scales;
//   * weights are 6-bit values minus 32: the MFMA runs on the unsigned values 0..63 and the offset is taken out as
//     32 * sum_is sc_is * (sum of a over group is), which is one more MFMA per group with the scale byte broadcast
//     as the column operand, chained through the accumulator (exact integers, like the CPU's use of bsums);
//   * blocks are 210 bytes and rows only 2-byte aligned, so weights are fetched with unaligned 16-byte register
//     loads (14 pieces per row, the last one overlapping) and written to the LDS stage with a row stride of 240 B.
constexpr int MMQ6_ROWB = 240;                    // LDS bytes per weight row of a stage (15 chunks: conflict-free)
constexpr int MMQ6_WBLK = 32 * MMQ6_ROWB;         // 7680
constexpr int MMQ6_STAGE = MMQ6_WBLK + MMQ_ABLK + MMQ_TOK * 4;

template <int NR>
__global__ __launch_bounds__(512) void k_mmq_q6k(const MmqParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    warm_kernel_arguments<sizeof(MmqParams), sizeof(MmqParams)>();
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = blockDim.x >> 6;
    const int j = lane & 31, kh = lane >> 5;
    const int split = (int)blockIdx.y / p.nw;
    const int which = (int)blockIdx.y - split * p.nw;
    const uint8_t *wbase = p.w[which];
    size_t n0 = p.n0;
    int ncols = p.ncols;
    if (p.items != nullptr) {
        if ((int)blockIdx.z >= *p.n_items) {
            return;
        }
        const int4 it = p.items[blockIdx.z];
        wbase += (size_t)it.x * p.expert_stride;
        n0 = (size_t)it.y;
        ncols = it.z;
    }
    const size_t b0 = ((size_t)split * W + wave) * p.bpw;
    size_t b1 = b0 + p.bpw;
    if (b1 > p.nb) {
        b1 = p.nb;
    }
    const int nblk = b1 > b0 ? (int)(b1 - b0) : 0;
    uint8_t *ring = lds + (size_t)wave * 2 * MMQ6_STAGE;

    const size_t row0 = (size_t)blockIdx.x * 32;
    uint32_t w_off[7], w_lds[7];  // 448 pieces of 16 bytes: 14 per row, piece 13 covers bytes 194..209
#pragma unroll
    for (int c = 0; c < 7; ++c) {
        const int idx = c * 64 + lane;
        const int row = idx / 14, pc = idx - row * 14;
        size_t m = row0 + row;
        if (m >= p.M) {
            m = p.M - 1;  // harmless re-read; never stored
        }
        w_off[c] = (uint32_t)((m - row0) * p.nb * Q6_K_BYTES + (pc < 13 ? 16 * pc : 194));
        w_lds[c] = (uint32_t)(row * MMQ6_ROWB + 16 * pc);
    }
    const uint8_t *wgroup = wbase + row0 * p.nb * Q6_K_BYTES;
    uint32_t a_off[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int chunk = c * 64 + lane;
        const int slot = chunk & 15, tk = chunk >> 4;
        const int tt = tk < ncols ? tk : 0;
        const size_t arow = p.act_index != nullptr ? (size_t)p.act_index[n0 + tt] : n0 + tt;
        a_off[c] = (uint32_t)(arow * p.kp + 16 * (slot ^ tk));
    }
    uint32_t ad_off;
    {
        const int tk = lane & 15;
        const int tt = tk < ncols ? tk : 0;
        const size_t arow = p.act_index != nullptr ? (size_t)p.act_index[n0 + tt] : n0 + tt;
        ad_off = (uint32_t)(arow * p.nb);
    }
    uint4 wreg[7];
    auto fetch_block = [&](size_t b, uint8_t *dst) {
#pragma unroll
        for (int c = 0; c < 7; ++c) {
            uint4 t;
            __builtin_memcpy(&t, wgroup + w_off[c] + b * Q6_K_BYTES, 16);  // unaligned 16-byte load
            wreg[c] = t;
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            __builtin_amdgcn_global_load_lds((glb_u8 *)(p.qs + a_off[c] + b * QK_K),
                                             (lds_u8 *)(dst + MMQ6_WBLK + c * 1024), 16, 0, 0);
        }
        if (lane < MMQ_TOK) {
            __builtin_amdgcn_global_load_lds((glb_u8 *)(p.ad + ad_off + b), (lds_u8 *)(dst + MMQ6_WBLK + MMQ_ABLK), 4,
                                             0, 0);
        }
    };
    auto commit_weights = [&](uint8_t *dst) {
#pragma unroll
        for (int c = 0; c < 7; ++c) {
            *(uint4 *)(dst + w_lds[c]) = wreg[c];
        }
    };
    if (nblk > 0) {
        fetch_block(b0, ring);
        __builtin_amdgcn_s_waitcnt(0);
        commit_weights(ring);
    }

    float acc[NR];
    int tok[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        acc[r] = 0.0f;
        tok[r] = 8 * (r >> 2) + 4 * kh + (r & 3);
    }
    const int ti = j & 15;

    for (int blk = 0; blk < nblk; ++blk) {
        const bool more = blk + 1 < nblk;
        uint8_t *next_stage = ring + ((blk + 1) & 1) * MMQ6_STAGE;
        const uint8_t *stage = ring + (blk & 1) * MMQ6_STAGE;
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the weight rows written by this wavefront are in LDS
        if (more) {
            fetch_block(b0 + blk + 1, next_stage);  // the other stage was last read one block ago
        }
        const uint8_t *wrow = stage + j * MMQ6_ROWB;
        const uint8_t *a_blk = stage + MMQ6_WBLK + ti * QK_K + 8 * kh;
        const float *ad_blk = (const float *)(stage + MMQ6_WBLK + MMQ_ABLK);
        const uint4 scv = *(const uint4 *)(wrow + 192);
        const float d = h2f(*(const uint16_t *)(wrow + 222));
        uint2 ql[2][2][2], qh[2][2];  // [half][second 32][second 16], [half][second 16]: this lane's 8 bytes each
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int s16 = 0; s16 < 2; ++s16) {
                qh[h][s16] = *(const uint2 *)(wrow + 128 + 32 * h + 16 * s16 + 8 * kh);
#pragma unroll
                for (int h32 = 0; h32 < 2; ++h32) {
                    ql[h][h32][s16] = *(const uint2 *)(wrow + 64 * h + 32 * h32 + 16 * s16 + 8 * kh);
                }
            }
        }
        float adr[NR];
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            adr[r] = ad_blk[tok[r]];
        }
        int bsum[NR];
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            bsum[r] = 0;
        }
        const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
        auto acts_of = [&](int is) {
            const uint2 v = *(const uint2 *)(a_blk + 16 * (is ^ ti));
            return (long)(((unsigned long)v.y << 32) | v.x);
        };
        auto weights_of = [&](int is) {
            const int h = is >> 3, q = (is >> 1) & 3, s16 = is & 1;
            const uint2 l = ql[h][q & 1][s16], hh = qh[h][s16];
            uint32_t x = (q >> 1) ? ((l.x >> 4) & 0x0f0f0f0fu) : (l.x & 0x0f0f0f0fu);
            uint32_t y = (q >> 1) ? ((l.y >> 4) & 0x0f0f0f0fu) : (l.y & 0x0f0f0f0fu);
            x |= ((hh.x >> (2 * q)) & 0x03030303u) << 4;
            y |= ((hh.y >> (2 * q)) & 0x03030303u) << 4;
            return (long)(((unsigned long)y << 32) | x);
        };
        const intx16 zero = {0};
        intx16 ds = {0};
        intx16 dq[2];
        long av[2];
        av[0] = acts_of(0);
        dq[0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[0], weights_of(0), zero, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int is = 0; is < 16; ++is) {
            const uint32_t scb = (scw[is >> 2] >> (8 * (is & 3))) & 0xffu;
            const int sc = (int)(int8_t)scb;
            const uint32_t sc4 = __builtin_amdgcn_perm(0u, scw[is >> 2], 0x01010101u * (is & 3));  // byte broadcast
            ds = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[is & 1], (long)(((unsigned long)sc4 << 32) | sc4), ds, 0, 0, 0);
            if (is < 15) {
                av[(is + 1) & 1] = acts_of(is + 1);
                dq[(is + 1) & 1] =
                    __builtin_amdgcn_mfma_i32_32x32x16_i8(av[(is + 1) & 1], weights_of(is + 1), zero, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                bsum[r] += __mul24(dq[is & 1][r], sc);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            acc[r] += (adr[r] * d) * (float)(bsum[r] - 32 * ds[r]);
        }
        if (more) {
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the next block's weights and activations have landed
            commit_weights(next_stage);
        }
    }

    if (W > 1) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        float *red = (float *)lds;
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            red[(wave * NR + r) * 64 + lane] = acc[r];
        }
        __syncthreads();
        if (wave != 0) {
            return;
        }
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            float sum = red[r * 64 + lane];
            for (int w2 = 1; w2 < W; ++w2) {
                sum += red[(w2 * NR + r) * 64 + lane];
            }
            acc[r] = sum;
        }
    }
    mmq_store<NR>(p, which, split, row0 + j, n0, ncols, tok, acc);
}

// ------------------------------------------------------------------ Q6_K x Q8_K, loader / consumer wavefronts
// For rows of a multiple of 8 blocks (K a multiple of 2048) a weight row is 16-byte aligned and the loader can copy
// with direct-to-LDS loads like the Q4_K kernel. A block starts at byte 210 * b of its row, i.e. o = (2 * b) % 16
// bytes into a 16-byte chunk: the stage holds, for each of the 32 rows, the 15 chunks from the one that contains the
// block start (stride 240 B as above; the 15th chunk is never needed and is not loaded), and the consumers read the
// block at offset o inside the row slot, relying on unaligned LDS reads. Same arithmetic and MFMA sequence as
// k_mmq_q6k, same step protocol as k_mmq_q4k.
template <int NR, int STAGES>
__global__ __launch_bounds__(320) void k_mmq_q6k_ls(const MmqParams p) {
    constexpr int TOK = 2 * NR;
    constexpr int A_OFF = MMQ6_WBLK, D_OFF = A_OFF + TOK * QK_K, STAGE = D_OFF + TOK * 4;
    constexpr int W_LOADS = 8;                 // 32 rows x 15 chunk slots = 480 lanes of 16 bytes
    constexpr int A_LOADS = TOK / 4;
    constexpr int LOADS = W_LOADS + A_LOADS + 1;
    constexpr int AHEAD = STAGES - 1;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    warm_kernel_arguments<sizeof(MmqParams), sizeof(MmqParams)>();
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, W = (int)(blockDim.x >> 6) - 1;
    const bool loader = wave == W;
    const int j = lane & 31, kh = lane >> 5;
    const int split = (int)blockIdx.y / p.nw;
    const int which = (int)blockIdx.y - split * p.nw;
    const uint8_t *wbase = p.w[which];
    size_t n0 = p.n0;
    int ncols = p.ncols;
    if (p.items != nullptr) {
        if ((int)blockIdx.z >= *p.n_items) {
            return;  // uniform for the whole workgroup, before any barrier
        }
        const int4 it = p.items[blockIdx.z];
        wbase += (size_t)it.x * p.expert_stride;
        n0 = (size_t)it.y;
        ncols = it.z;
    } else if (gridDim.z > 1) {
        // dense call with several passes in one launch: blockIdx.z selects the pass of TOK activation rows
        n0 = p.n0 + (size_t)blockIdx.z * TOK;
        const size_t left = p.N - n0;
        ncols = left < (size_t)TOK ? (int)left : TOK;
    }
    const size_t row0 = (size_t)blockIdx.x * 32;
    const int steps = p.bpw + AHEAD;
    auto first_block = [&](int w) { return ((size_t)split * W + w) * p.bpw; };
    auto block_count = [&](int w) {
        const size_t b0 = first_block(w);
        size_t b1 = b0 + p.bpw;
        if (b1 > p.nb) {
            b1 = p.nb;
        }
        return b1 > b0 ? (int)(b1 - b0) : 0;
    };

    float acc[NR];
    int tok[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        acc[r] = 0.0f;
        tok[r] = 8 * (r >> 2) + 4 * kh + (r & 3);
    }

    const size_t row_bytes = p.nb * Q6_K_BYTES;
    const uint32_t lead = (uint32_t)((row0 * row_bytes) & 15);
    if (loader) {
        // Rows need not start on 16-byte boundaries (they do only when a row is a multiple of 8 blocks): every row's 14
        // chunks start at ITS OWN boundary below the block start; the group's first row is addressed from the boundary
        // below it (`lead` bytes before it).
        uint32_t w_row[W_LOADS], w_pc[W_LOADS];
        bool w_on[W_LOADS];
#pragma unroll
        for (int c = 0; c < W_LOADS; ++c) {
            const int idx = c * 64 + lane;
            const int row = idx / 15, pc = idx - row * 15;
            size_t m = row0 + (row < 32 ? row : 31);
            if (m >= p.M) {
                m = p.M - 1;  // harmless re-read; never stored
            }
            w_row[c] = lead + (uint32_t)((m - row0) * row_bytes);
            w_pc[c] = (uint32_t)(16 * pc);
            w_on[c] = row < 32 && pc < 14;
        }
        const uint8_t *wgroup = wbase + ((row0 * row_bytes) & ~(size_t)15);
        // the tensor's end from wgroup: a chunk that would end behind it (the tensor's size need not be a multiple of
        // 16) comes two bytes at a time through registers, and the loads in flight are then not whole steps
        const size_t w_end64 = (size_t)lead + (p.M - row0) * row_bytes;
        const uint32_t w_end = w_end64 > 0xffffffffull ? 0xffffffffu : (uint32_t)w_end64;
        const bool ragged_end = row0 + 32 >= p.M && (w_end & 15u) != 0;
        uint32_t a_off[A_LOADS];
#pragma unroll
        for (int c = 0; c < A_LOADS; ++c) {
            const int chunk = c * 64 + lane;
            const int slot = chunk & 15, tk = chunk >> 4;
            const int tt = tk < ncols ? tk : 0;
            const size_t arow = p.act_index != nullptr ? (size_t)p.act_index[n0 + tt] : n0 + tt;
            a_off[c] = (uint32_t)(arow * p.kp + 16 * (slot ^ (tk & 15)));
        }
        uint32_t ad_off;
        {
            const int tk = lane & (TOK - 1);
            const int tt = tk < ncols ? tk : 0;
            const size_t arow = p.act_index != nullptr ? (size_t)p.act_index[n0 + tt] : n0 + tt;
            ad_off = (uint32_t)(arow * p.nb);
        }
        for (int t = 0; t < steps; ++t) {
            if (t < p.bpw) {
                for (int w = 0; w < W; ++w) {
                    const int nb_w = block_count(w);
                    size_t b = first_block(w) + (t < nb_w ? t : (nb_w > 0 ? nb_w - 1 : 0));
                    if (b >= p.nb) {
                        b = p.nb - 1;
                    }
                    const uint32_t boff = (uint32_t)(b * Q6_K_BYTES);
                    uint8_t *dst = lds + ((size_t)w * STAGES + (t % STAGES)) * STAGE;
#pragma unroll
                    for (int c = 0; c < W_LOADS; ++c) {
                        const uint32_t voff = ((w_row[c] + boff) & ~15u) + w_pc[c];  // from the chunk with the block start
                        const bool past = voff + 16u > w_end;
                        if (w_on[c] && !past) {
                            __builtin_amdgcn_global_load_lds((glb_u8 *)(wgroup + voff), (lds_u8 *)(dst + c * 1024), 16, 0,
                                                             0);
                        }
                        if (w_on[c] && past) {
                            for (uint32_t e = 0; e < 16u && voff + e < w_end; e += 2u) {
                                *(uint16_t *)(dst + c * 1024 + 16 * lane + e) = *(const uint16_t *)(wgroup + voff + e);
                            }
                        }
                    }
#pragma unroll
                    for (int c = 0; c < A_LOADS; ++c) {
                        __builtin_amdgcn_global_load_lds((glb_u8 *)(p.qs + a_off[c] + b * QK_K),
                                                         (lds_u8 *)(dst + A_OFF + c * 1024), 16, 0, 0);
                    }
                    if (lane < TOK) {
                        __builtin_amdgcn_global_load_lds((glb_u8 *)(p.ad + ad_off + b), (lds_u8 *)(dst + D_OFF), 4, 0,
                                                         0);
                    }
                }
            }
            const int newer = t < p.bpw ? (AHEAD - 1) : (AHEAD - 1) - (t - p.bpw + 1);
            wait_vmcnt_at_most(newer > 0 && !ragged_end ? newer * W * LOADS : 0);
            __builtin_amdgcn_s_waitcnt(0xc07f);  // the LDS stores of a tensor-end chunk
            __builtin_amdgcn_s_barrier();
        }
    } else {
        const int nblk = block_count(wave);
        const size_t b_first = first_block(wave);
        const uint8_t *ring = lds + (size_t)wave * STAGES * STAGE;
        const int ti = j & (TOK - 1);
        uint32_t w_own;  // byte offset of this lane's weight row from the group's 16-byte boundary (the clamped row)
        {
            size_t m = row0 + (size_t)j;
            if (m >= p.M) {
                m = p.M - 1;
            }
            w_own = lead + (uint32_t)((m - row0) * row_bytes);
        }
        for (int t = 0; t < steps; ++t) {
            const int blk = t - AHEAD;
            if (blk >= 0 && blk < nblk) {
                const uint8_t *stage = ring + (blk % STAGES) * STAGE;
                const uint32_t o = (w_own + (uint32_t)((b_first + blk) * Q6_K_BYTES)) & 15u;  // this lane's row
                const uint8_t *wrow = stage + j * MMQ6_ROWB + o;
                const uint8_t *a_blk = stage + A_OFF + ti * QK_K + 8 * kh;
                const float *ad_blk = (const float *)(stage + D_OFF);
                uint4 scv;
                __builtin_memcpy(&scv, wrow + 192, 16);
                uint16_t dh;
                __builtin_memcpy(&dh, wrow + 208, 2);
                const float d = h2f(dh);
                uint2 ql[2][2][2], qh[2][2];  // [half][second 32][second 16], [half][second 16]: this lane's 8 bytes each
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int s16 = 0; s16 < 2; ++s16) {
                        __builtin_memcpy(&qh[h][s16], wrow + 128 + 32 * h + 16 * s16 + 8 * kh, 8);
#pragma unroll
                        for (int h32 = 0; h32 < 2; ++h32) {
                            __builtin_memcpy(&ql[h][h32][s16], wrow + 64 * h + 32 * h32 + 16 * s16 + 8 * kh, 8);
                        }
                    }
                }
                float adr[NR];
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    adr[r] = ad_blk[tok[r] & (TOK - 1)];
                }
                int bsum[NR];
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    bsum[r] = 0;
                }
                const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
                auto acts_of = [&](int is) {
                    const uint2 v = *(const uint2 *)(a_blk + 16 * (is ^ (ti & 15)));
                    return (long)(((unsigned long)v.y << 32) | v.x);
                };
                auto weights_of = [&](int is) {
                    const int h = is >> 3, q = (is >> 1) & 3, s16 = is & 1;
                    const uint2 l = ql[h][q & 1][s16], hh = qh[h][s16];
                    uint32_t x = (q >> 1) ? ((l.x >> 4) & 0x0f0f0f0fu) : (l.x & 0x0f0f0f0fu);
                    uint32_t y = (q >> 1) ? ((l.y >> 4) & 0x0f0f0f0fu) : (l.y & 0x0f0f0f0fu);
                    x |= ((hh.x >> (2 * q)) & 0x03030303u) << 4;
                    y |= ((hh.y >> (2 * q)) & 0x03030303u) << 4;
                    return (long)(((unsigned long)y << 32) | x);
                };
                const intx16 zero = {0};
                intx16 ds = {0};
                intx16 dq[2];
                long av[2];
                av[0] = acts_of(0);
                dq[0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[0], weights_of(0), zero, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int is = 0; is < 16; ++is) {
                    const uint32_t scb = (scw[is >> 2] >> (8 * (is & 3))) & 0xffu;
                    const int sc = (int)(int8_t)scb;
                    const uint32_t sc4 = __builtin_amdgcn_perm(0u, scw[is >> 2], 0x01010101u * (is & 3));  // byte broadcast
                    ds = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[is & 1], (long)(((unsigned long)sc4 << 32) | sc4), ds,
                                                               0, 0, 0);
                    if (is < 15) {
                        av[(is + 1) & 1] = acts_of(is + 1);
                        dq[(is + 1) & 1] = __builtin_amdgcn_mfma_i32_32x32x16_i8(av[(is + 1) & 1], weights_of(is + 1),
                                                                                 zero, 0, 0, 0);
                    }
#pragma unroll
                    for (int r = 0; r < NR; ++r) {
                        bsum[r] += __mul24(dq[is & 1][r], sc);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    acc[r] += (adr[r] * d) * (float)(bsum[r] - 32 * ds[r]);
                }
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this step's LDS reads are done before the stage is reused
            __builtin_amdgcn_s_barrier();
        }
    }

    if (W > 1) {
        if (!mmq_reduce_consumers<NR>((float *)lds, W, wave, lane, !loader, acc)) {
            return;
        }
    } else if (loader) {
        return;
    }
    mmq_store<NR>(p, which, split, row0 + j, n0, ncols, tok, acc);
}

// Q4_K and Q5_K share one kernel and one launch plan
static bool mmq_is_q4k_family(int kind) {
    return kind == MARMOT_HIP_KIND_Q4_K || kind == MARMOT_HIP_KIND_Q5_K;
}

bool mmq_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, int weights) {
    if (dev->knobs.no_mmq) {
        return false;
    }
    // below these row counts the fused-quantization matvec is faster (no separate quantization pass)
    // (a Q6_K set of three weights crosses over earlier: the matvec streams every weight per column tile)
    const size_t q6_set_min = 3;
    const size_t min_rows = mmq_is_q4k_family(kind) ? 3 : (weights >= 3 ? q6_set_min : 5);
    return (mmq_is_q4k_family(kind) || kind == MARMOT_HIP_KIND_Q6_K) && N >= min_rows && K % QK_K == 0;
}

constexpr size_t MMQ_ROWS_PER_PASS = MMQ_TOK;

struct MmqPlan {
    int W, S, bpw;
};

// the loader / consumer kernel takes rows of any number of blocks (it rounds the 16-byte loads down per row)
static bool mmq6_uses_loader(size_t nb) {
    return nb != 0;
}

// W (consumer) wavefronts per workgroup and S workgroups split K.
//   * Many row groups (M / 32 >= CUs), Q4_K: the consumers of one workgroup split K (no partials); with more than 8
//     activation rows 16 rows are staged per block and two consumers keep the LDS ring small enough for three
//     workgroups per CU.
//   * Few row groups, and Q6_K with the loader (its stages are larger): one consumer per workgroup and K split over
//     about 4 (Q6_K: 3.5) workgroups per CU, which overlap each other's load and compute phases; the partials meet
//     in the reduction kernel. Measured per shape; e.g. Q4_K 4096 x 14336 N=8: 19.1 -> 18.0 us, Q6_K 14336 x 4096
//     N=8: 34.0 -> 28.4 us.
static MmqPlan mmq_plan(const marmot_hip_device *dev, int kind, size_t N, size_t M, size_t nb, int weights) {
    // row groups of the whole launch: the weights of a set (gate/up, q/k/v) are one grid
    const bool q6_loader = kind == MARMOT_HIP_KIND_Q6_K && mmq6_uses_loader(nb);
    // beyond 32 activation rows the 32-row passes of the loader / consumer kernels run as one launch: its workgroups
    // count like row groups (4096 x 4096, N = 512: 85.5 us with the K split chosen for one pass, 64.7 us without)
    const size_t passes = (N > 32 && (mmq_is_q4k_family(kind) || q6_loader)) ? (N + 31) / 32 : 1;
    const size_t rg = ((M + 31) / 32) * (size_t)(weights > 0 ? weights : 1) * passes;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    MmqPlan pl;
    size_t W, S = 1;
    if (passes > 1 && rg >= cus) {
        // several passes in one launch fill the chip by themselves: one consumer walks the whole row, which keeps
        // the LDS ring small (four workgroups per CU) and needs no partial sums
        W = 1;
    } else if (q6_loader && weights > 1 && rg >= cus) {
        // a set of weights that fills the chip by itself: two consumers per workgroup and no K split, so that no
        // reduction launch per weight follows (q/k/v 3 x 4096 x 4096, N=16: 41.3 us with the rule below, 33.6 with
        // two workgroups along K, 32.2 with this)
        W = nb < 2 ? nb : 2;
    } else if (q6_loader || (mmq_is_q4k_family(kind) && rg < cus)) {
        W = 1;
        const size_t want = ((q6_loader ? 7 : 8) * cus / 2 + rg - 1) / rg;  // workgroups along K
        while (S < want && S * 8 <= nb) {
            S *= 2;
        }
    } else {
        const size_t w_max = (mmq_is_q4k_family(kind) && N > 8) ? 2 : 4;
        W = nb < w_max ? nb : w_max;
        while (rg * S < cus && W * S * 2 <= nb) {
            S *= 2;
        }
    }
    const size_t bpw = (nb + W * S - 1) / (W * S);
    pl.W = (int)W;
    pl.S = (int)((nb + bpw * W - 1) / (bpw * W));
    pl.bpw = (int)bpw;
    return pl;
}

// bytes of fp32 partials launch_mmq needs for this shape (0 when K is not split across workgroups)
size_t mmq_scratch_bytes(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M, int weights) {
    const MmqPlan pl = mmq_plan(dev, kind, N, M, K / QK_K, weights);
    const size_t passes = pl.S > 1 ? (size_t)pl.S * N * M * sizeof(float) * (size_t)weights : 0;
    // the tiled GEMM may take the call instead (decided at launch, when the operands' alignment is known)
    const size_t tiled = ((mmq_is_q4k_family(kind) || kind == MARMOT_HIP_KIND_Q6_K) && !dev->knobs.no_gemm_i8)
        ? gemm_i8_scratch_bytes(dev, N, K, M, weights) : 0;
    return passes > tiled ? passes : tiled;
}

static size_t mmq6_lds_bytes(int W) {
    const size_t ring = (size_t)W * MMQ_STAGES * MMQ6_STAGE;
    const size_t red = (size_t)W * 8 * 64 * sizeof(float);
    return ring > red ? ring : red;
}

// the Q6_K loader / consumer kernel copies 16-byte chunks: rows, bases and expert strides must be 16-byte aligned
static bool mmq6_loader_applies(const MmqParams &p, const MmqPlan &pl) {
    return mmq6_uses_loader(p.nb) && pl.W <= 4 && (((uintptr_t)p.w[0]) & 15) == 0 && (((uintptr_t)p.w[1]) & 15) == 0 &&
           (((uintptr_t)p.w[2]) & 15) == 0 && (p.expert_stride & 15) == 0;
}

template <int NR>
static int mmq_launch_q6k_ls(marmot_hip_device *dev, const MmqParams &p, const MmqPlan &pl, const dim3 grid) {
    // two stages for the grouped call and for several passes in one launch: many workgroups per CU overlap each other,
    // and five of them fit instead of three (4096 x 4096 at 512 rows: 133.6 -> 116.2 us)
    const int stages = (p.items != nullptr || grid.z > 1) ? 2 : 3;
    const size_t stage = MMQ6_WBLK + 2 * NR * QK_K + 2 * NR * 4;
    const size_t ring = (size_t)pl.W * stages * stage;
    const size_t red = (size_t)pl.W * NR * 64 * sizeof(float);
    const dim3 block((pl.W + 1) * 64);
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_q6k_ls<NR, 2>));
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_q6k_ls<NR, 3>));
    if (stages == 2) {
        hipLaunchKernelGGL((k_mmq_q6k_ls<NR, 2>), grid, block, ring > red ? ring : red, dev->stream, p);
    } else {
        hipLaunchKernelGGL((k_mmq_q6k_ls<NR, 3>), grid, block, ring > red ? ring : red, dev->stream, p);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

template <int NR>
static int mmq_launch_any(marmot_hip_device *dev, int kind, const MmqParams &p, const MmqPlan &pl, const dim3 grid);
template <int NR>
static int mmq_launch_q4k(marmot_hip_device *dev, int kind, const MmqParams &p, const MmqPlan &pl, const dim3 grid);

template <int NR>
static int mmq_launch(marmot_hip_device *dev, int kind, const MmqParams &p, const MmqPlan &pl, size_t M,
                      unsigned items) {
    const dim3 grid((unsigned)((M + 31) / 32), (unsigned)(pl.S * p.nw), items);
    if constexpr (NR > 8) {
        // 32 activation rows per pass: the loader / consumer kernels are built for it
        if (mmq_is_q4k_family(kind)) {
            return mmq_launch_q4k<NR>(dev, kind, p, pl, grid);
        }
        if (kind == MARMOT_HIP_KIND_Q6_K && mmq6_loader_applies(p, pl)) {
            return mmq_launch_q6k_ls<NR>(dev, p, pl, grid);
        }
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "mmq: no 32-row pass for this kind or alignment");
    } else {
        return mmq_launch_any<NR>(dev, kind, p, pl, grid);
    }
}

template <int NR>
static int mmq_launch_any(marmot_hip_device *dev, int kind, const MmqParams &p, const MmqPlan &pl, const dim3 grid) {
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_q6k<NR>));
    if (kind == MARMOT_HIP_KIND_Q6_K && mmq6_loader_applies(p, pl)) {
        return mmq_launch_q6k_ls<NR>(dev, p, pl, grid);
    } else if (kind == MARMOT_HIP_KIND_Q6_K) {
        hipLaunchKernelGGL((k_mmq_q6k<NR>), grid, dim3(pl.W * 64), mmq6_lds_bytes(pl.W), dev->stream, p);
    } else {
        return mmq_launch_q4k<NR>(dev, kind, p, pl, grid);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

// Q4_K / Q5_K: W consumers + 1 loader. Three stages (the loader two blocks ahead) for the dense call; the grouped call
// runs many small workgroups per CU, which overlap each other, and takes two to fit more of them.
template <int NR>
static int mmq_launch_q4k(marmot_hip_device *dev, int kind, const MmqParams &p, const MmqPlan &pl, const dim3 grid) {
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_q4k<NR, 2>));
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_q4k<NR, 3>));
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_q4k<NR, 2, true>));
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_q4k<NR, 3, true>));
    {
        if (pl.W < 1 || pl.W > 4) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "mmq: %d consumer wavefronts are not supported", pl.W);
        }
        const bool q5 = kind == MARMOT_HIP_KIND_Q5_K;
        // Q5_K with 32-row passes: three stages of two consumers would take 84 KB and leave one workgroup per CU
        const int stages = (p.items != nullptr || (q5 && NR > 8)) ? 2 : 3;
        const size_t stage = 32 * (size_t)(q5 ? Q5_K_BYTES : Q4_K_BYTES) + 2 * NR * QK_K + 2 * NR * 4;
        const size_t ring = (size_t)pl.W * stages * stage;
        const size_t red = (size_t)pl.W * NR * 64 * sizeof(float);
        const size_t lds_bytes = ring > red ? ring : red;
        const dim3 block((pl.W + 1) * 64);
        if (stages == 2) {
            if (q5) {
                hipLaunchKernelGGL((k_mmq_q4k<NR, 2, true>), grid, block, lds_bytes, dev->stream, p);
            } else {
                hipLaunchKernelGGL((k_mmq_q4k<NR, 2>), grid, block, lds_bytes, dev->stream, p);
            }
        } else if (q5) {
            hipLaunchKernelGGL((k_mmq_q4k<NR, 3, true>), grid, block, lds_bytes, dev->stream, p);
        } else {
            hipLaunchKernelGGL((k_mmq_q4k<NR, 3>), grid, block, lds_bytes, dev->stream, p);
        }
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

// Dense: N activation rows in passes of up to 32. scratch: mmq_scratch_bytes() bytes, or nullptr to take them from
// the device workspace (only when the activations do not live there).
int launch_mmq(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, const ActScratch &act, size_t N,
               size_t K, size_t M, const void *d_bias, int bias_dtype, void *d_out0, void *d_out1, int out_dtype,
               void *scratch) {
    WeightSet ws;
    ws.count = d_w1 != nullptr ? 2 : 1;
    ws.w[0] = d_w0;
    ws.w[1] = d_w1;
    ws.out[0] = d_out0;
    ws.out[1] = d_out1;
    ws.bias[0] = d_bias;
    ws.bias[1] = d_bias;
    ws.bias_dtype = bias_dtype;
    return launch_mmq_set(dev, kind, ws, act, N, K, M, out_dtype, scratch);
}

int launch_mmq_set(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                   size_t M, int out_dtype, void *scratch) {
    if (!mmq_supported(dev, kind, N, K, ws.count)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "small-batch MFMA matmul: unsupported kind or shape");
    }
    if (gemm_i8_applies(dev, kind, N, K, ws.w, ws.count, act)) {
        return launch_gemm_i8(dev, kind, ws, act, N, K, M, out_dtype, scratch);
    }
    const size_t nb = K / QK_K;
    const MmqPlan pl = mmq_plan(dev, kind, N, M, nb, ws.count);
    float *partial = (float *)scratch;
    if (pl.S > 1 && partial == nullptr) {
        void *wsp = nullptr;
        int st = workspace_reserve(dev, mmq_scratch_bytes(dev, kind, N, K, M, ws.count), &wsp);
        if (st != MARMOT_HIP_SUCCESS) {
            return st;
        }
        partial = (float *)wsp;
    }
    MmqParams p;
    p.nw = ws.count;
    for (int i = 0; i < 3; ++i) {  // unused slots repeat weight 0 (the alignment checks look at all three)
        const int src = i < ws.count ? i : 0;
        p.w[i] = (const uint8_t *)ws.w[src];
        p.out[i] = pl.S > 1 ? (void *)(partial + (size_t)src * pl.S * N * M) : ws.out[src];
        p.bias[i] = ws.bias[src];
    }
    p.qs = act.qs;
    p.ad = act.d;
    p.kp = act.kp;
    p.N = N;
    p.M = M;
    p.nb = nb;
    p.bpw = pl.bpw;
    p.splits = pl.S;
    p.bias_is_f16 = ws.bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.bias_first = ws.bias_first ? 1 : 0;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.items = nullptr;
    p.n_items = nullptr;
    p.act_index = nullptr;
    p.expert_stride = 0;
    // 16 activation rows per pass (8 live accumulator registers per lane). The loader / consumer kernels (Q4_K, Q5_K,
    // Q6_K with 16-byte aligned rows) from 17 rows on: 32 rows per pass, which uses all 32 rows of the matrix-core product instead of half of them and halves the number of
    // passes over the weights.
    const bool wide_ok = mmq_is_q4k_family(kind) || (kind == MARMOT_HIP_KIND_Q6_K && mmq6_loader_applies(p, pl));
    const size_t wide_from = 17;  // more than one 16-row pass: one 32-row pass streams the weights once instead of twice
    const size_t rows_per_pass = (wide_ok && N >= wide_from) ? 32 : MMQ_ROWS_PER_PASS;
    if (rows_per_pass == 32 && N > 32) {
        // all passes in one launch (grid z): no launch gap, ramp and tail per pass
        p.n0 = 0;
        p.ncols = 32;
        const int st = mmq_launch<16>(dev, kind, p, pl, M, (unsigned)((N + 31) / 32));
        if (st != MARMOT_HIP_SUCCESS) {
            return st;
        }
    } else {
        for (size_t n0 = 0; n0 < N; n0 += rows_per_pass) {
            p.n0 = n0;
            p.ncols = (int)(N - n0 < rows_per_pass ? N - n0 : rows_per_pass);
            const int st = p.ncols <= 8    ? mmq_launch<4>(dev, kind, p, pl, M, 1)
                           : p.ncols <= 16 ? mmq_launch<8>(dev, kind, p, pl, M, 1)
                                           : mmq_launch<16>(dev, kind, p, pl, M, 1);
            if (st != MARMOT_HIP_SUCCESS) {
                return st;
            }
        }
    }
    if (pl.S > 1) {
        for (int which = 0; which < ws.count; ++which) {
            int st = launch_splitk_reduce(dev, partial + (size_t)which * pl.S * N * M, pl.S, N, M, ws.bias[which],
                                          ws.bias_dtype, ws.out[which], out_dtype, ws.bias_first);
            if (st != MARMOT_HIP_SUCCESS) {
                return st;
            }
        }
    }
    set_route(kind == MARMOT_HIP_KIND_Q6_K       ? "mmq_q6_k_q8_k_mfma"
              : kind == MARMOT_HIP_KIND_Q5_K     ? "mmq_q5_k_q8_k_mfma"
                                                 : "mmq_q4_k_q8_k_mfma");
    return MARMOT_HIP_SUCCESS;
}

// Grouped (MoE): every work item is up to 8 consecutive routes of one expert; blockIdx.z walks the item list the
// route kernel wrote (workgroups beyond *d_n_items exit at once).
bool mmq_grouped_supported(const marmot_hip_device *dev, int kind, size_t K) {
    return (mmq_is_q4k_family(kind) || kind == MARMOT_HIP_KIND_Q6_K) && K % QK_K == 0 && !dev->knobs.no_mmq;
}

int launch_mmq_grouped(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, size_t expert_stride,
                       const ActScratch &act, const uint32_t *d_act_index, const int4 *d_items, const int *d_n_items,
                       size_t max_items, size_t K, size_t M, void *d_out0, void *d_out1, int item_cols) {
    if (max_items == 0 || M == 0 || K == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    if (!mmq_grouped_supported(dev, kind, K)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "grouped MFMA matmul: unsupported kind or shape");
    }
    if (max_items > 65535) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "grouped MFMA matmul: %zu work items exceed the grid limit",
                         max_items);
    }
    const size_t nb = K / QK_K;
    MmqPlan pl;
    // one consumer per workgroup walks the whole row: expert matrices are small and there are thousands of
    // workgroups, which overlap each other's load and compute phases (2 or 4 consumers measured slower)
    pl.W = 1;
    pl.S = 1;
    pl.bpw = (int)nb;
    MmqParams p;
    p.nw = d_w1 != nullptr ? 2 : 1;
    p.w[0] = (const uint8_t *)d_w0;
    p.w[1] = (const uint8_t *)(d_w1 != nullptr ? d_w1 : d_w0);
    p.w[2] = p.w[0];
    p.out[0] = d_out0;
    p.out[1] = d_out1 != nullptr ? d_out1 : d_out0;
    p.out[2] = p.out[0];
    p.qs = act.qs;
    p.ad = act.d;
    p.kp = act.kp;
    p.N = 0;
    p.M = M;
    p.nb = nb;
    p.n0 = 0;
    p.ncols = 0;
    p.bpw = pl.bpw;
    p.splits = 1;
    p.bias[0] = p.bias[1] = p.bias[2] = nullptr;
    p.bias_is_f16 = 0;
    p.bias_first = 0;
    p.out_is_f16 = 0;
    p.items = d_items;
    p.n_items = d_n_items;
    p.act_index = d_act_index;
    p.expert_stride = expert_stride;
    // work items of up to 8, 16 or 32 routes (the caller cut them to match)
    const int st = item_cols <= 8    ? mmq_launch<4>(dev, kind, p, pl, M, (unsigned)max_items)
                   : item_cols <= 16 ? mmq_launch<8>(dev, kind, p, pl, M, (unsigned)max_items)
                                     : mmq_launch<16>(dev, kind, p, pl, M, (unsigned)max_items);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    set_route(kind == MARMOT_HIP_KIND_Q6_K       ? "moe_grouped_q6_k_q8_k_mfma"
              : kind == MARMOT_HIP_KIND_Q5_K     ? "moe_grouped_q5_k_q8_k_mfma"
                                                 : "moe_grouped_q4_k_q8_k_mfma");
    return MARMOT_HIP_SUCCESS;
}

} // namespace mh

// Small-batch Q4_K matmul (3..16 fp32 activation rows), "row-owning" form on the int8 matrix cores: the launch shape
// of the decode matvec of mh_matvec_rows.hip (ONE workgroup per compute unit that owns a contiguous share of the weight
// rows, loader wavefronts feeding an LDS ring, no barrier per step) with the arithmetic of the small-batch kernel of
// mh_mmq.hip (v_mfma on int8, per-lane 6-bit scales).
//   * The activations are quantized to Q8_K once per WORKGROUP, inside the kernel, into LDS: no quantization launch in
//     front of the matmul, and 256 workgroups repeat the work instead of one workgroup per 32 weight rows. They are
//     stored in the operand order of the 16x16x32 matrix instruction ([block][sub-block][8-byte k group][token]), so a
//     wavefront reads the operand of one sub-block as 512 contiguous bytes.
//   * A task is one group of up to 16 weight rows x an ODD number of 256-value blocks, laid out in its ring slot as
//     [row][blocks x 144 B]: every row's segment is one contiguous run in memory, and with an odd number of 16-byte
//     chunks per row the reads of 16 consecutive rows fall into different banks. A consumer
//     wavefront multiplies the 16 rows by all tokens: tokens are the row operand, weight rows the column operand, so
//     lane l ends up with weight row l % 16 x tokens 4 (l / 16) .. + 3 and applies ITS row's 6-bit scale with one
//     integer multiply-add per token. The min term sum_j mn_j * (sum of a over sub-block j) is a second matrix
//     instruction per sub-block with the min byte broadcast as the column operand, chained through its accumulator.
//   * Consumers that share a row group split K between them (each walks a contiguous range of blocks, fp32 sum in
//     block order); their partial sums meet in LDS and the wavefront that arrives last adds them in K order and
//     stores. No partial sums in memory, no reduction kernel.
// Integer results are exact; the arithmetic per block is cpu_vec_dot_q4_k_q8_k (vec_dot_impl.h:689-732) on activations
// packed like cpu_matmul_quant_pack_q8_k_f32 (matmul_quant_pack.c:106-142). Only the order of the fp32 sum over blocks
// differs from the CPU (per K part sequential, then across parts in a fixed order).
#include "mh_rows.h"

namespace mh {

typedef int mr_intx4 __attribute__((ext_vector_type(4)));

constexpr int MR_IPT_MAX = 9;  // load instructions (1 KiB each) per task at most

struct MmqRowsParams {
    const uint8_t *w[3];  // weights of one shape sharing the activations; blockIdx.y selects one
    void *out[3];
    const void *bias[3];
    const float *x;        // fp32 activations [N][K] (quantized inside the kernel), or
    const int8_t *pq;      // packed activations: int8 rows of kp bytes,
    const float *pd;       //   block scales [row][nb]
    uint32_t kp;
    uint32_t K, M, N;
    uint32_t nb;             // blocks per weight row
    uint32_t row_bytes;
    uint32_t total_bytes;    // M * row_bytes
    uint32_t rows_per_wg;    // a multiple of R
    uint32_t R;              // weight rows per row group (<= 16)
    uint32_t seg_blocks;     // blocks per task
    uint32_t segs;           // tasks along K per row group
    uint32_t ks;             // consumers that share a row group (K parts)
    uint32_t spk;            // tasks per K part
    uint32_t rgs_per_round;  // row groups in work at a time: task consumers / ks
    uint32_t rounds;
    uint32_t task_consumers;  // rgs_per_round * ks: the consumers that take tasks (the others only quantize)
    uint32_t consumers;       // wavefronts 0 .. consumers - 1 quantize, the rest load
    uint32_t nslots, slot_stride, ipt, lag, pre;
    uint32_t lag_prologue;  // tasks a loader keeps in flight until the activations are quantized
    uint32_t magic_row;  // ceil(2^20 / (9 seg_blocks)): piece index -> row of the task
    uint32_t xq_off, xd_off, partial_off, ring_off;
    uint64_t div_tab;  // 4 bits per consumer: consumer / ks
    int bias_is_f16, bias_first, out_is_f16;
    uint32_t *fault;      // device word for SpinGuard, and the polls a wavefront may spend
    uint32_t spin_limit;
};

// control words: [0] wavefronts that stored their quantized activations, then landed[nslots], consumed[nslots],
// arrived[row groups of the workgroup]
constexpr int MR_CTRL_XQ = 0, MR_CTRL_SLOTS = 4;
__host__ __device__ constexpr uint32_t mr_ctrl_words(uint32_t nslots, uint32_t groups) {
    return (MR_CTRL_SLOTS + 2u * nslots + groups + 3u) & ~3u;
}

__device__ __forceinline__ void mr_store(const MmqRowsParams &p, void *out, const void *bias, size_t n, size_t row,
                                         float v) {
    const size_t o = n * p.M + row;
    float bv = 0.0f;
    if (bias != nullptr) {
        bv = p.bias_is_f16 ? h2f(((const uint16_t *)bias)[row]) : ((const float *)bias)[row];
    }
    if (!p.out_is_f16) {
        ((float *)out)[o] = bias != nullptr ? v + bv : v;
    } else if (p.bias_first) {
        ((uint16_t *)out)[o] = f2h(bias != nullptr ? v + bv : v);
    } else {
        uint16_t h = f2h(v);
        if (bias != nullptr) {
            h = f2h(h2f(h) + bv);
        }
        ((uint16_t *)out)[o] = h;
    }
}

// direct-to-LDS load of 64 x 4 bytes: lane l's 4 bytes at base + voff land at LDS byte address M0 + 4 l
__device__ __forceinline__ void mr_dma4_to_lds(const void *base, uint32_t voff) {
    asm volatile("global_load_lds_dword %0, %1" : : "v"(voff), "s"(base) : "memory");
}

__device__ __forceinline__ void mr_load16(const float *src, float (&v)[16]) {
    const float4 a0 = ((const float4 *)src)[0], a1 = ((const float4 *)src)[1], a2 = ((const float4 *)src)[2],
                 a3 = ((const float4 *)src)[3];
    v[0] = a0.x, v[1] = a0.y, v[2] = a0.z, v[3] = a0.w;
    v[4] = a1.x, v[5] = a1.y, v[6] = a1.z, v[7] = a1.w;
    v[8] = a2.x, v[9] = a2.y, v[10] = a2.z, v[11] = a2.w;
    v[12] = a3.x, v[13] = a3.y, v[14] = a3.z, v[15] = a3.w;
}

// NT: token slots of the matrix instruction's row operand that are stored in LDS (4, 8 or 16 >= N).
// PACKED: the activations arrive quantized (the library's packed layout) and the loaders copy them into LDS ahead of
// the weights; otherwise the consumers quantize fp32 rows (at most XI * 16 values per thread, all requested before the
// first weight request).
// LDS layout of the activations: int8 values [block][16-byte chunk of the block][NT tokens][16 B] (the row operand of
// sub-block sb, k group kg is the half kg % 2 of chunk 2 sb + kg / 2; a wavefront's 8-byte reads of one sub-block
// cover whole 16-byte units of 32 consecutive lanes), block scales [block][NT].
constexpr int MR_XI = 3;
template <int NT, bool PACKED>
__global__ __launch_bounds__(1024) void k_mmq_rows_q4k(const MmqRowsParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    warm_kernel_arguments<sizeof(MmqRowsParams), sizeof(MmqRowsParams)>();
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    SpinGuard guard{p.spin_limit, p.fault};
    uint32_t *const ctrl = (uint32_t *)lds;
    uint32_t *const landed = ctrl + MR_CTRL_SLOTS;
    uint32_t *const consumed = ctrl + MR_CTRL_SLOTS + p.nslots;
    uint32_t *const arrived = ctrl + MR_CTRL_SLOTS + 2u * p.nslots;
    const uint32_t W = (uint32_t)(blockDim.x >> 6);
    const uint32_t C = p.consumers, L = W - C, TC = p.task_consumers;
    const uint32_t row0 = blockIdx.x * p.rows_per_wg;
    const uint32_t rows_here = p.M - row0 < p.rows_per_wg ? p.M - row0 : p.rows_per_wg;
    uint32_t groups = 0;
    for (uint32_t r = 0; r < rows_here; r += p.R) {
        ++groups;
    }
    const uint8_t *__restrict__ wbase = p.w[blockIdx.y];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    const uint32_t steps = p.rounds * p.spk;
    // Task order: index gi = step * TC + c, step = round * spk + s; task consumer c works on K part c % ks of row group
    // round * rgs_per_round + c / ks and takes that part's s-th task in step (round, s). A task whose row group or
    // block range does not exist still takes its turn in the ring (the loader requests 16 bytes for it, the consumer
    // passes), so slot reuse needs no bookkeeping beyond the two counters per slot.

    if ((uint32_t)wave >= C) {
        // ---------------------------------------------------------------- loader
        const uint32_t l = (uint32_t)wave - C;
        const uint32_t ipt = p.ipt;
        // piece i (16 bytes) of a task: row i / (9 seg_blocks), 16-byte chunk i % (9 seg_blocks) of the row's segment
        const uint32_t ppr = p.seg_blocks * 9u;
        const uint32_t pieces = ppr * p.R;
        uint32_t voff[MR_IPT_MAX];
#pragma unroll
        for (int k = 0; k < MR_IPT_MAX; ++k) {
            uint32_t i = (uint32_t)k * 64u + (uint32_t)lane;
            i = i < pieces ? i : pieces - 1u;  // the tail of the last instruction re-reads the last piece into the padding
            const uint32_t r = (i * p.magic_row) >> 20;
            voff[k] = r * p.row_bytes + (i - r * ppr) * 16u;
        }
        // rows beyond M and blocks beyond a row's end exist only in the workgroup that holds the last row; there
        // every address is clamped to the end of the weight
        const bool clamp = row0 + p.rows_per_wg + 1u > p.M;
        const uint32_t last16 = p.total_bytes - 16u;
        uint32_t gi = l, slot = l;  // l < nslots
        uint32_t c = l, step = 0, round = 0, s = 0;
        while (c >= TC) {
            c -= TC;
            ++step;
            ++s;
            if (s == p.spk) {
                s = 0;
                ++round;
            }
        }
        uint32_t pub_gi = l, pub_slot = l;
        uint32_t dst = lds_base + p.ring_off + slot * p.slot_stride;
        const uint32_t dst_step = L * p.slot_stride, dst_wrap = p.nslots * p.slot_stride;
        uint32_t issued = 0, published = 0;
        uint32_t after_acts = 0;  // load instructions issued behind the copy of the packed activations
        bool acts_signalled = !PACKED;
        auto publish = [&]() {
            if (lane == 0) {
                __atomic_store_n(landed + pub_slot, pub_gi + 1u, __ATOMIC_RELAXED);
            }
            pub_gi += L;
            pub_slot += L;
            while (pub_slot >= p.nslots) {
                pub_slot -= p.nslots;
            }
            ++published;
        };
        auto issue_task = [&]() {
            const uint32_t cq = (uint32_t)(p.div_tab >> (4u * c)) & 15u;  // c / ks
            const uint32_t kp = c - cq * p.ks;
            const uint32_t rgi = round * p.rgs_per_round + cq;
            const uint32_t seg = kp * p.spk + s;
            const bool exists = rgi < groups && seg < p.segs;
            const uint32_t task_off = exists ? (row0 + rgi * p.R) * p.row_bytes + seg * p.seg_blocks * (uint32_t)Q4_K_BYTES : 0u;
            const uint8_t *src = wbase + task_off;
#pragma unroll
            for (int k = 0; k < MR_IPT_MAX; ++k) {
                if ((uint32_t)k < ipt) {
                    uint32_t off = exists ? voff[k] : 0u;
                    if (clamp) {
                        off = task_off + off < last16 ? off : last16 - task_off;
                    }
                    dma_set_lds_base(dst + (uint32_t)k * 1024u);
                    dma16_to_lds<0>(src, off);
                }
            }
            ++issued;
            after_acts += ipt;
            gi += L;
            slot += L;
            dst += dst_step;
            while (slot >= p.nslots) {
                slot -= p.nslots;
                dst -= dst_wrap;
            }
            c += L;
            while (c >= TC) {
                c -= TC;
                ++step;
                ++s;
                if (s == p.spk) {
                    s = 0;
                    ++round;
                }
            }
        };
        // Packed activations: the loaders gather them into LDS before any weight request (16-byte chunks of the
        // int8 rows, 4-byte block scales); load instruction i of the copy belongs to loader i % L.
        if constexpr (PACKED) {
            const uint32_t ntok_last = p.N - 1u;
            const uint32_t q_units = p.K * (uint32_t)NT / 16u, d_units = p.nb * (uint32_t)NT;
            for (uint32_t u0 = l * 64u; u0 < q_units; u0 += L * 64u) {
                const uint32_t u = u0 + (uint32_t)lane;  // q_units is a multiple of 64
                uint32_t t = u & (NT - 1);
                t = t < p.N ? t : ntok_last;  // token slots beyond N repeat the last row (never stored)
                dma_set_lds_base(lds_base + p.xq_off + u0 * 16u);
                dma16_to_lds<0>((const uint8_t *)p.pq, t * p.kp + (u / NT) * 16u);
            }
            for (uint32_t u0 = l * 64u; u0 < d_units; u0 += L * 64u) {
                const uint32_t u = u0 + (uint32_t)lane;
                uint32_t t = u & (NT - 1);
                t = t < p.N ? t : ntok_last;
                dma_set_lds_base(lds_base + p.xd_off + u0 * 4u);
                if (u < d_units) {
                    mr_dma4_to_lds(p.pd, (t * p.nb + u / NT) * 4u);
                }
            }
        }
        // A first few tasks are requested before the workgroup barrier (no slot is reused there); nothing is published
        // before the control words are zero.
        for (uint32_t i = 0; i < p.pre && step < steps; ++i) {
            issue_task();
        }
        __builtin_amdgcn_s_barrier();
        // publish what has landed without waiting for it: loads complete in issue order
        auto publish_landed = [&]() {
            const uint32_t outstanding = vmcnt_now();
            if constexpr (PACKED) {
                if (!acts_signalled) {
                    if (outstanding <= after_acts) {  // loads complete in issue order
                        if (lane == 0) {
                            __atomic_fetch_add(ctrl + MR_CTRL_XQ, 1u, __ATOMIC_RELAXED);
                        }
                        acts_signalled = true;
                    } else {
                        return;
                    }
                }
            }
            uint32_t pending = 0;  // ceil(outstanding / ipt) without a division
            for (uint32_t o = 0; o < outstanding; o += ipt) {
                ++pending;
            }
            while (published + pending < issued) {
                publish();
            }
        };
        bool quantized = false;
        while (step < steps) {
            if (!quantized) {
                // While the consumers still fetch and quantize the activations the loaders keep only a few tasks in
                // flight: the memory pipeline of the compute unit serves requests in arrival order, and an activation
                // load behind a long queue of weight requests waits for all of them.
                quantized = PACKED || lds_peek(ctrl + MR_CTRL_XQ) >= C;
                while (!quantized && issued - published >= p.lag_prologue) {
                    wait_vmcnt_at_most((int)((p.lag_prologue - 1u) * ipt));
                    publish();
                }
            }
            if (gi >= p.nslots) {
                // The slot's previous task must have been read. Tasks of this loader that land meanwhile are still
                // published: the consumer that frees the slot may itself be waiting for a task of another loader
                // that waits for a consumer of one of those.
                while (lds_peek(consumed + slot) < gi - p.nslots + 1u) {
                    if (!guard.spend()) {
                        return;
                    }
                    publish_landed();
                    __builtin_amdgcn_s_sleep(1);
                }
                compiler_memory_fence();
            }
            issue_task();
            publish_landed();
            if (issued - published >= p.lag) {
                wait_vmcnt_at_most((int)((p.lag - 1u) * ipt));
                publish();
            }
        }
        if constexpr (PACKED) {
            if (!acts_signalled) {
                wait_vmcnt_at_most((int)(after_acts < 63u ? after_acts : 63u));
                if (lane == 0) {
                    __atomic_fetch_add(ctrl + MR_CTRL_XQ, 1u, __ATOMIC_RELAXED);
                }
                acts_signalled = true;
            }
        }
        while (published < issued) {
            wait_vmcnt_at_most((int)((issued - published - 1u) * ipt));
            publish();
        }
        return;
    }

    // -------------------------------------------------------------------- consumers
    // -- 1. activations into LDS
    uint8_t *const xq = lds + p.xq_off;
    float *const xd = (float *)(lds + p.xd_off);
    const uint32_t qthreads = C * 64u;
    if constexpr (PACKED) {
        for (uint32_t i = threadIdx.x; i < mr_ctrl_words(p.nslots, p.rounds * p.rgs_per_round); i += qthreads) {
            ctrl[i] = 0;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        if ((uint32_t)wave >= TC) {
            return;  // this wavefront takes no tasks
        }
        if (!lds_wait_at_least(ctrl + MR_CTRL_XQ, L, guard)) {  // every loader's share of the activation copy has landed
            return;
        }
    } else {
        // 16 values per thread and pass, every pass requested before anything else happens in this workgroup (the
        // memory pipeline serves requests in arrival order: a load behind the weight requests waits for all of them)
        const uint32_t qpieces = p.N * p.nb * 16u;  // piece = ((token * nb) + block) * 16 + sixteenth
        float xv[MR_XI][16];
#pragma unroll
        for (int it = 0; it < MR_XI; ++it) {
            const uint32_t piece = threadIdx.x + (uint32_t)it * qthreads;
            if (piece < qpieces) {
                mr_load16(p.x + (size_t)piece * 16u, xv[it]);  // the rows are contiguous: piece index = offset / 16
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    xv[it][i] = 0.0f;
                }
            }
        }
        for (uint32_t i = threadIdx.x; i < mr_ctrl_words(p.nslots, p.rounds * p.rgs_per_round); i += qthreads) {
            ctrl[i] = 0;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        const uint32_t per_token = p.nb * 16u;
        uint32_t tok = 0, in_tok = threadIdx.x;  // token of this thread's piece and the piece's position in the token
#pragma unroll
        for (int it = 0; it < MR_XI; ++it) {
            const uint32_t piece = threadIdx.x + (uint32_t)it * qthreads;
            if ((uint32_t)it * qthreads < qpieces) {  // uniform
                while (in_tok >= per_token) {
                    in_tok -= per_token;
                    ++tok;
                }
                const uint32_t qb = in_tok >> 4, qi = in_tok & 15u;
                uint4 q;
                int bsum;
                float d;
                q8k_quantize16(xv[it], (int)qi, q, bsum, d);
                if (piece < qpieces) {
                    *(uint4 *)(xq + (((size_t)qb * 16u + qi) * NT + tok) * 16u) = q;
                    if (qi == 0) {
                        xd[qb * NT + tok] = d;
                    }
                }
                in_tok += qthreads;
            }
        }
        // consumer-only barrier through an LDS counter (the loaders must not stop issuing for it)
        __builtin_amdgcn_s_waitcnt(0xc07f);
        if (lane == 0) {
            __atomic_fetch_add(ctrl + MR_CTRL_XQ, 1u, __ATOMIC_RELAXED);
        }
        if ((uint32_t)wave >= TC) {
            return;  // this wavefront takes no tasks
        }
        if (!lds_wait_at_least(ctrl + MR_CTRL_XQ, C, guard)) {
            return;
        }
    }

    // -- 2. tasks, as they land
    void *const out = p.out[blockIdx.y];
    const void *const bias = p.bias[blockIdx.y];
    const uint32_t c = (uint32_t)wave;
    const uint32_t cq = (uint32_t)(p.div_tab >> (4u * c)) & 15u;
    const uint32_t kp = c - cq * p.ks;
    const int j = lane & 15, kg = lane >> 4;
    const uint32_t jr = (uint32_t)j < p.R ? (uint32_t)j : p.R - 1u;  // lanes beyond the group repeat its last row
    const uint32_t seg_stride = p.seg_blocks * (uint32_t)Q4_K_BYTES;  // bytes of a row's segment in a slot
    // this lane's 8 bytes of a sub-block's row operand: token j (tokens beyond NT repeat the stored ones), half
    // kg % 2 of the sub-block's chunk kg / 2
    const uint8_t *const a_lane = xq + ((size_t)(kg >> 1) * NT + ((uint32_t)j & (NT - 1))) * 16u + (uint32_t)(kg & 1) * 8u;
    const uint32_t tok4 = (4u * (uint32_t)kg) & (NT - 1);  // first of this lane's 4 tokens (repeats beyond NT)
    float *const partial = (float *)(lds + p.partial_off);  // [row group][K part][64 lanes][4]
    uint32_t gi = c, rslot = c;
    while (rslot >= p.nslots) {
        rslot -= p.nslots;
    }
    for (uint32_t round = 0; round < p.rounds; ++round) {
        const uint32_t rgi = round * p.rgs_per_round + cq;
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t s = 0; s < p.spk; ++s) {
            const uint32_t seg = kp * p.spk + s;
            const bool exists = rgi < groups && seg < p.segs;
            if (!lds_wait_at_least(landed + rslot, gi + 1u, guard)) {
                return;
            }
            if (exists) {
                const uint32_t b_first = seg * p.seg_blocks;
                const uint32_t seg_nb = p.nb - b_first < p.seg_blocks ? p.nb - b_first : p.seg_blocks;
                const uint8_t *slot_w = lds + p.ring_off + (size_t)rslot * p.slot_stride + jr * seg_stride;
                for (uint32_t b = 0; b < seg_nb; ++b) {
                    const uint8_t *wrow = slot_w + b * (uint32_t)Q4_K_BYTES;
                    const uint4 hdr = *(const uint4 *)wrow;
                    uint2 wq[4];
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        wq[g] = *(const uint2 *)(wrow + 16 + 32 * g + 8 * kg);
                    }
                    const uint8_t *ab = a_lane + (size_t)(b_first + b) * (256u * NT);
                    uint2 aq[8];
#pragma unroll
                    for (int sb = 0; sb < 8; ++sb) {
                        aq[sb] = *(const uint2 *)(ab + sb * (2 * NT * 16));
                    }
                    const float4 adv = *(const float4 *)(xd + (b_first + b) * NT + tok4);
                    if (b + 1u == seg_nb) {
                        __builtin_amdgcn_s_waitcnt(0xc07f);  // the slot is in registers and may be refilled
                        if (lane == 0) {
                            __atomic_store_n(consumed + rslot, gi + 1u, __ATOMIC_RELAXED);
                        }
                    }
                    // 6-bit scales and mins as bytes (get_scale_min_k4, kquant_common.h:29-37)
                    const float wd = h2f((uint16_t)(hdr.x & 0xffffu));
                    const float wdmin = h2f((uint16_t)(hdr.x >> 16));
                    const uint32_t sc_lo = hdr.y & 0x3f3f3f3fu, mn_lo = hdr.z & 0x3f3f3f3fu;
                    const uint32_t sc_hi = (hdr.w & 0x0f0f0f0fu) | ((hdr.y >> 2) & 0x30303030u);
                    const uint32_t mn_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | ((hdr.z >> 2) & 0x30303030u);
                    int bsum[4] = {0, 0, 0, 0};
                    const mr_intx4 zero = {0, 0, 0, 0};
                    // min term: sum_j mn_j * (sum of a over sub-block j), mins as int16 pairs for the 2-way dot
                    // min term: sum_j mn_j * (sum of a over sub-block j) as a second matrix instruction per sub-block
                    // with the min byte broadcast as the column operand, chained through its accumulator
                    mr_intx4 dm = {0, 0, 0, 0};
#pragma unroll
                    for (int sb = 0; sb < 8; ++sb) {
                        const uint2 wsrc = wq[sb >> 1];
                        const uint2 wv = (sb & 1) ? make_uint2((wsrc.x >> 4) & 0x0f0f0f0fu, (wsrc.y >> 4) & 0x0f0f0f0fu)
                                                  : make_uint2(wsrc.x & 0x0f0f0f0fu, wsrc.y & 0x0f0f0f0fu);
                        const long av = __builtin_bit_cast(long, aq[sb]);
                        const mr_intx4 dq =
                            __builtin_amdgcn_mfma_i32_16x16x32_i8(av, __builtin_bit_cast(long, wv), zero, 0, 0, 0);
                        const uint32_t mn4 =
                            __builtin_amdgcn_perm(0u, sb < 4 ? mn_lo : mn_hi, 0x01010101u * (uint32_t)(sb & 3));
                        dm = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, __builtin_bit_cast(long, make_uint2(mn4, mn4)),
                                                                   dm, 0, 0, 0);
                        const int sc = (int)(((sb < 4 ? sc_lo : sc_hi) >> (8 * (sb & 3))) & 0xffu);
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            bsum[v] += __mul24(dq[v], sc);
                        }
                    }
                    const float ad4[4] = {adv.x, adv.y, adv.z, adv.w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        acc[v] += (ad4[v] * wd) * (float)bsum[v] - (ad4[v] * wdmin) * (float)dm[v];
                    }
                }
            } else if (lane == 0) {
                __atomic_store_n(consumed + rslot, gi + 1u, __ATOMIC_RELAXED);
            }
            gi += TC;
            rslot += TC;
            while (rslot >= p.nslots) {
                rslot -= p.nslots;
            }
        }
        if (rgi >= groups) {
            continue;
        }
        const uint32_t row_in_wg = rgi * p.R + (uint32_t)j;
        const bool row_ok = (uint32_t)j < p.R && row_in_wg < rows_here;
        if (p.ks == 1) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t n = 4u * (uint32_t)kg + (uint32_t)v;
                if (row_ok && n < p.N) {
                    mr_store(p, out, bias, n, row0 + row_in_wg, acc[v]);
                }
            }
            continue;
        }
        // The wavefront that brings a row group's last K part adds the parts in K order (the same bits whoever
        // arrives last) and stores.
        float4 *mine = (float4 *)(partial + ((size_t)(rgi * p.ks + kp) * 64u + (uint32_t)lane) * 4u);
        *mine = make_float4(acc[0], acc[1], acc[2], acc[3]);
        uint32_t before = 0;
        __builtin_amdgcn_s_waitcnt(0xc07f);
        if (lane == 0) {
            before = __atomic_fetch_add(arrived + rgi, 1u, __ATOMIC_RELAXED);
        }
        before = __builtin_amdgcn_readfirstlane(before);
        if (before == p.ks - 1u) {
            compiler_memory_fence();
            float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (uint32_t part = 0; part < p.ks; ++part) {
                const volatile float *src = partial + ((size_t)(rgi * p.ks + part) * 64u + (uint32_t)lane) * 4u;
                sum[0] += src[0];
                sum[1] += src[1];
                sum[2] += src[2];
                sum[3] += src[3];
            }
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t n = 4u * (uint32_t)kg + (uint32_t)v;
                if (row_ok && n < p.N) {
                    mr_store(p, out, bias, n, row0 + row_in_wg, sum[v]);
                }
            }
        }
    }
}

// Launch plan. Returns false when the shape is outside what the kernel covers (the caller uses the other kernels).
struct MmqRowsPlan {
    int NT;
    uint32_t W, rows_per_wg, R, seg_blocks, segs, ks, spk, rgs_per_round, rounds, task_consumers, consumers, nslots,
        slot_stride, ipt, lag, pre, xq_off, xd_off, partial_off, ring_off, grid;
    size_t lds;
};

static bool mmq_rows_plan(const marmot_hip_device *dev, size_t N, size_t K, size_t M, int nw, bool packed,
                          MmqRowsPlan &pl) {
    const size_t weight_bytes = M * (K / QK_K) * Q4_K_BYTES;
    if (K % QK_K != 0 || N < 1 || N > 16 || M == 0 || nw < 1 || nw > 3 || weight_bytes > 0xffffffffull ||
        N * K > 0x7fffffffull / 4) {
        return false;
    }
    // Packed activations: measured against the small-batch kernel with one workgroup per 32 rows (MI355X, 16 rows):
    // 4096 x 4096 12.7 / 14.1 us, 1024 x 4096 11.8 / 13.1, 4096 x 8192 (8 rows) 14.4 / 15.2, 14336 x 4096 18.6 / 18.6,
    // 8192 x 8192 (8 rows) 19.4 / 17.9: this kernel's per-block work on the vector units (scale unpacking, one
    // multiply-add per output and sub-block) and matrix cores is what bounds it once the weights are large.
    if (packed && weight_bytes * (size_t)nw > ((size_t)24 << 20)) {
        return false;
    }
    const uint32_t nb = (uint32_t)(K / QK_K);
    const uint32_t cus = (uint32_t)dev->props.multiProcessorCount;
    pl.NT = N <= 4 ? 4 : (N <= 8 ? 8 : 16);
    const uint32_t loaders = 4, consumers = 12;
    pl.consumers = consumers;
    pl.W = loaders + consumers;
    // fp32 activations: every thread requests all its pieces (16 values each) before the first weight request
    if (!packed && N * nb * 16u > (size_t)MR_XI * consumers * 64u) {
        return false;
    }
    // one workgroup per compute unit and weight; rows spread evenly, in groups of up to 16 of equal size
    const uint32_t wgs = cus / (uint32_t)nw > 0 ? cus / (uint32_t)nw : 1;
    const uint32_t rows0 = (uint32_t)((M + wgs - 1) / wgs);
    const uint32_t groups = (rows0 + 15u) / 16u;
    pl.R = (rows0 + groups - 1) / groups;
    pl.rows_per_wg = groups * pl.R;
    pl.grid = (uint32_t)((M + pl.rows_per_wg - 1) / pl.rows_per_wg);
    if (groups > 64) {
        return false;
    }
    // consumers per row group: all consumers busy when the workgroup has few row groups
    // blocks per task: an odd number (see the slot layout); three when the ring then still holds two tasks per
    // consumer, else one
    const uint32_t budget = 160u * 1024u;
    const uint32_t xq_bytes = (uint32_t)K * (uint32_t)pl.NT;
    const uint32_t xd_bytes = nb * (uint32_t)pl.NT * 4u;
    uint32_t nslots = 0;
    for (uint32_t seg_blocks = nb >= 3 ? 3u : 1u;; seg_blocks = 1u) {
        pl.seg_blocks = seg_blocks;
        pl.segs = (nb + seg_blocks - 1) / seg_blocks;
        uint32_t ks = consumers / groups;
        ks = ks < 1 ? 1 : ks;
        ks = ks > pl.segs ? pl.segs : ks;
        pl.ks = ks;
        pl.spk = (pl.segs + ks - 1) / ks;
        pl.rgs_per_round = consumers / ks;
        pl.task_consumers = pl.rgs_per_round * ks;
        pl.rounds = (groups + pl.rgs_per_round - 1) / pl.rgs_per_round;
        const uint32_t task_bytes = pl.R * seg_blocks * Q4_K_BYTES;
        pl.slot_stride = (task_bytes + 1023u) & ~1023u;
        pl.ipt = pl.slot_stride >> 10;
        const uint32_t partial_bytes = ks > 1 ? pl.rounds * pl.rgs_per_round * ks * 1024u : 0u;
        const uint32_t tasks = pl.rounds * pl.spk * pl.task_consumers;
        bool fits = pl.ipt <= (uint32_t)MR_IPT_MAX;
        nslots = tasks;
        while (fits) {
            pl.xq_off = (mr_ctrl_words(nslots, pl.rounds * pl.rgs_per_round) * 4u + 255u) & ~255u;
            pl.xd_off = pl.xq_off + xq_bytes;
            pl.partial_off = pl.xd_off + xd_bytes;
            pl.ring_off = (pl.partial_off + partial_bytes + 1023u) & ~1023u;
            if (pl.ring_off + pl.slot_stride > budget) {
                fits = false;
                break;
            }
            const uint32_t fit = (budget - pl.ring_off) / pl.slot_stride;
            if (fit >= nslots) {
                break;
            }
            nslots = fit;
        }
        // every consumer's current task has a slot, and the loaders can work ahead
        const uint32_t want = 2u * pl.task_consumers < tasks ? 2u * pl.task_consumers : tasks;
        if (fits && nslots >= want) {
            break;
        }
        if (seg_blocks == 1u) {
            if (fits && nslots >= loaders && nslots >= (pl.task_consumers + loaders < tasks ? pl.task_consumers + loaders : tasks)) {
                break;
            }
            return false;
        }
    }
    pl.nslots = nslots;
    // tasks a loader keeps in flight: what the 6-bit load counter can count, and about 48 KB per workgroup (beyond
    // that the first tasks land as late as the last, see the decode matvec)
    pl.lag = 60u / pl.ipt < 1u ? 1u : 60u / pl.ipt;
    {
        const uint32_t task_bytes = pl.R * pl.seg_blocks * Q4_K_BYTES;
        uint32_t v = (48u * 1024u) / (loaders * task_bytes);
        v = v < 2u ? 2u : v;
        pl.lag = v < pl.lag ? v : pl.lag;
    }
    pl.pre = 2u;
    pl.pre = pl.pre > nslots / loaders ? nslots / loaders : pl.pre;
    pl.pre = pl.pre > pl.lag ? pl.lag : pl.pre;
    pl.lds = (size_t)pl.ring_off + (size_t)nslots * pl.slot_stride;
    return true;
}

// The launch plan as numbers, for the host-side model of the ring protocol (tests/test_rows_protocol.py)
bool mmq_rows_plan_probe(uint32_t cus, size_t N, size_t K, size_t M, int nw, bool packed, uint32_t *out, size_t n_out) {
    marmot_hip_device fake;
    fake.props.multiProcessorCount = (int)cus;
    MmqRowsPlan pl;
    if (n_out < 20 || !mmq_rows_plan(&fake, N, K, M, nw, packed, pl)) {
        return false;
    }
    const uint32_t v[20] = {(uint32_t)pl.NT, pl.W, pl.rows_per_wg, pl.R, pl.seg_blocks, pl.segs, pl.ks, pl.spk,
                            pl.rgs_per_round, pl.rounds, pl.task_consumers, pl.consumers, pl.nslots, pl.slot_stride,
                            pl.ipt, pl.lag, pl.pre, pl.grid, pl.lag < 2u ? pl.lag : 2u, (uint32_t)pl.lds};
    for (int i = 0; i < 20; ++i) {
        out[i] = v[i];
    }
    return true;
}

template <int NT, bool PACKED>
static int launch_mmq_rows_nt(marmot_hip_device *dev, const MmqRowsParams &p, const MmqRowsPlan &pl, int nw) {
    MH_TRY(allow_large_lds(dev, (const void *)k_mmq_rows_q4k<NT, PACKED>));
    hipLaunchKernelGGL((k_mmq_rows_q4k<NT, PACKED>), dim3(pl.grid, (unsigned)nw, 1), dim3(pl.W * 64), pl.lds,
                       dev->stream, p);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

bool mmq_rows_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M, int nw, bool packed) {
    MmqRowsPlan pl;
    return kind == MARMOT_HIP_KIND_Q4_K && mmq_rows_plan(dev, N, K, M, nw, packed, pl);
}

// Q4_K weight set x 1..16 activation rows: fp32 rows (d_x_f32, quantized inside the kernel) or packed Q8_K rows (act).
// Returns MARMOT_HIP_ERROR_NOT_IMPLEMENTED (error text untouched) when the shape is not covered.
int launch_mmq_rows_q4k(marmot_hip_device *dev, const WeightSet &ws, const float *d_x_f32, const ActScratch *act,
                        size_t N, size_t K, size_t M, int out_dtype) {
    MmqRowsPlan pl;
    const bool packed = act != nullptr;
    if ((!packed && (d_x_f32 == nullptr || (((uintptr_t)d_x_f32) & 15) != 0)) ||
        !mmq_rows_plan(dev, N, K, M, ws.count, packed, pl)) {
        return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
    }
    if (packed && ((((uintptr_t)act->qs) & 15) != 0 || (((uintptr_t)act->d) & 3) != 0 || (act->kp & 15) != 0 ||
                   act->kp != K || act->nb != K / QK_K || N * act->kp > 0xffffffffull)) {
        return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
    }
    for (int i = 0; i < ws.count; ++i) {
        if ((((uintptr_t)ws.w[i]) & 15) != 0) {
            return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
        }
    }
    MmqRowsParams p;
    p.fault = dev->fault_word;
    p.spin_limit = dev->spin_limit;
    for (int i = 0; i < 3; ++i) {
        const int src = i < ws.count ? i : 0;
        p.w[i] = (const uint8_t *)ws.w[src];
        p.out[i] = ws.out[src];
        p.bias[i] = ws.bias[src];
    }
    p.x = d_x_f32;
    p.pq = packed ? act->qs : nullptr;
    p.pd = packed ? act->d : nullptr;
    p.kp = packed ? (uint32_t)act->kp : 0u;
    p.K = (uint32_t)K;
    p.M = (uint32_t)M;
    p.N = (uint32_t)N;
    p.nb = (uint32_t)(K / QK_K);
    p.row_bytes = p.nb * Q4_K_BYTES;
    p.total_bytes = p.M * p.row_bytes;
    p.rows_per_wg = pl.rows_per_wg;
    p.R = pl.R;
    p.seg_blocks = pl.seg_blocks;
    p.segs = pl.segs;
    p.ks = pl.ks;
    p.spk = pl.spk;
    p.rgs_per_round = pl.rgs_per_round;
    p.rounds = pl.rounds;
    p.task_consumers = pl.task_consumers;
    p.consumers = pl.consumers;
    p.nslots = pl.nslots;
    p.slot_stride = pl.slot_stride;
    p.ipt = pl.ipt;
    p.lag = pl.lag;
    p.pre = pl.pre;
    p.lag_prologue = pl.lag < 2u ? pl.lag : 2u;  // (mmq_rows_plan_probe reports the same expression)
    p.magic_row = ((1u << 20) + 9u * pl.seg_blocks - 1u) / (9u * pl.seg_blocks);
    p.xq_off = pl.xq_off;
    p.xd_off = pl.xd_off;
    p.partial_off = pl.partial_off;
    p.ring_off = pl.ring_off;
    p.div_tab = 0;
    for (uint32_t c = 0; c < 16; ++c) {
        p.div_tab |= (uint64_t)((c / pl.ks) & 15u) << (4u * c);
    }
    p.bias_is_f16 = ws.bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.bias_first = ws.bias_first ? 1 : 0;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    set_route(packed ? "mmq_rows_q4_k_q8_k" : "mmq_rows_q4_k_q8_k_fused");
    const int nw = ws.count;
    if (packed) {
        return pl.NT == 4   ? launch_mmq_rows_nt<4, true>(dev, p, pl, nw)
               : pl.NT == 8 ? launch_mmq_rows_nt<8, true>(dev, p, pl, nw)
                            : launch_mmq_rows_nt<16, true>(dev, p, pl, nw);
    }
    return pl.NT == 4   ? launch_mmq_rows_nt<4, false>(dev, p, pl, nw)
           : pl.NT == 8 ? launch_mmq_rows_nt<8, false>(dev, p, pl, nw)
                        : launch_mmq_rows_nt<16, false>(dev, p, pl, nw);
}

} // namespace mh

// Decode matvec for Q4_K weights, "row-owning" form: ONE workgroup per compute unit holds that unit's whole share of
// the weight rows in LDS (160 KiB) when it fits, or streams it through an LDS ring when it does not.
//   * Loader wavefronts (one or two of the 16) do nothing but issue direct-to-LDS loads of the row segments, in the
//     order the consumers need them, and publish "segments landed" counters in LDS. A wavefront that issues loads
//     under a saturated memory pipeline is held at the issue stage (measured: 1 - 5 us for 8 instructions when every
//     wavefront of the workgroup requested its share at kernel entry), so wavefronts that compute never issue one.
//   * Consumer wavefronts load the fp32 activation row first (those requests enter the memory pipeline before any
//     weight request: one workgroup barrier), quantize it to Q8_K ONCE per workgroup into LDS, fetch their own slice
//     of it into registers, then take row segments as the counters say they have landed: no barrier per step, a
//     wavefront waits for its own segment only.
//   * A lane owns half (G = 2) or a quarter (G = 1) of a 256-value block, so scale unpacking, the fp32
//     scale-accumulate and the lane reduction are paid once per 128 (64) values instead of once per 32.
// Measured background (MI355X): a dependent 33 MB launch costs 1.5 us before its first wavefront runs; a plain read
// of those bytes then streams at the rate of a large read (6.2 TB/s). The register-streaming matvec issued 3.75 M
// vector instructions per launch at this shape, 43 % of them the activation quantization repeated by each of its 512
// workgroups, and kept the vector units busy for 64 % of the kernel.
// Arithmetic is the reference's: cpu_vec_dot_q4_k_q8_k (vec_dot_impl.h:689-732) per block on Q8_K activations packed
// like cpu_matmul_quant_pack_q8_k_f32 (matmul_quant_pack.c:106-142); only the fp32 summation order over blocks differs.
#include "mh_rows.h"

namespace mh {

struct RowsParams {
    const uint8_t *w[3];  // weights of one shape sharing the activations; blockIdx.y selects one
    void *out[3];
    const void *bias[3];
    const float *x;       // fp32 activations [N][K]
    uint32_t K;
    uint32_t M;
    uint32_t nb;           // blocks per weight row
    uint32_t row_bytes;
    uint32_t rows_per_wg;  // a multiple of rpt
    uint32_t segs;         // K segments per row (each wavefront always works on segment wave % segs)
    uint32_t seg_blocks;   // blocks per segment (the last one may be shorter)
    uint32_t rpt;          // rows per task (> 1 only with one segment per row), a power of two
    uint32_t rpt_shift;
    uint32_t wstep;        // consumers / segs: row groups advance by this much per round
    uint32_t lag;          // segments a loader requests beyond the one it publishes next
    uint32_t loader_rg_step;  // loaders / segs
    uint32_t pre;             // segments each loader requests before the workgroup barrier
    uint32_t pad_shift;    // lane slot = row_in_task << pad_shift | block_in_segment
    uint32_t consumers;    // wavefronts 0 .. consumers-1 compute, the rest load
    uint32_t nslots;       // LDS slots of the segment ring (segment i lands in slot i % nslots)
    uint32_t slot_stride;  // bytes between slots (multiple of 1024: whole load instructions)
    uint32_t xq_stride;    // bytes of one quantized activation row in LDS
    uint32_t xq_off;       // LDS offsets: [control words][quantized activations][partial sums][ring]
    uint32_t ring_off;
    uint32_t partial_off;
    uint32_t n0;           // first activation row
    int bias_is_f16;
    int bias_first;
    int out_is_f16;
    uint32_t *fault;      // device word for SpinGuard, and the polls a wavefront may spend
    uint32_t spin_limit;
    MH_TIMELINE_FIELD
};

// LDS control words (uint32): [0] wavefronts that have stored their quantized activations; then per ring slot
// "segment index + 1 that has landed here" (written by the loaders) and "segment index + 1 that has been read from
// here" (written by the consumers: the slot may be refilled).
constexpr int CTRL_XQ = 0, CTRL_SLOTS = 4;
__host__ __device__ constexpr uint32_t ctrl_words(uint32_t nslots, uint32_t groups) {
    return (CTRL_SLOTS + 2u * nslots + groups + 3u) & ~3u;  // + per row group: K segments added up so far
}

__device__ __forceinline__ void store_result(const RowsParams &p, void *out, const void *bias, size_t n, size_t row,
                                             float v) {
    const size_t o = n * p.M + row;
    float bv = 0.0f;
    if (bias != nullptr) {
        bv = p.bias_is_f16 ? h2f(((const uint16_t *)bias)[row]) : ((const float *)bias)[row];
    }
    if (!p.out_is_f16) {
        ((float *)out)[o] = bias != nullptr ? v + bv : v;
    } else if (p.bias_first) {
        // q/k/v projection: the fp32 accumulator starts from the bias, one rounding at the store
        ((uint16_t *)out)[o] = f2h(bias != nullptr ? v + bv : v);
    } else {
        // matmul: store f16(dot), then the epilogue adds the bias to the stored f16 value
        uint16_t h = f2h(v);
        if (bias != nullptr) {
            h = f2h(h2f(h) + bv);
        }
        ((uint16_t *)out)[o] = h;
    }
}

// NC fp32 activation rows; a lane covers G groups of 64 values of one block (G = 2: two lanes per block, G = 1: four).
template <int NC, int G>
__global__ __launch_bounds__(1024) void k_matvec_rows_q4k(const RowsParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    MH_MARK_DECL
    MH_MARK(p, 0);  // timeline: wavefront started
    warm_kernel_arguments<sizeof(RowsParams), sizeof(RowsParams)>();
    constexpr int SB = 16 * G;   // block positions per wavefront
    constexpr int NQ = 2 * G;    // 16-byte pieces of packed nibbles per lane and block
    constexpr int NA = 4 * G;    // 16-byte pieces of int8 activations per lane and block
    constexpr int NS = 2 * G;    // 32-value sub-blocks per lane and block
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // uniform: scalar registers and branches
    SpinGuard guard{p.spin_limit, p.fault};
    uint32_t *const ctrl = (uint32_t *)lds;
    uint32_t *const landed = ctrl + CTRL_SLOTS;
    uint32_t *const consumed = ctrl + CTRL_SLOTS + p.nslots;
    uint32_t *const arrived = ctrl + CTRL_SLOTS + 2u * p.nslots;  // per row group: K segments summed so far
    const int W = (int)(blockDim.x >> 6);
    const uint32_t C = p.consumers;
    const uint32_t L = (uint32_t)W - C;  // W = consumers + loaders
    const uint32_t segs = p.segs;
    const uint32_t wstep = p.wstep;  // consumers / segs (integer divisions are kept out of the kernel: ~40 scalar instructions each)
    const uint32_t row0 = blockIdx.x * p.rows_per_wg;
    const uint32_t rows_here = p.M - row0 < p.rows_per_wg ? p.M - row0 : p.rows_per_wg;
    const uint32_t groups = (rows_here + p.rpt - 1) >> p.rpt_shift;
    const uint8_t *__restrict__ wbase = uniform_pointer(p.w[blockIdx.y]);  // the loads take it in scalar registers
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    // Segment order: index gi = round * C + consumer; consumer c works on K segment c % segs of row group
    // c / segs + round * wstep. Only the last round can be incomplete, and there the missing segments are the last
    // ones, so "segment gi exists" is monotone in gi.

    if ((uint32_t)wave >= C) {
        // ---------------------------------------------------------------- loader
        // This wavefront's instruction stream is the rate at which the workgroup can request bytes (a wavefront issues
        // about one instruction every five clocks), so the loop is kept to a few dozen instructions per segment: the
        // loader count is a multiple of segs and divides the consumer count, which makes loader l's segments
        // l, l + L, l + 2 L, ... one K segment (l % segs) of row groups l / segs + j * (L / segs): constant strides.
        const uint32_t l = (uint32_t)wave - C;
        const uint32_t lane16 = (uint32_t)lane * 16u;
        uint32_t lseg = l, rg = 0;
        while (lseg >= segs) {
            lseg -= segs;
            ++rg;
        }
        const uint32_t rg_step = p.loader_rg_step;  // L / segs
        const uint32_t seg_first = lseg * p.seg_blocks;
        const uint32_t seg_nb = p.nb - seg_first < p.seg_blocks ? p.nb - seg_first : p.seg_blocks;
        const uint32_t task_bytes = segs == 1 ? p.rpt * p.row_bytes : seg_nb * (uint32_t)Q4_K_BYTES;
        const uint32_t full = task_bytes >> 10;  // whole KiBs of a segment
        // Load instructions per segment of THIS loader (it always works on one K segment, and the last K segment of a
        // row can be shorter than the others): the landed-segment arithmetic below divides the outstanding
        // instructions by it, so it must be the number actually issued, not the slot size.
        const uint32_t ipt = (task_bytes + 1023u) >> 10;
        // per-lane offset of the (possibly partial) last KiB: lanes beyond the segment re-read its last 16 bytes into
        // the padding of the slot, so every instruction is issued by all lanes and the count per segment is exact
        uint32_t tail_in = full * 1024u + lane16;
        tail_in = tail_in < task_bytes ? tail_in : task_bytes - 16u;
        const uint32_t off_step = rg_step * p.rpt * p.row_bytes;
        uint32_t task_off = (row0 + rg * p.rpt) * p.row_bytes + seg_first * (uint32_t)Q4_K_BYTES;
        // rows beyond M exist only in the last workgroup; their reads are clamped to the end of the weight
        const uint32_t w_last16 = p.M * p.row_bytes - 16u;
        const bool ragged = (row0 + p.rows_per_wg) > p.M;
        uint32_t gi = l, slot = l;                  // l < nslots
        uint32_t pub_gi = l, pub_slot = l;
        uint32_t dst = lds_base + p.ring_off + slot * p.slot_stride;
        const uint32_t dst_step = L * p.slot_stride, dst_wrap = p.nslots * p.slot_stride;
        uint32_t issued = 0, published = 0;
        auto publish = [&]() {
            if (published == 0) {
                MH_MARK(p, 4);  // loader: its first segment has landed
            }
            if (lane == 0) {
                __atomic_store_n(landed + pub_slot, pub_gi + 1u, __ATOMIC_RELAXED);
            }
            pub_gi += L;
            pub_slot += L;
            pub_slot = pub_slot >= p.nslots ? pub_slot - p.nslots : pub_slot;
            ++published;
        };
        const uint32_t max_lag = p.lag;  // segments in flight: vmcnt counts 6 bits
        auto issue_segment = [&]() {
            if (!ragged) {
                uint32_t k = 0;
                for (; k + 4 <= full; k += 4) {
                    dma_set_lds_base(dst + k * 1024u);
                    const uint32_t off = task_off + k * 1024u + lane16;
                    dma16_to_lds<0>(wbase, off);
                    dma16_to_lds<1>(wbase, off);
                    dma16_to_lds<2>(wbase, off);
                    dma16_to_lds<3>(wbase, off);
                }
                if (k < ipt) {
                    dma_set_lds_base(dst + k * 1024u);
                    const uint32_t off = task_off + k * 1024u + lane16;
                    const uint32_t rem = full - k;  // 0..3 whole KiBs go out under this M0, then the partial one
                    if (rem > 0) dma16_to_lds<0>(wbase, off);
                    if (rem > 1) dma16_to_lds<1>(wbase, off);
                    if (rem > 2) dma16_to_lds<2>(wbase, off);
                    if (full < ipt) {
                        const uint32_t o = task_off + tail_in - rem * 1024u;
                        if (rem == 0) dma16_to_lds<0>(wbase, o);
                        else if (rem == 1) dma16_to_lds<1>(wbase, o);
                        else if (rem == 2) dma16_to_lds<2>(wbase, o);
                        else dma16_to_lds<3>(wbase, o);
                    }
                }
            } else {
                for (uint32_t k = 0; k < ipt; ++k) {
                    uint32_t in_task = k * 1024u + lane16;
                    in_task = in_task < task_bytes ? in_task : task_bytes - 16u;
                    uint32_t off = task_off + in_task;
                    off = off < w_last16 ? off : w_last16;
                    dma_set_lds_base(dst + k * 1024u);
                    dma16_to_lds<0>(wbase, off);
                }
            }
            ++issued;
            gi += L;
            slot += L;
            dst += dst_step;
            if (slot >= p.nslots) {
                slot -= p.nslots;
                dst -= dst_wrap;
            }
            task_off += off_step;
        };
        // A first few segments are requested before the workgroup barrier (the consumers are still fetching their
        // kernel arguments and requesting the activations then); nothing is published before the control words are zero.
        MH_MARK(p, 1);  // loader: about to issue its first request
        for (uint32_t i = 0; i < p.pre && rg < groups; ++i, rg += rg_step) {
            issue_segment();
        }
        MH_MARK(p, 2);  // loader: first requests issued
        __builtin_amdgcn_s_barrier();
        MH_MARK(p, 3);  // loader: workgroup barrier passed
        // publish what has landed without waiting for it: loads complete in issue order, so the segments behind the
        // `outstanding` youngest instructions are in LDS
        auto publish_landed = [&]() {
            uint32_t pending = 0;  // ceil(outstanding / ipt) without a division
            for (uint32_t o = 0, outstanding = vmcnt_now(); o < outstanding; o += ipt) {
                ++pending;
            }
            while (published + pending < issued) {
                publish();
            }
        };
        for (; rg < groups; rg += rg_step) {
            if (gi >= p.nslots) {
                // The slot's previous segment must have been read. Segments of this loader that land meanwhile are
                // still published: the consumer that frees the slot may itself be waiting for a segment of another
                // loader that waits for a consumer of one of those.
                while (lds_peek(consumed + slot) < gi - p.nslots + 1u) {
                    if (!guard.spend()) {
                        return;
                    }
                    publish_landed();
                    __builtin_amdgcn_s_sleep(1);
                }
                compiler_memory_fence();
            }
            issue_segment();
            publish_landed();
            if (issued - published >= max_lag) {
                wait_vmcnt_at_most((int)((max_lag - 1u) * ipt));
                publish();
            }
        }
        MH_MARK(p, 5);  // loader: last request issued
        while (published < issued) {
            wait_vmcnt_at_most((int)((issued - published - 1u) * ipt));
            publish();
        }
        MH_MARK(p, 6);  // loader: its last segment has landed
        MH_MARK_FLUSH(p);
        return;
    }
    // -------------------------------------------------------------------- consumer
    // -- 1. consumers request their activations before anything else happens in this workgroup
    // Thread t quantizes sixteenths t and t + (consumer threads) of the activation row (block = sixteenth / 16);
    // the consumers are the low wavefronts
    constexpr int XI = 2;
    float xv[NC][XI][16];
    const uint32_t qthreads = p.consumers * 64u;
    {
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            const uint32_t qslot = threadIdx.x + (uint32_t)it * qthreads;
            if (threadIdx.x < qthreads && qslot < p.nb * 16u) {
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    const float4 *src = (const float4 *)(p.x + (size_t)(p.n0 + n) * p.K + (size_t)qslot * 16);
                    const float4 a0 = src[0], a1 = src[1], a2 = src[2], a3 = src[3];
                    xv[n][it][0] = a0.x, xv[n][it][1] = a0.y, xv[n][it][2] = a0.z, xv[n][it][3] = a0.w;
                    xv[n][it][4] = a1.x, xv[n][it][5] = a1.y, xv[n][it][6] = a1.z, xv[n][it][7] = a1.w;
                    xv[n][it][8] = a2.x, xv[n][it][9] = a2.y, xv[n][it][10] = a2.z, xv[n][it][11] = a2.w;
                    xv[n][it][12] = a3.x, xv[n][it][13] = a3.y, xv[n][it][14] = a3.z, xv[n][it][15] = a3.w;
                }
            }
        }
    }
    MH_MARK(p, 1);  // consumer: activation loads issued
    for (uint32_t i = threadIdx.x; i < ctrl_words(p.nslots, p.rows_per_wg >> p.rpt_shift); i += C * 64u) {
        ctrl[i] = 0;
    }
    // The activation loads are in the memory pipeline (mostly ahead of the weight requests: the pipeline serves
    // requests in arrival order) and the control words are zero.
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    MH_MARK(p, 2);  // consumer: workgroup barrier passed
    void *const out = p.out[blockIdx.y];
    const void *const bias = p.bias[blockIdx.y];
    {
        const int part = lane / SB;  // which G groups of the block
        const int slot = lane % SB;
        const uint32_t r_in = (uint32_t)slot >> p.pad_shift;
        const uint32_t b = (uint32_t)slot & ((1u << p.pad_shift) - 1u);
        uint32_t seg = (uint32_t)wave, wq = 0;  // wave % segs, wave / segs
        while (seg >= segs) {
            seg -= segs;
            ++wq;
        }
        const uint32_t seg_first = seg * p.seg_blocks;
        const uint32_t seg_nb = p.nb - seg_first < p.seg_blocks ? p.nb - seg_first : p.seg_blocks;
        const uint32_t b_global = seg_first + b;
        const bool lane_valid = b < seg_nb && r_in < p.rpt;

        // -- 2. activations: quantize once per workgroup into LDS, then every lane fetches its block share
        uint4 a[NC][NA];
        int bs[NC][NS];
        float ad[NC];
        {
#pragma unroll
            for (int it = 0; it < XI; ++it) {
                const uint32_t qslot = threadIdx.x + (uint32_t)it * qthreads;
                if (qslot < p.nb * 16u) {
                    const uint32_t qb = qslot >> 4, qi = qslot & 15u;
#pragma unroll
                    for (int n = 0; n < NC; ++n) {
                        uint4 q;
                        int bsum;
                        float d;
                        q8k_quantize16(xv[n][it], (int)qi, q, bsum, d);
                        uint8_t *xq = lds + p.xq_off + (size_t)n * p.xq_stride;
                        // 16-byte pieces of a block are XOR-swizzled by the block index: conflict-free for this store
                        // (16 lanes, one block) and for the strided fetch below (16 lanes, 16 blocks, one piece index)
                        *(uint4 *)(xq + (size_t)qb * QK_K + 16u * (qi ^ (qb & 15u))) = q;
                        ((int16_t *)(xq + (size_t)p.nb * QK_K))[qb * 16 + qi] = (int16_t)bsum;
                        if (qi == 0) {
                            ((float *)(xq + (size_t)p.nb * (QK_K + 32)))[qb] = d;
                        }
                    }
                }
            }
            // consumer-only barrier through an LDS counter (the loaders must not stop issuing for it)
            __builtin_amdgcn_s_waitcnt(0xc07f);
            if (lane == 0) {
                __atomic_fetch_add(ctrl + CTRL_XQ, 1u, __ATOMIC_RELAXED);
            }
            MH_MARK(p, 3);  // consumer: own part of the activations quantized (their loads have arrived)
            if (!lds_wait_at_least(ctrl + CTRL_XQ, C, guard)) {
                return;
            }
            MH_MARK(p, 4);  // consumer: every consumer's part is in LDS
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                const uint8_t *xq = lds + p.xq_off + (size_t)n * p.xq_stride;
                if (lane_valid) {
#pragma unroll
                    for (int c = 0; c < NA; ++c) {
                        const uint32_t piece = (uint32_t)(part * NA + c);
                        a[n][c] = *(const uint4 *)(xq + (size_t)b_global * QK_K + 16u * (piece ^ (b_global & 15u)));
                    }
                    const int16_t *bsp = (const int16_t *)(xq + (size_t)p.nb * QK_K) + b_global * 16 + part * (4 * G);
#pragma unroll
                    for (int j = 0; j < NS; ++j) {
                        const uint32_t two = *(const uint32_t *)(bsp + 2 * j);
                        bs[n][j] = (int)(int16_t)(two & 0xffffu) + (int)(int16_t)(two >> 16);
                    }
                    ad[n] = ((const float *)(xq + (size_t)p.nb * (QK_K + 32)))[b_global];
                } else {
#pragma unroll
                    for (int c = 0; c < NA; ++c) {
                        a[n][c] = make_uint4(0, 0, 0, 0);
                    }
#pragma unroll
                    for (int j = 0; j < NS; ++j) {
                        bs[n][j] = 0;
                    }
                    ad[n] = 0.0f;
                }
            }
        }

        // -- 3. segments, as they land
        float *partial = (float *)(lds + p.partial_off);  // [row in workgroup][NC][segs]
        const uint32_t blk_off = (segs == 1 ? r_in * p.row_bytes : 0u) + b * (uint32_t)Q4_K_BYTES;
        // 6-bit scales / mins of this lane's sub-blocks (get_scale_min_k4, kquant_common.h:29-37) as packed bytes:
        // sub-blocks 0..3 are (s[j] & 63, s[j+4] & 63); sub-blocks 4..7 take their low nibbles from s[j+4] and their
        // two high bits from s[j-4] / s[j]. G = 2: part selects the low or the high four; G = 1: two of the four.
        const bool hi_half = (part * NS) >= 4;
        const int byte_shift = 8 * ((part * NS) & 3);
        uint32_t gi = (uint32_t)wave, rslot = (uint32_t)wave;
        while (rslot >= p.nslots) {
            rslot -= p.nslots;
        }
        MH_MARK(p, 5);  // consumer: ready for its first segment
        for (uint32_t rg = wq; rg < groups; rg += wstep) {
            if (!lds_wait_at_least(landed + rslot, gi + 1u, guard)) {
                return;
            }
            if (rg == wq) {
                MH_MARK(p, 6);  // consumer: first segment there
            }
            if (rg + wstep >= groups) {
                MH_MARK(p, 7);  // consumer: last segment there
            }
            const uint8_t *blk = lds + p.ring_off + (size_t)rslot * p.slot_stride + blk_off;
            const uint4 hdr = *(const uint4 *)blk;
            uint4 q[NQ];
#pragma unroll
            for (int c = 0; c < NQ; ++c) {
                q[c] = *(const uint4 *)(blk + 16 + part * (32 * G) + 16 * c);
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the slot is in registers and may be overwritten
            if (lane == 0) {
                __atomic_store_n(consumed + rslot, gi + 1u, __ATOMIC_RELAXED);
            }
            gi += C;
            rslot += C;
            while (rslot >= p.nslots) {
                rslot -= p.nslots;
            }
            const float wd = h2f((uint16_t)(hdr.x & 0xffffu));
            const float wdmin = h2f((uint16_t)(hdr.x >> 16));
            const uint32_t sc_lo = hdr.y & 0x3f3f3f3fu, mn_lo = hdr.z & 0x3f3f3f3fu;
            const uint32_t sc_hi = (hdr.w & 0x0f0f0f0fu) | ((hdr.y >> 2) & 0x30303030u);
            const uint32_t mn_hi = ((hdr.w >> 4) & 0x0f0f0f0fu) | ((hdr.z >> 2) & 0x30303030u);
            const uint32_t sc4 = (hi_half ? sc_hi : sc_lo) >> byte_shift;
            const uint32_t mn4 = (hi_half ? mn_hi : mn_lo) >> byte_shift;
            int isum[NC], msum[NC];
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                isum[n] = 0;
                msum[n] = 0;
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                uint4 lo0, hi0, lo1, hi1;
                lo0.x = q[2 * g].x & 0x0f0f0f0fu, hi0.x = (q[2 * g].x >> 4) & 0x0f0f0f0fu;
                lo0.y = q[2 * g].y & 0x0f0f0f0fu, hi0.y = (q[2 * g].y >> 4) & 0x0f0f0f0fu;
                lo0.z = q[2 * g].z & 0x0f0f0f0fu, hi0.z = (q[2 * g].z >> 4) & 0x0f0f0f0fu;
                lo0.w = q[2 * g].w & 0x0f0f0f0fu, hi0.w = (q[2 * g].w >> 4) & 0x0f0f0f0fu;
                lo1.x = q[2 * g + 1].x & 0x0f0f0f0fu, hi1.x = (q[2 * g + 1].x >> 4) & 0x0f0f0f0fu;
                lo1.y = q[2 * g + 1].y & 0x0f0f0f0fu, hi1.y = (q[2 * g + 1].y >> 4) & 0x0f0f0f0fu;
                lo1.z = q[2 * g + 1].z & 0x0f0f0f0fu, hi1.z = (q[2 * g + 1].z >> 4) & 0x0f0f0f0fu;
                lo1.w = q[2 * g + 1].w & 0x0f0f0f0fu, hi1.w = (q[2 * g + 1].w >> 4) & 0x0f0f0f0fu;
                const int s0 = (int)((sc4 >> (16 * g)) & 0xffu), s1 = (int)((sc4 >> (16 * g + 8)) & 0xffu);
                const int m0 = (int)((mn4 >> (16 * g)) & 0xffu), m1 = (int)((mn4 >> (16 * g + 8)) & 0xffu);
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    // values 64 g' + 0..31 sit in the low nibbles, 64 g' + 32..63 in the high nibbles of the same bytes
                    const int dl = dot16r(lo1, a[n][4 * g + 1], dot16r(lo0, a[n][4 * g], 0));
                    const int dh = dot16r(hi1, a[n][4 * g + 3], dot16r(hi0, a[n][4 * g + 2], 0));
                    isum[n] += __mul24(s0, dl) + __mul24(s1, dh);
                    msum[n] += __mul24(m0, bs[n][2 * g]) + __mul24(m1, bs[n][2 * g + 1]);
                }
            }
#pragma unroll
            for (int n = 0; n < NC; ++n) {
                float v = (ad[n] * wd) * (float)isum[n] - (ad[n] * wdmin) * (float)msum[n];
                v = lane_valid ? v : 0.0f;
                v = row16_sum(v);
                const int iv = __builtin_bit_cast(int, v);
                const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
                const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
                const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
                const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
                if (G == 2 && p.rpt == 2) {
                    // one segment per row here: lanes 0..15 and 32..47 hold row 0 of the task, 16..31 and 48..63 row 1
                    const uint32_t rl = rg * 2 + (uint32_t)lane;
                    if (lane < 2 && rl < rows_here) {
                        store_result(p, out, bias, p.n0 + n, row0 + rl, lane == 0 ? r0 + r2 : r1 + r3);
                    }
                } else if (segs == 1) {
                    if (lane == 0) {
                        store_result(p, out, bias, p.n0 + n, row0 + rg, (r0 + r1) + (r2 + r3));
                    }
                } else if (lane == 0) {
                    partial[(rg * NC + n) * segs + seg] = (r0 + r1) + (r2 + r3);
                }
            }
            if (segs > 1) {
                // The wavefront that brings a row's last K segment adds them up, in segment order (the same bits
                // whoever arrives last), and stores the row: no workgroup barrier, no epilogue.
                uint32_t before = 0;
                __builtin_amdgcn_s_waitcnt(0xc07f);  // this wavefront's partial sums are in LDS
                if (lane == 0) {
                    before = __atomic_fetch_add(arrived + rg, 1u, __ATOMIC_RELAXED);
                }
                before = __builtin_amdgcn_readfirstlane(before);
                if (before == segs - 1u && lane < NC) {
                    float v = 0.0f;
                    for (uint32_t sgm = 0; sgm < segs; ++sgm) {
                        v += __builtin_bit_cast(float, __atomic_load_n((const uint32_t *)partial + (rg * NC + lane) * segs + sgm,
                                                                       __ATOMIC_RELAXED));
                    }
                    store_result(p, out, bias, p.n0 + lane, row0 + rg, v);
                }
            }
        }
        MH_MARK(p, 8);  // consumer: done
        MH_MARK_FLUSH(p);
    }
}

// Launch plan. Returns false when the shape is outside what the kernel covers (the caller uses the other kernels).
struct RowsPlan {
    int G, W;
    uint32_t rows_per_wg, segs, seg_blocks, rpt, pad_shift, lag, pre, consumers, nslots, slot_stride, xq_stride, xq_off,
        ring_off, partial_off, grid;
    size_t lds;
};

static bool rows_plan(const marmot_hip_device *dev, size_t N, size_t K, size_t M, int nw, RowsPlan &pl) {
    const size_t weight_bytes = M * (K / QK_K) * Q4_K_BYTES;
    // Sizes: below ~4 MB the launch dominates and the other kernels' smaller workgroups start sooner; beyond 128 MB the
    // register-streaming kernels stream better (measured at 128256 x 4096: 55 against 60 us).
    if (K % QK_K != 0 || N == 0 || N > 2 || M == 0 || nw < 1 || weight_bytes < ((size_t)4 << 20) ||
        weight_bytes > ((size_t)128 << 20)) {
        return false;
    }
    const uint32_t nb = (uint32_t)(K / QK_K);
    const uint32_t cus = (uint32_t)dev->props.multiProcessorCount;
    const uint32_t row_bytes = nb * Q4_K_BYTES;
    // two activation rows with two groups per lane do not fit the 128 registers of 16 wavefronts per compute unit
    const int G = N == 1 ? 2 : 1;
    const uint32_t SB = 16u * (uint32_t)G;
    pl.G = G;
    if (nb <= SB) {
        pl.segs = 1;
        pl.seg_blocks = nb;
        pl.pad_shift = nb <= 16 ? 4 : 5;
        pl.rpt = SB >> pl.pad_shift;
    } else {
        pl.segs = (nb + SB - 1) / SB;
        pl.seg_blocks = (nb + pl.segs - 1) / pl.segs;
        pl.pad_shift = G == 2 ? 5 : 4;
        pl.rpt = 1;
    }
    if (pl.segs > 4 || (pl.segs - 1) * pl.seg_blocks >= nb) {
        return false;
    }
    // one workgroup per compute unit and weight; rows spread evenly
    const uint32_t wgs = cus / (uint32_t)nw > 0 ? cus / (uint32_t)nw : 1;
    uint32_t rows = (uint32_t)((M + wgs - 1) / wgs);
    rows = ((rows + pl.rpt - 1) / pl.rpt) * pl.rpt;
    pl.rows_per_wg = rows;
    pl.grid = (uint32_t)((M + rows - 1) / rows);
    // 16 wavefronts: four load (a multiple of segs that divides the consumer count, see the loader loop), twelve
    // compute and quantize (16 values per thread, two passes at most). Measured at 4096 x 14336 / 14336 x 4096 with
    // 2 / 4 / 6 loaders: 11.0 / 9.3 / 9.8 and 9.0 / 8.4 / 9.0 us.
    const uint32_t loaders = pl.segs == 3 ? 3u : 4u;
    pl.consumers = ((16u - loaders) / loaders) * loaders;
    pl.W = (int)(pl.consumers + loaders);
    if (nb * 16u > 2u * pl.consumers * 64u) {
        return false;
    }
    const uint32_t task_bytes = pl.segs == 1 ? pl.rpt * row_bytes : pl.seg_blocks * Q4_K_BYTES;
    pl.slot_stride = (task_bytes + 1023u) & ~1023u;
    if (pl.slot_stride > 15u * 1024u) {
        return false;
    }
    pl.xq_stride = (nb * (QK_K + 32 + 4) + 15u) & ~15u;
    const uint32_t partial_bytes = ((rows * (uint32_t)N * pl.segs * 4u) + 15u) & ~15u;
    const uint32_t budget = 160u * 1024u;
    const uint32_t tasks = (rows / pl.rpt) * pl.segs;
    uint32_t nslots = tasks;
    for (;;) {  // the control words grow with the slot count, which decides where the ring starts
        pl.xq_off = ctrl_words(nslots, rows / pl.rpt) * 4u;
        pl.partial_off = pl.xq_off + pl.xq_stride * (uint32_t)N;
        pl.ring_off = (pl.partial_off + partial_bytes + 1023u) & ~1023u;
        if (pl.ring_off + 4u * pl.slot_stride > budget) {
            return false;
        }
        const uint32_t fit = (budget - pl.ring_off) / pl.slot_stride;
        if (fit >= nslots) {
            break;
        }
        nslots = fit;
    }
    if (nslots < 8 || nslots < loaders) {
        return false;
    }
    pl.nslots = nslots;
    // Segments a loader may have in flight: at most what the 6-bit load counter can count (landed segments are
    // published by polling the counter) ...
    const uint32_t ipt = pl.slot_stride >> 10;
    pl.lag = 60u / ipt < 1u ? 1u : 60u / ipt;
    // ... and about 48 KB per workgroup: with everything requested at once the memory system serves all of a
    // workgroup's segments side by side, the first ones land as late as the last, and the consumers start when the
    // stream is nearly over (measured at 4096 x 14336: segments in flight per loader unlimited / 4 / 3 / 2:
    // 9.45 / 9.34 / 8.80 / 9.12 us).
    {
        uint32_t v = (48u * 1024u) / (loaders * task_bytes);
        v = v < 2u ? 2u : v;
        pl.lag = v < pl.lag ? v : pl.lag;
    }
    // Segments requested before the workgroup barrier: no slot is reused there. Measured 0 / 2 / 4: 9.8 / 9.3 / 9.6 us.
    pl.pre = 2u;
    pl.pre = pl.pre > nslots / loaders ? nslots / loaders : pl.pre;
    pl.pre = pl.pre > pl.lag ? pl.lag : pl.pre;
    pl.lds = (size_t)pl.ring_off + (size_t)nslots * pl.slot_stride;
    return true;
}

// The launch plan as numbers, for the host-side model of the ring protocol (tests/test_rows_protocol.py)
bool rows_plan_probe(uint32_t cus, size_t N, size_t K, size_t M, int nw, uint32_t *out, size_t n_out) {
    marmot_hip_device fake;
    fake.props.multiProcessorCount = (int)cus;
    RowsPlan pl;
    if (n_out < 13 || !rows_plan(&fake, N, K, M, nw, pl)) {
        return false;
    }
    const uint32_t v[13] = {(uint32_t)pl.G, (uint32_t)pl.W, pl.rows_per_wg, pl.segs, pl.seg_blocks, pl.rpt, pl.lag,
                            pl.pre, pl.consumers, pl.nslots, pl.slot_stride, pl.grid, (uint32_t)pl.lds};
    for (int i = 0; i < 13; ++i) {
        out[i] = v[i];
    }
    return true;
}

template <int NC, int G>
static int launch_rows(marmot_hip_device *dev, const RowsParams &p, const RowsPlan &pl, int nw) {
    MH_TRY(allow_large_lds(dev, (const void *)k_matvec_rows_q4k<NC, G>));
    hipLaunchKernelGGL((k_matvec_rows_q4k<NC, G>), dim3(pl.grid, (unsigned)nw, 1), dim3((unsigned)pl.W * 64), pl.lds,
                       dev->stream, p);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

// Tries the row-owning kernel for a Q4_K weight set with fp32 activations. Returns MARMOT_HIP_ERROR_NOT_IMPLEMENTED
// (error text untouched) when the shape is not covered.
int launch_matvec_rows_q4k(marmot_hip_device *dev, const WeightSet &ws, const float *d_x_f32, size_t N, size_t K,
                           size_t M, int out_dtype) {
    RowsPlan pl;
    if (d_x_f32 == nullptr || (((uintptr_t)d_x_f32) & 15) != 0 || M * (K / QK_K) * Q4_K_BYTES > 0xffffffffull ||
        !rows_plan(dev, N, K, M, ws.count, pl)) {
        return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
    }
    for (int i = 0; i < ws.count; ++i) {
        if ((((uintptr_t)ws.w[i]) & 15) != 0) {
            return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
        }
    }
    RowsParams p;
    for (int i = 0; i < 3; ++i) {
        const int src = i < ws.count ? i : 0;
        p.w[i] = (const uint8_t *)ws.w[src];
        p.out[i] = ws.out[src];
        p.bias[i] = ws.bias[src];
    }
    p.x = d_x_f32;
    p.K = (uint32_t)K;
    p.M = (uint32_t)M;
    p.nb = (uint32_t)(K / QK_K);
    p.row_bytes = p.nb * Q4_K_BYTES;
    p.rows_per_wg = pl.rows_per_wg;
    p.segs = pl.segs;
    p.seg_blocks = pl.seg_blocks;
    p.rpt = pl.rpt;
    p.rpt_shift = pl.rpt == 1 ? 0 : (pl.rpt == 2 ? 1 : 2);
    p.wstep = pl.consumers / pl.segs;
    p.lag = pl.lag;
    p.loader_rg_step = ((uint32_t)pl.W - pl.consumers) / pl.segs;
    p.pre = pl.pre;
    p.pad_shift = pl.pad_shift;
    p.consumers = pl.consumers;
    p.nslots = pl.nslots;
    p.slot_stride = pl.slot_stride;
    p.xq_stride = pl.xq_stride;
    p.xq_off = pl.xq_off;
    p.ring_off = pl.ring_off;
    p.partial_off = pl.partial_off;
    p.n0 = 0;
    p.bias_is_f16 = ws.bias_dtype == MARMOT_HIP_DTYPE_F16;
    p.bias_first = ws.bias_first ? 1 : 0;
    p.out_is_f16 = out_dtype == MARMOT_HIP_DTYPE_F16;
    p.fault = dev->fault_word;
    p.spin_limit = dev->spin_limit;
    MH_TIMELINE_SET(p, dev);
    set_route("matvec_rows_q4_k_q8_k_fused");
    const int nw = ws.count;
    if (N == 1) {
        return launch_rows<1, 2>(dev, p, pl, nw);
    }
    return launch_rows<2, 1>(dev, p, pl, nw);
}

} // namespace mh

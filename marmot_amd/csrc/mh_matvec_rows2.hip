// Decode matvec for Q4_K weights and ONE fp32 activation row, "resident share" form: one workgroup per compute unit
// owns a contiguous run of weight rows, and that run (up to ~140 KB) is copied into LDS exactly once, byte for byte as
// it lies in memory (no ring, no slot reuse, LDS offset = offset in the share).
//   * Four loader wavefronts (wavefronts 0..3, the first ones the dispatcher starts) request the share front to back
//     with direct-to-LDS loads of 1 KiB per instruction, KiB c by loader c % 4, a bounded number of instructions in
//     flight each. They publish "instructions completed" counters read from their own load counter without waiting.
//   * Twelve consumer wavefronts first request THEIR blocks of the activation row (four 256-value blocks each, the
//     same 1 KiB instructions into a staging area that the LAST weight bytes reuse later), wait on their own load
//     counter, quantize to Q8_K once per workgroup (bit-identical to cpu_matmul_quant_pack_q8_k_f32,
//     matmul_quant_pack.c:106-142), keep their own slice in registers and then take (row, K half) tasks as the
//     loaders' counters say the bytes are there. After the activation row they touch memory only once more: finished
//     rows are collected in LDS and the wavefront that finishes last stores them with one instruction (a store issued
//     under the stream queues behind the loaders' requests and holds its wavefront at the issue stage).
//   * The two K halves of a row meet through ONE LDS exchange per wavefront (no counters, no barrier): the second
//     arriver gets the first one's partial sum back and adds in K order, the same bits whoever comes first.
// What the cycle-counter timeline of this kernel shows (make TIMELINE=1, 4096 x 14336 on MI355X): the first request
// waits ~1 us for the address translation of the weight pages, the share then streams at the rate of a large read
// (24 GB/s per compute unit = 6.1 TB/s), the consumers' vector instructions (~1,500 per workgroup for the activation
// row, ~150 per 4 KiB task) fill ~60 % of the stream time and end 0.5 - 0.9 us after the last byte, and ~1.2 us pass
// between the last wavefront of one launch and the first of the next.
// Arithmetic per block is the reference's cpu_vec_dot_q4_k_q8_k (vec_dot_impl.h:689-732); only the fp32 summation
// order over blocks differs.
#include "mh_rows.h"

namespace mh {

namespace rows2 {
constexpr uint32_t LOADERS = 4;         // two cannot issue fast enough (measured: +0.8 us); 2 or 4: one vector read polls their counters
constexpr uint32_t GROUP_BYTES = 4096;  // the share's LDS region is rounded up to this
// LDS control words
constexpr uint32_t CTRL_LANDED = 0;     // [LOADERS <= 4] load instructions of loader l that have completed
constexpr uint32_t CTRL_X_TAKEN = 4;    // consumer wavefronts that have read their part of the staged activations
constexpr uint32_t CTRL_XQ_DONE = 5;    // consumer wavefronts that have stored their part of the quantized activations
constexpr uint32_t CTRL_DONE = 6;       // consumer wavefronts that have finished their tasks
constexpr uint32_t CTRL_BYTES = 32;
// A bit pattern no fp32 operation produces (a signaling NaN): "no partial sum here yet"
constexpr uint32_t EXCH_EMPTY = 0x7fa5a5a5u;
// Load instructions a loader keeps in flight (the counter holds 63): 48 KiB per compute unit. With less the stream
// starves (8: -0.1 .. +0.1 us, 4: +1.3 us), with more the last window lands as one burst and its products are the
// tail (16: +0.4 us, 60: +1.5 us).
constexpr uint32_t VM_MAX = 12;
// Instructions a loader issues before the workgroup barrier: more would queue behind the first address-translation miss
// and hold the loader, and with it the barrier, for about a microsecond.
constexpr uint32_t PRE_BARRIER = 2;
// flags
constexpr uint32_t F_OUT_F16 = 1, F_BIAS_F16 = 2, F_BIAS_FIRST = 4;
}  // namespace rows2

#if defined(MH_TIMELINE)
#define R2_TIMELINE_PARAM , TimelineArg timeline_arg
#define R2_TIMELINE_LOCAL                                                                                              \
    struct {                                                                                                           \
        TimelineArg timeline;                                                                                          \
    } tl{timeline_arg};
#else
#define R2_TIMELINE_PARAM
#define R2_TIMELINE_LOCAL
#endif

__device__ __forceinline__ void rows2_store(void *out, const void *bias, uint32_t flags, uint32_t row, float v) {
    float bv = 0.0f;
    if (bias != nullptr) {
        bv = (flags & rows2::F_BIAS_F16) ? h2f(((const uint16_t *)bias)[row]) : ((const float *)bias)[row];
    }
    if (!(flags & rows2::F_OUT_F16)) {
        ((float *)out)[row] = bias != nullptr ? v + bv : v;
    } else if (flags & rows2::F_BIAS_FIRST) {
        ((uint16_t *)out)[row] = f2h(bias != nullptr ? v + bv : v);
    } else {
        uint16_t h = f2h(v);
        if (bias != nullptr) {
            h = f2h(h2f(h) + bv);
        }
        ((uint16_t *)out)[row] = h;
    }
}

// shape: pad_shift | rpt_shift << 4 | seg_blocks << 8. Plain scalar arguments, ordered by first use. (Preloading the
// first fourteen words into scalar registers, -mllvm -amdgpu-kernarg-preload-count=14, was measured at 0.03 us per
// launch and is not used: rocprofv3's kernel trace crashes in hipGraphLaunch on graphs that hold such a kernel.)
template <int SEGS>
__global__ __launch_bounds__(1024) void k_matvec_rows2_q4k(const uint8_t *__restrict__ w, const float *__restrict__ x,
                                                          void *__restrict__ out, uint32_t M, uint32_t nb,
                                                          uint32_t rows_per_wg, uint32_t w_off, uint32_t xs_off,
                                                          uint32_t c_wait, uint32_t shape, uint32_t flags,
                                                          const void *__restrict__ bias, uint32_t xq_off, uint32_t *fault,
                                                          uint32_t spin_limit R2_TIMELINE_PARAM) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    R2_TIMELINE_LOCAL
    MH_MARK_DECL
    MH_MARK(tl, 0);
    using namespace rows2;
    const int lane = threadIdx.x & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    uint32_t *const ctrl = (uint32_t *)lds;
    uint32_t *const landed = ctrl + CTRL_LANDED;
    float *const res = (float *)(lds + CTRL_BYTES);                       // [rows of the workgroup] finished rows
    uint32_t *const exch = (uint32_t *)(lds + CTRL_BYTES) + rows_per_wg;  // [rows of the workgroup], SEGS == 2 only
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_u8_t *)lds;
    const uint32_t C = (uint32_t)(blockDim.x >> 6) - LOADERS;
    const uint32_t row_bytes = nb * (uint32_t)Q4_K_BYTES;
    const uint32_t row0 = blockIdx.x * rows_per_wg;
    const uint32_t rows_here = M - row0 < rows_per_wg ? M - row0 : rows_per_wg;
    const uint32_t share = rows_here * row_bytes;  // bytes this workgroup owns: one contiguous run
    const uint32_t lane16 = (uint32_t)lane * 16u;
    SpinGuard guard{spin_limit, fault};

    if (wave < LOADERS) {
        // ---------------------------------------------------------------- loader
        // KiB c of the share is requested by loader c % LOADERS as its (c / LOADERS)-th instruction and lands at LDS
        // offset w_off + 1024 c. At most VM_MAX instructions of a loader are in flight: the memory system serves what
        // is outstanding in no particular order while a wavefront's loads complete in issue order, so with everything
        // requested at once the first KiB would land about as late as the last one.
        const uint32_t l = wave;
        const uint8_t *const wsrc = uniform_pointer(w + (size_t)row0 * row_bytes);
        const uint32_t n_chunks = (share + 1023u) >> 10;
        if (lane == 0) {
            landed[l] = 0;
        }
        uint32_t issued = 0, pub = 0;
        auto issue_chunk = [&](uint32_t c) {
            uint32_t off = c * 1024u + lane16;
            off = off < share ? off : share - 16u;  // the last KiB may be partial: its lanes re-read the last 16 bytes
            dma_set_lds_base(lds_base + w_off + c * 1024u);
            dma16_to_lds<0>(wsrc, off);
            ++issued;
        };
        uint32_t c = l;
        for (; c < n_chunks && c < c_wait && issued < PRE_BARRIER; c += LOADERS) {
            issue_chunk(c);
        }
        MH_MARK(tl, 2);  // loader: first window requested
        __builtin_amdgcn_s_waitcnt(0xc07f);  // landed[l] = 0 is in LDS
        __builtin_amdgcn_s_barrier();        // the control words are initialized: publishing may start
        MH_MARK(tl, 3);  // loader: barrier passed
        // Loads complete in issue order, so `issued - outstanding` instructions have landed; read without waiting.
        auto publish = [&]() {
            const uint32_t done = issued - vmcnt_now();
            if (done != pub) {
#if defined(MH_TIMELINE)
                if (pub == 0) {
                    MH_MARK(tl, 4);  // loader: first instruction landed
                }
                {
                    const uint32_t mine = (n_chunks + LOADERS - 1u - l) / LOADERS;
                    if (pub * 4u < mine && done * 4u >= mine) {
                        MH_MARK(tl, 8);  // loader: a quarter landed
                    }
                    if (pub * 2u < mine && done * 2u >= mine) {
                        MH_MARK(tl, 9);  // loader: half landed
                    }
                    if (pub * 4u < mine * 3u && done * 4u >= mine * 3u) {
                        MH_MARK(tl, 10);  // loader: three quarters landed
                    }
                }
#endif
                pub = done;
                if (lane == 0) {
                    __atomic_store_n(landed + l, done, __ATOMIC_RELAXED);
                }
            }
        };
        bool staging_free = false;
        for (; c < n_chunks; c += LOADERS) {
            if (c >= c_wait && !staging_free) {
                // this KiB overwrites staged activations: every consumer must have taken its part
                while (lds_peek(ctrl + CTRL_X_TAKEN) < C) {
                    if (!guard.spend()) {
                        return;
                    }
                    publish();
                }
                staging_free = true;
                compiler_memory_fence();
            }
            publish();
            while (issued - pub >= VM_MAX) {
                publish();
            }
            issue_chunk(c);
        }
        MH_MARK(tl, 6);  // loader: everything requested
        while (pub < issued) {
            publish();
        }
        MH_MARK(tl, 7);  // loader: everything landed
        MH_MARK_FLUSH(tl);
        return;
    }

    // -------------------------------------------------------------------- consumer
    const uint32_t c = wave - LOADERS;
    const uint32_t ct = threadIdx.x - LOADERS * 64u;  // thread index among the consumers
    const uint32_t pad_shift = shape & 15u, rpt_shift = (shape >> 4) & 15u, seg_blocks = (shape >> 8) & 255u;
    const uint32_t rpt = 1u << rpt_shift;
    // -- 1. the activation row. Consumer c quantizes blocks 4 (c + C it) .. + 3 (256 values each, 16 lanes per block,
    // 16 consecutive values per lane). It requests its blocks itself, first thing, 1 KiB per instruction into the
    // staging area (contiguous lanes: anything else costs the address unit four times as long), and its own load
    // counter says when they have landed (no polling).
    constexpr int XI = 2;
    {
        const uint8_t *const xsrc = uniform_pointer((const uint8_t *)x);
        const uint32_t piece_off = lane16;
#pragma unroll
        for (int it = 0; it < XI; ++it) {
            const uint32_t b0 = 4u * (c + (uint32_t)it * C);
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                if (b0 + j < nb) {
                    dma_set_lds_base(lds_base + xs_off + (b0 + j) * 1024u);
                    dma16_to_lds<0>(xsrc, (b0 + j) * 1024u + piece_off);
                }
            }
        }
    }
    if (SEGS == 2) {
        for (uint32_t i = ct; i < rows_per_wg; i += C * 64u) {
            exch[i] = EXCH_EMPTY;
        }
    }
    if (ct == 0) {
        ctrl[CTRL_X_TAKEN] = 0;
        ctrl[CTRL_XQ_DONE] = 0;
        ctrl[CTRL_DONE] = 0;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    MH_MARK(tl, 1);  // consumer: barrier passed
    float xv[XI][16];
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's blocks of the activation row are in LDS
    compiler_memory_fence();
    MH_MARK(tl, 2);  // consumer: own activations landed
#pragma unroll
    for (int it = 0; it < XI; ++it) {
        const uint32_t qb = 4u * (c + (uint32_t)it * C) + ((uint32_t)lane >> 4);
        if (qb < nb) {
            // Lane q's 16 values are the 16-byte pieces 4 q .. 4 q + 3 of the block. Read in that order, lanes q, q + 4,
            // q + 8, q + 12 would hit the same banks; lane q starts with piece 4 q + q / 4 instead, so the 16 lanes of
            // a block cover 256 distinct bytes per read. The quantizer is told the rotation and stores its four output
            // words where they belong.
            const uint32_t q = (uint32_t)lane & 15u, rot = q >> 2;
            const uint8_t *src = lds + xs_off + (size_t)qb * 1024u + q * 64u;
            const float4 a0 = *(const float4 *)(src + 16u * (rot & 3u)), a1 = *(const float4 *)(src + 16u * ((rot + 1u) & 3u)),
                         a2 = *(const float4 *)(src + 16u * ((rot + 2u) & 3u)), a3 = *(const float4 *)(src + 16u * ((rot + 3u) & 3u));
            xv[it][0] = a0.x, xv[it][1] = a0.y, xv[it][2] = a0.z, xv[it][3] = a0.w;
            xv[it][4] = a1.x, xv[it][5] = a1.y, xv[it][6] = a1.z, xv[it][7] = a1.w;
            xv[it][8] = a2.x, xv[it][9] = a2.y, xv[it][10] = a2.z, xv[it][11] = a2.w;
            xv[it][12] = a3.x, xv[it][13] = a3.y, xv[it][14] = a3.z, xv[it][15] = a3.w;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // the values are in registers: the staging area may be overwritten
    if (lane == 0) {
        __atomic_fetch_add(ctrl + CTRL_X_TAKEN, 1u, __ATOMIC_RELAXED);
    }
    MH_MARK(tl, 3);  // consumer: own activations in registers
    uint8_t *const xq = lds + xq_off;
#pragma unroll
    for (int it = 0; it < XI; ++it) {
        const uint32_t qb = 4u * (c + (uint32_t)it * C) + ((uint32_t)lane >> 4), qi = (uint32_t)lane & 15u;
        if (qb < nb) {
            uint4 q;
            int bsum;
            float d;
            q8k_quantize16(xv[it], (int)qi, q, bsum, d, (int)(qi >> 2));
            // 16-byte pieces of a block are XOR-swizzled by the block index: conflict-free for these stores (16 lanes,
            // one block) and for the strided fetch below (16 lanes, 16 blocks, one piece index). The lane's four words
            // are in the rotated order of its reads.
            uint32_t *dst = (uint32_t *)(xq + (size_t)qb * QK_K + 16u * (qi ^ (qb & 15u)));
            const uint32_t rot = qi >> 2;
            dst[rot & 3u] = q.x;
            dst[(rot + 1u) & 3u] = q.y;
            dst[(rot + 2u) & 3u] = q.z;
            dst[(rot + 3u) & 3u] = q.w;
            ((int16_t *)(xq + (size_t)nb * QK_K))[qb * 16 + qi] = (int16_t)bsum;
            if (qi == 0) {
                ((float *)(xq + (size_t)nb * (QK_K + 32)))[qb] = d;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    if (lane == 0) {
        __atomic_fetch_add(ctrl + CTRL_XQ_DONE, 1u, __ATOMIC_RELAXED);
    }
    MH_MARK(tl, 4);  // consumer: own part quantized
    if (!lds_wait_at_least(ctrl + CTRL_XQ_DONE, C, guard)) {
        return;
    }
    MH_MARK(tl, 5);  // consumer: all parts quantized

    // -- 2. this lane's slice: a lane owns half a block (sub-blocks 0..3 or 4..7) at block position b of its K segment
    const uint32_t part = (uint32_t)lane >> 5;
    const uint32_t slot = (uint32_t)lane & 31u;
    const uint32_t r_in = slot >> pad_shift;
    const uint32_t b = slot & ((1u << pad_shift) - 1u);
    const uint32_t seg = SEGS == 1 ? 0u : (c & 1u);
    const uint32_t seg_first = seg * seg_blocks;
    const uint32_t seg_nb = nb - seg_first < seg_blocks ? nb - seg_first : seg_blocks;
    const uint32_t b_global = seg_first + b;
    const bool lane_valid = b < seg_nb && r_in < rpt;
    uint4 a[8];
    int bs[4];
    float ad = 0.0f;
    if (lane_valid) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t piece = part * 8u + (uint32_t)i;
            a[i] = *(const uint4 *)(xq + (size_t)b_global * QK_K + 16u * (piece ^ (b_global & 15u)));
        }
        const int16_t *bsp = (const int16_t *)(xq + (size_t)nb * QK_K) + b_global * 16 + part * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t two = *(const uint32_t *)(bsp + 2 * j);
            bs[j] = (int)(int16_t)(two & 0xffffu) + (int)(int16_t)(two >> 16);
        }
        ad = ((const float *)(xq + (size_t)nb * (QK_K + 32)))[b_global];
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[i] = make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            bs[j] = 0;
        }
    }

    // -- 3. tasks, as their bytes land: row group rg = c / SEGS + i * (C / SEGS), K segment c % SEGS
    const uint32_t groups = (rows_here + rpt - 1u) >> rpt_shift;
    const uint32_t task_bytes = SEGS == 1 ? rpt * row_bytes : seg_nb * (uint32_t)Q4_K_BYTES;
    const uint32_t lane_off = (SEGS == 1 ? r_in * row_bytes : 0u) + b * (uint32_t)Q4_K_BYTES;
    // lanes of the low half of a block take scale bytes 0..3 / min bytes 4..7 as they are; the high half builds its
    // four from the nibbles of bytes 8..11 and the top bits of the others (get_scale_min_k4, kquant_common.h:29-37)
    const uint32_t keep_lo = part != 0 ? 0u : 0x3f3f3f3fu;
    const uint32_t keep_hi = part != 0 ? 0xffffffffu : 0u;
    MH_MARK(tl, 6);  // consumer: slice in registers, task loop starts
    for (uint32_t rg = c / SEGS; rg < groups; rg += C / SEGS) {
        const uint32_t first = SEGS == 1 ? rg * rpt * row_bytes : rg * row_bytes + seg_first * (uint32_t)Q4_K_BYTES;
        uint32_t last = first + task_bytes - 1u;
        last = last < share ? last : share - 1u;
        // KiB (last >> 10) and everything before it must have landed: loader l has then completed the instructions
        // of all its KiBs up to that one
        {
            const uint32_t c_last = last >> 10;
            typedef uint32_t u32xl __attribute__((ext_vector_type(LOADERS)));
            for (;;) {
                const u32xl have = *(volatile const u32xl *)landed;
                bool ok = true;
#pragma unroll
                for (uint32_t l = 0; l < LOADERS; ++l) {
                    ok = ok && have[l] >= (c_last + LOADERS - l) / LOADERS;
                }
                if (__builtin_amdgcn_readfirstlane((int)ok)) {
                    break;
                }
                if (!guard.spend()) {
                    return;
                }
            }
            compiler_memory_fence();
        }
#if defined(MH_TIMELINE)
        if (rg == c / SEGS) {
            MH_MARK(tl, 7);  // consumer: first task's bytes there
        }
        if (rg + C / SEGS >= groups) {
            MH_MARK(tl, 9);  // consumer: last task's bytes there
        }
#endif
        float v = 0.0f;
        if (lane_valid && first + lane_off < share) {
            const uint8_t *blk = lds + w_off + first + lane_off;
            const uint4 hdr = *(const uint4 *)blk;
            uint4 q[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                q[i] = *(const uint4 *)(blk + 16 + part * 64u + 16 * i);
            }
            const float wd = h2f((uint16_t)(hdr.x & 0xffffu));
            const float wdmin = h2f((uint16_t)(hdr.x >> 16));
            const uint32_t sc4 = (hdr.y & keep_lo) | (((hdr.w & 0x0f0f0f0fu) | ((hdr.y >> 2) & 0x30303030u)) & keep_hi);
            const uint32_t mn4 = (hdr.z & keep_lo) | ((((hdr.w >> 4) & 0x0f0f0f0fu) | ((hdr.z >> 2) & 0x30303030u)) & keep_hi);
            int isum = 0, msum = 0;
#pragma unroll
            for (int gq = 0; gq < 2; ++gq) {
                uint4 lo0, hi0, lo1, hi1;
                lo0.x = q[2 * gq].x & 0x0f0f0f0fu, hi0.x = (q[2 * gq].x >> 4) & 0x0f0f0f0fu;
                lo0.y = q[2 * gq].y & 0x0f0f0f0fu, hi0.y = (q[2 * gq].y >> 4) & 0x0f0f0f0fu;
                lo0.z = q[2 * gq].z & 0x0f0f0f0fu, hi0.z = (q[2 * gq].z >> 4) & 0x0f0f0f0fu;
                lo0.w = q[2 * gq].w & 0x0f0f0f0fu, hi0.w = (q[2 * gq].w >> 4) & 0x0f0f0f0fu;
                lo1.x = q[2 * gq + 1].x & 0x0f0f0f0fu, hi1.x = (q[2 * gq + 1].x >> 4) & 0x0f0f0f0fu;
                lo1.y = q[2 * gq + 1].y & 0x0f0f0f0fu, hi1.y = (q[2 * gq + 1].y >> 4) & 0x0f0f0f0fu;
                lo1.z = q[2 * gq + 1].z & 0x0f0f0f0fu, hi1.z = (q[2 * gq + 1].z >> 4) & 0x0f0f0f0fu;
                lo1.w = q[2 * gq + 1].w & 0x0f0f0f0fu, hi1.w = (q[2 * gq + 1].w >> 4) & 0x0f0f0f0fu;
                const int s0 = (int)((sc4 >> (16 * gq)) & 0xffu), s1 = (int)((sc4 >> (16 * gq + 8)) & 0xffu);
                const int m0 = (int)((mn4 >> (16 * gq)) & 0xffu), m1 = (int)((mn4 >> (16 * gq + 8)) & 0xffu);
                // values 64 g + 0..31 sit in the low nibbles, 64 g + 32..63 in the high nibbles of the same bytes
                const int dl = dot16r(lo1, a[4 * gq + 1], dot16r(lo0, a[4 * gq], 0));
                const int dh = dot16r(hi1, a[4 * gq + 3], dot16r(hi0, a[4 * gq + 2], 0));
                isum += __mul24(s0, dl) + __mul24(s1, dh);
                msum += __mul24(m0, bs[2 * gq]) + __mul24(m1, bs[2 * gq + 1]);
            }
            v = (ad * wd) * (float)isum - (ad * wdmin) * (float)msum;
        }
#if defined(MH_TIMELINE)
        asm volatile("" ::"v"(v));
        if (rg == c / SEGS) {
            MH_MARK(tl, 8);  // consumer: first task's products done
        }
#endif
        v = row16_sum(v);
        const int iv = __builtin_bit_cast(int, v);
        const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
        const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
        const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
        const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
        // Finished rows go to LDS, not to memory: a store issued under the stream queues behind the loaders' requests
        // and holds its wavefront at the issue stage. The wavefront that finishes last stores all rows of the
        // workgroup with one instruction, when nothing is in flight any more.
        if (SEGS == 1) {
            if (rpt == 2) {
                // lanes 0..15 and 32..47 hold row 0 of the task, 16..31 and 48..63 row 1
                if (lane < 2) {
                    res[rg * 2u + (uint32_t)lane] = lane == 0 ? r0 + r2 : r1 + r3;
                }
            } else if (lane == 0) {
                res[rg] = (r0 + r1) + (r2 + r3);
            }
        } else if (lane == 0) {
            // The K halves of a row meet here: the first arriver leaves its partial sum, the second takes it and adds
            // in K order (the same bits whoever comes first).
            const float mine = (r0 + r1) + (r2 + r3);
            const uint32_t other = __atomic_exchange_n(exch + rg, __float_as_uint(mine), __ATOMIC_RELAXED);
            if (other != EXCH_EMPTY) {
                const float o = __uint_as_float(other);
                res[rg] = seg == 0 ? mine + o : o + mine;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // this wavefront's rows are in LDS
    MH_MARK(tl, 10);  // consumer: last task done
    uint32_t before = 0;
    if (lane == 0) {
        before = __atomic_fetch_add(ctrl + CTRL_DONE, 1u, __ATOMIC_RELAXED);
    }
    if ((uint32_t)__builtin_amdgcn_readfirstlane((int)before) == C - 1u) {
        for (uint32_t r = (uint32_t)lane; r < rows_here; r += 64u) {
            const float v = __builtin_bit_cast(float, __atomic_load_n((const uint32_t *)res + r, __ATOMIC_RELAXED));
            rows2_store(out, bias, flags, row0 + r, v);
        }
    }
    MH_MARK(tl, 11);  // consumer: leaves
    MH_MARK_FLUSH(tl);
}

// Launch plan; false when the shape is outside what the kernel covers.
struct Rows2Plan {
    int segs;
    uint32_t rows_per_wg, grid, pad_shift, rpt_shift, seg_blocks, xq_off, w_off, xs_off, c_wait, consumers;
    size_t lds;
};

static bool rows2_plan(const marmot_hip_device *dev, size_t K, size_t M, Rows2Plan &pl) {
    using namespace rows2;
    if (K % QK_K != 0 || M == 0) {
        return false;
    }
    const uint32_t nb = (uint32_t)(K / QK_K);
    const size_t weight_bytes = M * (size_t)nb * Q4_K_BYTES;
    // below ~16 MB the ring form of the row kernel is faster (measured at 4096 x 4096: 4.75 against 4.86 us)
    if (nb == 0 || nb > 64 || weight_bytes < ((size_t)16 << 20) || weight_bytes > 0xffffffffull) {
        return false;
    }
    const uint32_t cus = (uint32_t)dev->props.multiProcessorCount;
    const uint32_t row_bytes = nb * Q4_K_BYTES;
    uint32_t rpt;
    if (nb <= 32) {
        pl.segs = 1;
        pl.seg_blocks = nb;
        pl.pad_shift = nb <= 16 ? 4 : 5;
        rpt = 32u >> pl.pad_shift;
    } else {
        pl.segs = 2;
        pl.seg_blocks = (nb + 1) / 2;
        pl.pad_shift = 5;
        rpt = 1;
    }
    pl.rpt_shift = rpt == 1 ? 0 : 1;
    uint32_t rows = (uint32_t)((M + cus - 1) / cus);
    rows = ((rows + rpt - 1) / rpt) * rpt;
    pl.rows_per_wg = rows;
    pl.grid = (uint32_t)((M + rows - 1) / rows);
    pl.consumers = 16u - LOADERS;
    if (nb > 2u * 4u * pl.consumers) {  // a consumer quantizes four blocks per pass, two passes at most
        return false;
    }
    const uint32_t budget = 160u * 1024u;
    const uint32_t exch_bytes = ((rows * 4u * (pl.segs == 2 ? 2u : 1u)) + 15u) & ~15u;  // finished rows (+ exchange words)
    pl.xq_off = CTRL_BYTES + exch_bytes;
    const uint32_t xq_bytes = (nb * (QK_K + 32 + 4) + 15u) & ~15u;
    pl.w_off = (pl.xq_off + xq_bytes + 1023u) & ~1023u;
    const uint32_t wregion = ((rows * row_bytes + GROUP_BYTES - 1) / GROUP_BYTES) * GROUP_BYTES;
    const uint32_t x_bytes = nb * 1024u;
    if (pl.w_off + wregion > budget || pl.w_off + x_bytes > budget) {
        return false;
    }
    // staged activations: behind the weight region when that fits, else over its tail (the loaders wait for the
    // consumers to have taken them before they request those weight bytes)
    pl.xs_off = pl.w_off + wregion + x_bytes <= budget ? pl.w_off + wregion : budget - x_bytes;
    pl.c_wait = (pl.xs_off - pl.w_off) / 1024u;  // first KiB of the share that lands on staged activations
    const uint32_t end = pl.xs_off + x_bytes > pl.w_off + wregion ? pl.xs_off + x_bytes : pl.w_off + wregion;
    pl.lds = end;
    return true;
}

// Tries the resident-share kernel for one Q4_K weight and one fp32 activation row. Returns
// MARMOT_HIP_ERROR_NOT_IMPLEMENTED (error text untouched) when the shape is not covered.
int launch_matvec_rows2_q4k(marmot_hip_device *dev, const WeightSet &ws, const float *d_x_f32, size_t N, size_t K,
                            size_t M, int out_dtype) {
    Rows2Plan pl;
    if (N != 1 || ws.count != 1 || d_x_f32 == nullptr || (((uintptr_t)d_x_f32) & 15) != 0 ||
        (((uintptr_t)ws.w[0]) & 15) != 0 || !rows2_plan(dev, K, M, pl)) {
        return MARMOT_HIP_ERROR_NOT_IMPLEMENTED;
    }
    uint32_t flags = 0;
    flags |= out_dtype == MARMOT_HIP_DTYPE_F16 ? rows2::F_OUT_F16 : 0u;
    flags |= ws.bias_dtype == MARMOT_HIP_DTYPE_F16 ? rows2::F_BIAS_F16 : 0u;
    flags |= ws.bias_first ? rows2::F_BIAS_FIRST : 0u;
    const uint32_t shape = pl.pad_shift | (pl.rpt_shift << 4) | (pl.seg_blocks << 8);
    const dim3 grid(pl.grid), block((pl.consumers + rows2::LOADERS) * 64u);
    set_route("matvec_rows2_q4_k_q8_k_fused");
#if defined(MH_TIMELINE)
    const TimelineArg tl{dev->timeline, dev->timeline_words};
#define R2_TIMELINE_VALUE , tl
#else
#define R2_TIMELINE_VALUE
#endif
    if (pl.segs == 1) {
        MH_TRY(allow_large_lds(dev, (const void *)k_matvec_rows2_q4k<1>));
        hipLaunchKernelGGL((k_matvec_rows2_q4k<1>), grid, block, pl.lds, dev->stream, (const uint8_t *)ws.w[0], d_x_f32,
                           ws.out[0], (uint32_t)M, (uint32_t)(K / QK_K), pl.rows_per_wg, pl.w_off, pl.xs_off, pl.c_wait,
                           shape, flags, ws.bias[0], pl.xq_off, dev->fault_word, dev->spin_limit R2_TIMELINE_VALUE);
    } else {
        MH_TRY(allow_large_lds(dev, (const void *)k_matvec_rows2_q4k<2>));
        hipLaunchKernelGGL((k_matvec_rows2_q4k<2>), grid, block, pl.lds, dev->stream, (const uint8_t *)ws.w[0], d_x_f32,
                           ws.out[0], (uint32_t)M, (uint32_t)(K / QK_K), pl.rows_per_wg, pl.w_off, pl.xs_off, pl.c_wait,
                           shape, flags, ws.bias[0], pl.xq_off, dev->fault_word, dev->spin_limit R2_TIMELINE_VALUE);
    }
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

} // namespace mh

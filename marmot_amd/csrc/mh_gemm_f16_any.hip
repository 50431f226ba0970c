// Prefill GEMM for fp16 activations and EVERY weight format but Q4_K (which has the kernels of mh_gemm.hip), on
// v_mfma_f32_32x32x16_f16 with fp32 accumulation.
//
// Arithmetic. The reference's direct fp16 dots (cpu_vec_dot_*_f16, vec_dot_impl.h:240-450 for the 32-value formats,
// :866-1128 for the K-quants) decode a weight to fp32 and add w * (float)x in fp32, element by element. The weight they
// see (direct_f16_weight<KIND>, mh_dequant.h: the reference's own index patterns, which for Q2_K / Q3_K / Q5_K / Q6_K
// differ from its dequantizers) is, in every format, scale * integer + offset with a scale and an offset that are
// constant over a round of 32 values or more (Q6_K and Q2_K, as those dots decode them: over 128; Q3_K's group scales
// go into the integer). Here the INTEGER is the fp16 operand (exact; its products with fp16 activations are exact in
// fp32), the scale is applied to the span's product in fp32 as d is in the Q4_K kernels, and the offset to the span's
// sum of activations, which one more matrix instruction against ones delivers. The result differs from exact
// arithmetic by the fp32 accumulation and two roundings per span, less than the reference's own sequential sum.
//
// Tiling. A workgroup of four wavefronts owns 128 weight rows x 64 tokens and walks K in rounds of 32 values (one block
// of the 32-value formats, an eighth of a K-quant block). Per round every thread turns 16 weights of one row (the same
// 16-value half of the round for all rows; the bytes are requested a round earlier) into fp16 integers and stores them
// into one of two LDS stages in MFMA operand order; wavefront c then multiplies its 32 rows with the 64 tokens: two
// K-steps x two token tiles = four matrix instructions (eight with an offset); the activations come through LDS in
// stages of four rounds (whole 256-byte runs of a token's row per 16 lanes: a lane-per-token gather of 16 bytes costs
// the compute unit's address unit 32 cache lines per instruction and was the bound of the first form, 102 us whatever
// the format). One barrier per round. K is split across workgroups when the tiles do not fill the chip; the partial
// sums meet in k_gemm_reduce.
#include <type_traits>

#include "mh_common.h"
#include "mh_dequant.h"

namespace mh {

typedef _Float16 fa_half8 __attribute__((ext_vector_type(8)));
typedef float fa_floatx16 __attribute__((ext_vector_type(16)));

constexpr int FA_TOK = 64;
constexpr int FA_WROWS = 128;
constexpr int FA_GROUP = 256;                          // threads of one K group: four wavefronts x 32 rows
constexpr int FA_THREADS = 2 * FA_GROUP;               // two K groups take alternate stages of the workgroup's rounds
constexpr int FA_ROUND = 32;                          // values of K per round
constexpr int FA_XROUNDS = 4;                         // rounds per activation stage (128 values of K)
constexpr int FA_XSTAGE = FA_TOK * FA_XROUNDS * FA_ROUND * 2;   // 16,384
constexpr int FA_OUT_PITCH = FA_WROWS + 4;             // floats per token of the output tile in LDS
// every token count (14336 x 4096 at 1 / 8 rows: Q8_0 30.4 / 30.6 us, Q6_K 28.2 / 28.4 us; the fp16 matvec, four rows
// at a time, 40.3 / 117 us and 49.2 / 133 us; only 4096 x 4096 at one row is 1.5 us behind it)
constexpr int FA_MIN_TOKENS = 1;
static_assert(FA_XROUNDS == 4, "the stage loops are written out for four rounds");

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

// Four bytes (each below 256 - the fp16 integers 1024 .. 1279 are exact) as two words of fp16 pairs holding byte - OFF
// + 1024: (0x64, byte) as fp16 bits is 1024 + byte.
template <int OFF>
__device__ __forceinline__ void any_bytes_to_f16(uint32_t bytes, uint32_t &lo, uint32_t &hi) {
    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
    const h2_t off = {(_Float16)(-(float)OFF), (_Float16)(-(float)OFF)};
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, bytes, 0x04010400u);
    const uint32_t b = __builtin_amdgcn_perm(0x64646464u, bytes, 0x04030402u);
    lo = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2_t, a) + off);
    hi = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2_t, b) + off);
}

// Every format's weight is an integer times a scale that is constant over a round of 32 values or more, plus (Q4_1,
// Q5_1, Q5_K, Q2_K) an offset that is constant over the same span: the integer is the exact fp16 operand, the scale goes
// onto the span's product like d in the Q4_K kernels, and the offset multiplies the span's sum of activations, which a
// matrix instruction against a row of ones delivers in the layout of the products.
template <int KIND>
struct AnyInt {
    static constexpr bool HAS_MIN = KIND == MARMOT_HIP_KIND_Q4_1 || KIND == MARMOT_HIP_KIND_Q5_1 ||
                                    KIND == MARMOT_HIP_KIND_Q5_K || KIND == MARMOT_HIP_KIND_Q2_K;
    // rounds that share a scale (and an offset): Q6_K and Q2_K as the reference's fp16 dots decode them, 128 values;
    // Q3_K's six-bit group scales (per 16 values) are multiplied into the integer operand, which leaves d per block,
    // applied per stage of four rounds (a K group sees every other stage)
    static constexpr int SCALE_ROUNDS =
        (KIND == MARMOT_HIP_KIND_Q6_K || KIND == MARMOT_HIP_KIND_Q2_K || KIND == MARMOT_HIP_KIND_Q3_K) ? 4 : 1;
    static_assert(SCALE_ROUNDS == 1 || SCALE_ROUNDS == FA_XROUNDS, "a span of rounds is a stage");
    // LDS: two activation stages; the output tile reuses them
    static constexpr int LDS_BYTES = 4 * FA_XSTAGE;  // two activation stages per K group; the output tile reuses them
    static_assert(FA_TOK * FA_OUT_PITCH * 4 <= LDS_BYTES, "the output tile reuses the stages");
};

// The 16 weights a thread handles per round, in two steps so that the bytes can be requested a round before they are
// needed: fetch(block, v) issues the loads for values v .. v + 15 of the block (v a multiple of 16), ints() turns them
// into the 16 integers as exact fp16 values (two per word, in order), the scale they share and their offset. The
// weight of direct_f16_weight<KIND> (mh_dequant.h) is scale * integer + offset, up to that function's own roundings.
template <int KIND>
struct AnyRaw;

// Blocks of 18, 22, 34, 110 and 210 bytes put their fields at addresses that are multiples of 2, not of 4, in every
// other block, and a vector load from such an address is slow (512 tokens x 4096 x 4096: Q4_0, whose nibbles start 2
// bytes into an 18-byte block, 57.7 us; Q4_1, whose nibbles start 4 bytes into a 20-byte block, 43.5 us with twice
// the matrix instructions). Any16 fetches 16 bytes from the multiple of 4 below and brings the last two bytes
// separately; the bytes are put together when they are used. No byte outside [p - 2, p + 16) is read. (For the 8- and
// 4-byte fields of Q6_K the second instruction cost more than the misalignment: 59.7 -> 70.5 us.)
typedef uint32_t any_u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
struct Any16 {  // 16 bytes at an even address
    any_u32x4_a4 d;
    uint16_t t;
    uint16_t mis;
    __device__ __forceinline__ void fetch(const uint8_t *p) {
        mis = (uint16_t)((uintptr_t)p & 2u);
        const uint8_t *base = p - mis;
        d = *(const any_u32x4_a4 *)base;
        t = *(const uint16_t *)(base + (mis ? 16 : 14));
    }
    __device__ __forceinline__ uint4 get() const {
        const uint32_t sh = 8u * mis;  // 0 or 16
        return make_uint4(__builtin_amdgcn_alignbit(d.y, d.x, sh), __builtin_amdgcn_alignbit(d.z, d.y, sh),
                          __builtin_amdgcn_alignbit(d.w, d.z, sh), mis ? (d.w >> 16) | ((uint32_t)t << 16) : d.w);
    }
};
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q8_0> {
    Any16 q16;
    uint16_t s;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        q16.fetch(b + 2 + v);
    }
    __device__ __forceinline__ void fetch_scale(const uint8_t *b, int) {
        __builtin_memcpy(&s, b, 2);
    }
    __device__ __forceinline__ void ints(uint32_t (&h)[8], float &scale, float &offset) const {
        scale = h2f(s);
        offset = 0.0f;
        const uint4 q = q16.get();
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            any_bytes_to_f16<1152>(qw[e] ^ 0x80808080u, h[2 * e], h[2 * e + 1]);  // byte + 128, then - 128
        }
    }
};
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q8_1> {  // scale, the carried sum (unused), 32 codes
    uint4 q;
    uint16_t s;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        __builtin_memcpy(&q, b + 4 + v, 16);
    }
    __device__ __forceinline__ void fetch_scale(const uint8_t *b, int) {
        __builtin_memcpy(&s, b, 2);
    }
    __device__ __forceinline__ void ints(uint32_t (&h)[8], float &scale, float &offset) const {
        scale = h2f(s);
        offset = 0.0f;
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            any_bytes_to_f16<1152>(qw[e] ^ 0x80808080u, h[2 * e], h[2 * e + 1]);
        }
    }
};

// The 32-value formats with nibbles: byte i of qs holds value i (low nibble) and value 16 + i (high nibble); Q5_0 / Q5_1
// keep the fifth bit of value i in bit i of a 32-bit word before qs. HDR: bytes before that word / before qs.
template <int HDR, bool FIFTH, bool MIN, int CENTRE>
struct AnyRawNibbles {
    // MIN formats have blocks of 20 / 24 bytes: every field on a multiple of 4, plain vector loads. The others (18 /
    // 22 bytes) take the nibbles through Any16.
    Any16 q16;
    any_u32x4_a4 qa;
    uint32_t qh, sm;
    int high;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        if constexpr (MIN) {
            sm = *(const uint32_t *)b;  // scale, min
            qa = *(const any_u32x4_a4 *)(b + HDR + (FIFTH ? 4 : 0));
        } else {
            uint16_t s;
            __builtin_memcpy(&s, b, 2);
            sm = s;
            q16.fetch(b + HDR + (FIFTH ? 4 : 0));
        }
        if constexpr (FIFTH) {
            __builtin_memcpy(&qh, b + HDR, 4);
        }
        high = v >= 16;
    }
    __device__ __forceinline__ void fetch_scale(const uint8_t *, int) {}
    __device__ __forceinline__ void ints(uint32_t (&h)[8], float &scale, float &offset) const {
        scale = h2f((uint16_t)(sm & 0xffffu));
        offset = MIN ? h2f((uint16_t)(sm >> 16)) : 0.0f;
        uint4 q;
        if constexpr (MIN) {
            q = make_uint4(qa.x, qa.y, qa.z, qa.w);
        } else {
            q = q16.get();
        }
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
        const uint32_t hbits = FIFTH ? (high ? qh >> 16 : qh) : 0u;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            uint32_t val = (high ? qw[e] >> 4 : qw[e]) & 0x0f0f0f0fu;
            if constexpr (FIFTH) {  // bits 4 e .. 4 e + 3 to bit 4 of bytes 0 .. 3
                val |= ((((hbits >> (4 * e)) & 0xfu) * 0x00204081u) & 0x01010101u) << 4;
            }
            any_bytes_to_f16<1024 + CENTRE>(val, h[2 * e], h[2 * e + 1]);
        }
    }
};
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q4_0> : AnyRawNibbles<2, false, false, 8> {};   // (nibble - 8) * d
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q4_1> : AnyRawNibbles<4, false, true, 0> {};    // nibble * d + m
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q5_0> : AnyRawNibbles<2, true, false, 16> {};   // (value - 16) * d
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q5_1> : AnyRawNibbles<4, true, true, 0> {};     // value * d + m

template <>
struct AnyRaw<MARMOT_HIP_KIND_Q6_K> {
    uint2 ql;  // (8 and 4 bytes at even addresses: plain loads; one more instruction each cost more than it saved)
    uint32_t qh;
    int8_t sc;
    uint16_t d;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        __builtin_memcpy(&ql, b + (v >> 1), 8);
        __builtin_memcpy(&qh, b + 128 + (v >> 2), 4);
    }
    __device__ __forceinline__ void fetch_scale(const uint8_t *b, int v) {  // one scale per 128 values
        sc = (int8_t)b[192 + (v >> 7)];
        __builtin_memcpy(&d, b + 208, 2);
    }
    __device__ __forceinline__ void ints(uint32_t (&h)[8], float &scale, float &offset) const {
        scale = h2f(d) * (float)sc;
        offset = 0.0f;
        // value i: nibble i % 2 of byte i / 2 of ql, bits 2 (i % 4) .. + 1 of byte i / 4 of qh as bits 4..5
        const uint32_t lw[2] = {ql.x, ql.y};
        // the high pairs of values 4 b + t, already at bits 4..5, in byte b of plane t
        const uint32_t pl[4] = {(qh << 4) & 0x30303030u, (qh << 2) & 0x30303030u, qh & 0x30303030u,
                                (qh >> 2) & 0x30303030u};
#pragma unroll
        for (int k = 0; k < 4; ++k) {  // values 4 k .. 4 k + 3: bytes 2 (k % 2), 2 (k % 2) + 1 of word k / 2 of ql
            const uint32_t even = lw[k >> 1] & 0x0f0f0f0fu, odd = (lw[k >> 1] >> 4) & 0x0f0f0f0fu;
            // [even byte 2 (k % 2), odd same, even next, odd next]; perm selectors 0..3 = second operand, 4..7 = first
            const uint32_t nibs = __builtin_amdgcn_perm(odd, even, (k & 1) ? 0x07030602u : 0x05010400u);
            // [plane 0 byte k, plane 1 byte k, plane 2 byte k, plane 3 byte k]
            const uint32_t sel = 0x04000400u + 0x01010101u * (uint32_t)k;
            const uint32_t p01 = __builtin_amdgcn_perm(pl[1], pl[0], sel);  // bytes (p0[k], p1[k], p0[k], p1[k])
            const uint32_t p23 = __builtin_amdgcn_perm(pl[3], pl[2], sel);
            const uint32_t his = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
            any_bytes_to_f16<1056>(nibs | his, h[2 * k], h[2 * k + 1]);  // 6-bit value - 32
        }
    }
};

// Q5_K as cpu_vec_dot_q5_k_f16 reads it (direct_f16_weight_q5_k): sub-block j = v / 32 has the Q4_K scale / min pair
// j; value l of it is nibble j % 2 of qs[32 (j / 2) + l] plus 16 x bit 0 of the byte 8 (j / 2) + l + 32 (j % 2) behind
// the start of qh (block bytes 16 ..; for most values a byte of qs).
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q5_K> {
    uint4 q, hb;
    uint32_t s0, s1, s2, dd;
    int j;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        j = v >> 5;
        const int l0 = v & 31, g = j >> 1;
        __builtin_memcpy(&dd, b, 4);
        __builtin_memcpy(&s0, b + 4, 4);
        __builtin_memcpy(&s1, b + 8, 4);
        __builtin_memcpy(&s2, b + 12, 4);
        __builtin_memcpy(&hb, b + 16 + 8 * g + l0 + 32 * (j & 1), 16);
        __builtin_memcpy(&q, b + 48 + 32 * g + l0, 16);
    }
    __device__ __forceinline__ void fetch_scale(const uint8_t *, int) {}
    __device__ __forceinline__ void ints(uint32_t (&h)[8], float &scale, float &offset) const {
        // scales[j], scales[j + 4] (j < 4) or scales[j + 4], scales[j - 4], scales[j] (j >= 4): byte j % 4 of a word
        const int sh = 8 * (j & 3);
        const uint32_t a = (s0 >> sh) & 0xffu, b = (s1 >> sh) & 0xffu, c = (s2 >> sh) & 0xffu;
        const uint32_t sc = j < 4 ? (a & 63u) : ((c & 0xfu) | ((a >> 6) << 4));
        const uint32_t mn = j < 4 ? (b & 63u) : ((c >> 4) | ((b >> 6) << 4));
        scale = h2f((uint16_t)(dd & 0xffffu)) * (float)sc;
        offset = -(h2f((uint16_t)(dd >> 16)) * (float)mn);
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w}, hw[4] = {hb.x, hb.y, hb.z, hb.w};
        const int shift = (j & 1) ? 4 : 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t val = ((qw[e] >> shift) & 0x0f0f0f0fu) | ((hw[e] & 0x01010101u) << 4);
            any_bytes_to_f16<1024>(val, h[2 * e], h[2 * e + 1]);
        }
    }
};

// Q2_K as cpu_vec_dot_q2_k_f16 reads it (direct_f16_weight_q2_k): one scale / min pair per 128 values (scales[v / 128]),
// value v in bits 2 (v % 4) .. + 1 of qs[v / 4].
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q2_K> {
    uint32_t q, dd;
    uint8_t sc;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        __builtin_memcpy(&q, b + 16 + (v >> 2), 4);
    }
    __device__ __forceinline__ void fetch_scale(const uint8_t *b, int v) {  // one scale / min pair per 128 values
        sc = b[v >> 7];
        __builtin_memcpy(&dd, b + 80, 4);
    }
    __device__ __forceinline__ void ints(uint32_t (&h)[8], float &scale, float &offset) const {
        scale = h2f((uint16_t)(dd & 0xffffu)) * (float)(sc & 0xFu);
        offset = -(h2f((uint16_t)(dd >> 16)) * (float)(sc >> 4));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t b = (q >> (8 * e)) & 0xffu;  // pair k of the byte to byte k: b << 6 k puts bit 2 k at 8 k
            const uint32_t val = (b | (b << 6) | (b << 12) | (b << 18)) & 0x03030303u;
            any_bytes_to_f16<1024>(val, h[2 * e], h[2 * e + 1]);
        }
    }
};

// Q3_K as cpu_vec_dot_q3_k_f16 reads it (direct_f16_weight_q3_k): value v = 128 c + 32 j + li is bits 2 j .. + 1 of
// qs[32 c + li], minus 4 unless bit c of hmask[li] is set, times the six-bit scale of group v / 16 (minus 32), times d.
// The integer operand is value x group scale (at most 128 in magnitude, exact in fp16); d is the block's scale.
template <>
struct AnyRaw<MARMOT_HIP_KIND_Q3_K> {
    Any16 q16, hm16, tail16;  // tail16: the block's last 16 bytes = two bytes of qs, the 12 scale bytes, d
    int v0;
    __device__ __forceinline__ void fetch(const uint8_t *b, int v) {
        v0 = v;
        const int c = v >> 7, li = v & 31;
        hm16.fetch(b + li);
        q16.fetch(b + 32 + 32 * c + li);
        tail16.fetch(b + 94);
    }
    __device__ __forceinline__ void fetch_scale(const uint8_t *, int) {}
    __device__ __forceinline__ void ints(uint32_t (&h)[8], float &scale, float &offset) const {
        typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
        const uint4 q = q16.get(), hm = hm16.get(), tail = tail16.get();
        const uint32_t t0 = __builtin_amdgcn_alignbit(tail.y, tail.x, 16), t1 = __builtin_amdgcn_alignbit(tail.z, tail.y, 16),
                       t2 = __builtin_amdgcn_alignbit(tail.w, tail.z, 16);
        scale = h2f((uint16_t)(tail.w >> 16));
        offset = 0.0f;
        const int c = v0 >> 7, j = (v0 >> 5) & 3, is = v0 >> 4;
        // q3k_group_scale(scales, is): low nibble from scales[is] (is < 8) or the high nibble of scales[is - 8], two
        // more bits from scales[8 + is % 4]
        const uint64_t low8 = (uint64_t)t0 | ((uint64_t)t1 << 32);
        const uint32_t low = (uint32_t)(low8 >> (8 * (is & 7) + (is < 8 ? 0 : 4))) & 0xfu;
        const uint32_t high = (t2 >> (8 * (is & 3) + 2 * (is >> 2))) & 3u;
        const _Float16 gs = (_Float16)(float)((int)(low | (high << 4)) - 32);
        const h2_t gs2 = {gs, gs};
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w}, hw[4] = {hm.x, hm.y, hm.z, hm.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t val = ((qw[e] >> (2 * j)) & 0x03030303u) | (((hw[e] >> c) & 0x01010101u) << 2);  // 0 .. 7
            uint32_t lo, hi;
            any_bytes_to_f16<1028>(val, lo, hi);  // value - 4
            h[2 * e] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2_t, lo) * gs2);
            h[2 * e + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2_t, hi) * gs2);
        }
    }
};

// Workgroup barrier that waits for this wavefront's LDS traffic only: __syncthreads() also waits for its outstanding
// global loads, which here are the weights and activations requested rounds ahead (measured: the kernel ran at the
// latency of one such request per round, 79 us at 512 tokens whatever the format).
__device__ __forceinline__ void fa_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int KIND>
__global__ __launch_bounds__(FA_THREADS) void k_gemm_any_f16(const GemmAnyParams p) {
    using KT = KindTraits<KIND>;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // two activation stages; later the output tile
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);  // rows 32 wave .. + 31 of the tile
    const int kg = __builtin_amdgcn_readfirstlane(tid >> 8);          // K group: stages kg, kg + 2, ... of the rounds
    const int gtid = tid & (FA_GROUP - 1);
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

    // Lane (j, kh) of wavefront c owns weight row 32 c + j and, of every round, its values 16 kh .. 16 kh + 15: the
    // first eight are its share of K-step 0, the other eight of K-step 1 (the activations are read to match). No other
    // lane needs these bytes, so they come from memory straight into this lane's registers, four rounds ahead, and
    // the products of row 32 c + j land in this lane's accumulators, where its scale and offset already are.
    constexpr bool HAS_MIN = AnyInt<KIND>::HAS_MIN;
    size_t wr = row0 + (size_t)(32 * wave + j);
    wr = wr < p.M ? wr : p.M - 1;  // rows beyond M re-read the last row (never stored)
    const uint8_t *const wrow = p.w + wr * p.row_bytes;
    // closes: the round ends a span of rounds that share a scale (the formats with such spans fetch the scale fields
    // only then; known at compile time: a stage is a span, its last round closes it)
    auto fetch = [&](size_t round, AnyRaw<KIND> &raw, auto closes) {
        const size_t k0 = round * FA_ROUND + (size_t)(16 * kh);
        const size_t b = k0 / KT::BV;
        raw.fetch(wrow + b * KT::BB, (int)(k0 - b * KT::BV));
        if constexpr (AnyInt<KIND>::SCALE_ROUNDS == 1 || decltype(closes)::value) {
            raw.fetch_scale(wrow + b * KT::BB, (int)(k0 - b * KT::BV));
        }
    };

    // Activations go through LDS in stages of four rounds (128 values of K): 64 tokens x 256 bytes, token t's 16-byte
    // chunk c in slot c ^ (t % 16) (the operand reads of 16 tokens x one chunk then fall into different banks). Every
    // thread brings four chunks per stage, consecutive lanes consecutive chunks of a token's row (16 lanes per token:
    // whole 256-byte runs), a stage ahead, and stores them before the barrier that ends the stage in work.
    uint8_t *const xlds = lds + (size_t)kg * 2 * FA_XSTAGE;  // this K group's two stages
    const uint16_t *xsrc[4];
    uint32_t xdst[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int piece = i * FA_GROUP + gtid;
        const int t = piece >> 4, c = piece & 15;
        size_t tok = tok0 + (size_t)t;
        tok = tok < p.N ? tok : p.N - 1;  // tokens beyond N re-read the last one (never stored)
        xsrc[i] = p.x + tok * p.K + (size_t)(8 * c);
        xdst[i] = (uint32_t)(t * 256 + 16 * (c ^ (t & 15)));
    }
    // (macros over four named registers, not lambdas over an array or a struct: handed over by reference, the values
    // stayed in private memory, and every stage waited for its loads at once to store them there)
    uint4 xg0, xg1, xg2, xg3;
#define FA_X_REQUEST(round_)                                         \
    do {                                                             \
        xg0 = *(const uint4 *)(xsrc[0] + (round_) * FA_ROUND);       \
        xg1 = *(const uint4 *)(xsrc[1] + (round_) * FA_ROUND);       \
        xg2 = *(const uint4 *)(xsrc[2] + (round_) * FA_ROUND);       \
        xg3 = *(const uint4 *)(xsrc[3] + (round_) * FA_ROUND);       \
    } while (0)
#define FA_X_STORE(xstage_)                                          \
    do {                                                             \
        uint8_t *st_ = xlds + (size_t)(xstage_) * FA_XSTAGE;         \
        *(uint4 *)(st_ + xdst[0]) = xg0;                             \
        *(uint4 *)(st_ + xdst[1]) = xg1;                             \
        *(uint4 *)(st_ + xdst[2]) = xg2;                             \
        *(uint4 *)(st_ + xdst[3]) = xg3;                             \
    } while (0)

    fa_floatx16 acc[2];
    fa_floatx16 grp[2];                      // the products of the rounds that share a scale
    fa_floatx16 xsum[HAS_MIN ? 2 : 1];       // the sums of their activations (every lane: its 16 tokens' sums)
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            acc[a][r] = 0.0f;
            grp[a][r] = 0.0f;
            xsum[HAS_MIN ? a : 0][r] = 0.0f;
        }
    }
    const fa_half8 ones = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f,
                           (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};

    // One round: the lane's 16 integers of the round as the operands of the two K-steps, then (in program order behind
    // the decode, so the registers are free) the request for the round four later into the same registers, then the
    // products with the 64 tokens.
    auto step = [&](size_t round, AnyRaw<KIND> &raw, auto refill, auto last_of_stage) {
        uint32_t h[8];
        float scale, offset;
        raw.ints(h, scale, offset);
        if constexpr (decltype(refill)::value) {
            fetch(round + 2 * FA_XROUNDS, raw, last_of_stage);  // this K group's next stage
        }
        // this round's activations: the group's stage (round / 8) % 2, token 32 a + j, chunk 4 (round % 4) + 2 kh + ks
        const size_t rel = round - r0;
        const uint8_t *xs = xlds + (size_t)((rel / (2 * FA_XROUNDS)) & 1) * FA_XSTAGE;
        const int q = (int)(rel % FA_XROUNDS);
        constexpr int SR = AnyInt<KIND>::SCALE_ROUNDS;
        const bool opens = SR == 1 || (round % SR) == 0, closes = SR == 1 || (round % SR) == SR - 1;
        if (opens) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    grp[a][r] = 0.0f;
                    xsum[HAS_MIN ? a : 0][r] = 0.0f;
                }
            }
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const fa_half8 wb = __builtin_bit_cast(fa_half8, make_uint4(h[4 * ks], h[4 * ks + 1], h[4 * ks + 2], h[4 * ks + 3]));
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const fa_half8 x = __builtin_bit_cast(
                    fa_half8, *(const uint4 *)(xs + (32 * a + j) * 256 + 16 * ((4 * q + 2 * kh + ks) ^ (j & 15))));
                grp[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, wb, grp[a], 0, 0, 0);
                if constexpr (HAS_MIN) {
                    xsum[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, ones, xsum[a], 0, 0, 0);
                }
            }
        }
        if (closes) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float t = __builtin_fmaf(scale, grp[a][r], acc[a][r]);
                    if constexpr (HAS_MIN) {
                        t = __builtin_fmaf(offset, xsum[a][r], t);
                    }
                    // keeps the scaling inside its round (an empty statement the optimizer cannot move): sunk behind
                    // the later rounds, every round would hold its own 32 product registers until the end of the stage
                    asm volatile("" : "+v"(t));
                    acc[a][r] = t;
                }
            }
        }
    };
    // The workgroup's rounds in stages of four; K group kg takes stages kg, kg + 2, ... (`mine` of them) in its own
    // pair of LDS stages. Both groups pass the same number of barriers (`iters` after the first one). Every stage of a
    // group but its last requests the next one; the last is peeled off so that the loop body has no branch (a load
    // behind a branch makes the compiler wait for every load in flight at the next use of any of them).
    const size_t nst = (r1 - r0) / FA_XROUNDS;  // (r0 and the number of rounds are multiples of four: the launcher)
    const size_t mine = (nst + 1 - (size_t)kg) / 2;
    const size_t iters = (nst + 1) / 2;
    AnyRaw<KIND> raw[FA_XROUNDS];
    size_t round = r0 + (size_t)(FA_XROUNDS * kg);
    if (mine > 0) {
        FA_X_REQUEST(round);
        fetch(round, raw[0], std::false_type{});
        fetch(round + 1, raw[1], std::false_type{});
        fetch(round + 2, raw[2], std::false_type{});
        fetch(round + 3, raw[3], std::true_type{});
        FA_X_STORE(0);
    }
    fa_barrier();
    size_t it = 0;
    for (; it + 1 < mine; ++it, round += 2 * FA_XROUNDS) {
        FA_X_REQUEST(round + 2 * FA_XROUNDS);
        step(round, raw[0], std::true_type{}, std::false_type{});
        step(round + 1, raw[1], std::true_type{}, std::false_type{});
        step(round + 2, raw[2], std::true_type{}, std::false_type{});
        step(round + 3, raw[3], std::true_type{}, std::true_type{});
        FA_X_STORE((int)((it + 1) & 1));
        fa_barrier();  // the stage just read is free for the stage after next; the next stage is complete
    }
    if (it < mine) {
        step(round, raw[0], std::false_type{}, std::false_type{});
        step(round + 1, raw[1], std::false_type{}, std::false_type{});
        step(round + 2, raw[2], std::false_type{}, std::false_type{});
        step(round + 3, raw[3], std::false_type{}, std::true_type{});
        fa_barrier();
        ++it;
    }
    for (; it < iters; ++it) {
        fa_barrier();  // the group with one stage fewer
    }

#undef FA_X_REQUEST
#undef FA_X_STORE
    // Lane (j, kh) of wavefront c holds weight row 32 c + j for tokens 32 a + 8 (r / 4) + 4 kh + r % 4: the tile goes
    // through LDS as [token][weight row] (the stages are free behind the loop's last barrier) and every thread stores 16
    // bytes per step (stores of one float per lane cost the address unit as much as these and move a quarter).
    float *tile = (float *)lds;
    if (kg == 1) {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                tile[(32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * FA_OUT_PITCH + 32 * wave + j] = acc[a][r];
            }
        }
    }
    fa_barrier();
    if (kg == 0) {  // the two K groups' sums meet: group 0's plus group 1's
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float *e = tile + (32 * a + 8 * (r >> 2) + 4 * kh + (r & 3)) * FA_OUT_PITCH + 32 * wave + j;
                *e = acc[a][r] + *e;
            }
        }
    }
    fa_barrier();
    const bool partials = p.splits > 1;
    const bool has_bias = !partials && p.bias != nullptr;
    const bool out_f16 = !partials && p.out_is_f16;
    float *const out32 = (float *)p.out + (partials ? (size_t)split * p.N * p.M : 0);
    const bool vec = (p.M & 3) == 0 && (((uintptr_t)p.out) & 15) == 0;
    for (int idx = tid; idx < FA_TOK * FA_WROWS / 4; idx += FA_THREADS) {
        const int t = idx >> 5, q4 = idx & 31;  // rows 4 q4 .. 4 q4 + 3 of token t
        const size_t n = tok0 + (size_t)t;
        const size_t m4 = row0 + 4 * (size_t)q4;
        if (n >= p.N || m4 >= p.M) {
            continue;
        }
        const float4 v = *(const float4 *)(tile + t * FA_OUT_PITCH + 4 * q4);
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

bool gemm_f16_any_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M) {
    if (dev->knobs.no_gemm || kind == MARMOT_HIP_KIND_Q4_K || kind == MARMOT_HIP_KIND_Q8_K) {
        return false;
    }
    return N >= FA_MIN_TOKENS && K % (FA_XROUNDS * FA_ROUND) == 0 && K % block_values(kind) == 0 && M >= 1;
}

template <int KIND>
static int launch_any_kind(marmot_hip_device *dev, GemmAnyParams p, const dim3 grid) {
    MH_TRY(allow_large_lds(dev, (const void *)k_gemm_any_f16<KIND>));
    hipLaunchKernelGGL((k_gemm_any_f16<KIND>), grid, dim3(FA_THREADS), AnyInt<KIND>::LDS_BYTES, dev->stream, p);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int launch_gemm_f16_any(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K,
                        size_t M, const void *d_bias, int bias_dtype, void *d_out, int out_dtype) {
    if (!gemm_f16_any_supported(dev, kind, N, K, M)) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "fp16 GEMM: unsupported kind or shape");
    }
    if ((((uintptr_t)d_x) & 15) != 0 || (((uintptr_t)d_w) & 3) != 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT,
                         "fp16 GEMM: activations must be 16-byte aligned, weights 4-byte aligned");
    }
    const size_t rounds = K / FA_ROUND;
    const size_t tiles_n = (N + FA_TOK - 1) / FA_TOK, tiles_m = (M + FA_WROWS - 1) / FA_WROWS;
    const size_t tiles = tiles_n * tiles_m;
    const size_t cus = (size_t)dev->props.multiProcessorCount;
    // Fewer tiles than compute units: split K until the chip is full once (at least 16 rounds per workgroup). More
    // workgroups per compute unit did not pay (512 tokens x 4096 rows, Q8_0: 58 us without a K split, 67 us with two
    // resident workgroups per compute unit and the reduction launch they need).
    size_t splits = 1;
    const size_t want = 1;
    if (tiles < want * cus) {
        splits = (want * cus) / tiles;
        const size_t max_splits = rounds / 16 > 0 ? rounds / 16 : 1;
        splits = splits > max_splits ? max_splits : splits;
        splits = splits > 16 ? 16 : splits;
    }
    size_t rps = (rounds + splits - 1) / splits;
    // whole activation stages per workgroup; whole K-quant blocks (the rounds that share a scale stay together)
    const size_t grain = block_values(kind) == QK_K ? 8 : FA_XROUNDS;
    rps = (rps + grain - 1) / grain * grain;
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

// Device helpers shared by the kernels that own weight rows per workgroup (one workgroup per compute unit, loader
// wavefronts feeding an LDS ring, consumers that quantize the activations once per workgroup).
#pragma once
#include "mh_common.h"

#include <float.h>

namespace mh {

typedef __attribute__((address_space(3))) uint8_t lds_u8_t;
typedef const __attribute__((address_space(1))) uint8_t glb_u8_t;

// One direct-to-LDS load of 64 x 16 bytes: lane l's 16 bytes at base + voff land at LDS byte address lds_addr + 16 l
// (lds_addr is the same in every lane and goes through M0). Written in assembly so that the compiler does not know
// that LDS is written asynchronously: it would otherwise put "s_waitcnt vmcnt(0)" in front of every later LDS access
// of the kernel. The kernel orders LDS reads behind these loads itself (counted vmcnt waits, then LDS counters).
// The instruction's immediate offset is added to the global address AND to the LDS address, so the KIB-th KiB of a
// contiguous copy needs neither a new M0 nor a new address register.
__device__ __forceinline__ void dma_set_lds_base(uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(__builtin_amdgcn_readfirstlane(lds_addr)) : "memory");
}
template <int KIB>
__device__ __forceinline__ void dma16_to_lds(const uint8_t *base, uint32_t voff) {
    static_assert(KIB >= 0 && KIB < 4, "the immediate offset holds 12 bits");
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(base), "n"(KIB * 1024) : "memory");
}
// Vector-memory instructions of this wavefront that have not completed yet: the vmcnt counter, read without
// waiting (instruction-buffer status register, fields VM_CNT [3:0] and VM_CNT_HI [23:22]).
__device__ __forceinline__ uint32_t vmcnt_now() {
    uint32_t v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_IB_STS)" : "=s"(v) : : "memory");
    return (v & 15u) | (((v >> 22) & 3u) << 4);
}
// A pointer that is the same in every lane, said so to the compiler (scalar registers)
template <class T>
__device__ __forceinline__ T *uniform_pointer(T *ptr) {
    const uint64_t v = (uint64_t)(uintptr_t)ptr;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (T *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ void compiler_memory_fence() {
    asm volatile("" ::: "memory");
}
// LDS words that other wavefronts of the workgroup update while this one runs
__device__ __forceinline__ uint32_t lds_peek(const uint32_t *word) {
    return __builtin_amdgcn_readfirstlane(__atomic_load_n(word, __ATOMIC_RELAXED));
}
// Bounded spinning. The wavefronts of a row-owning kernel wait for one another through LDS words (segments landed,
// slots read, activations quantized). Every poll takes one from the wavefront's budget; a wavefront whose budget runs
// out waits for its own outstanding loads (they may still be writing LDS), sets a bit in a device word that the host
// reads at the next synchronize, and leaves the kernel; the wavefronts that wait for it run out in turn. A protocol
// error therefore ends as MARMOT_HIP_ERROR_INVALID_OPERATION instead of a hang. The default budget (2^26 polls of
// >= 100 clocks) is seconds; MARMOT_HIP_SPIN_LIMIT sets another one when a device object is created.
struct SpinGuard {
    uint32_t left;
    uint32_t *fault;
    __device__ __forceinline__ bool spend() {  // false: the budget is gone and the fault is recorded
        if (left != 0) {
            --left;
            return true;
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
        if ((threadIdx.x & 63u) == 0 && fault != nullptr) {
            atomicOr(fault, 1u);
        }
        return false;
    }
};
__device__ __forceinline__ bool lds_wait_at_least(const uint32_t *word, uint32_t value, SpinGuard &guard) {
    while (lds_peek(word) < value) {
        if (!guard.spend()) {
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    compiler_memory_fence();
    return true;
}

// ---- 16-lane (one DPP row) reductions
template <class T, class F>
__device__ __forceinline__ T row16_reduce(T v, F f) {
    v = f(v, __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)));
    v = f(v, __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)));
    v = f(v, __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)));
    v = f(v, __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true)));
    return v;
}

__device__ __forceinline__ int dot16r(const uint4 &w, const uint4 &a, int acc) {
    acc = sdot4(w.x, a.x, acc);
    acc = sdot4(w.y, a.y, acc);
    acc = sdot4(w.z, a.z, acc);
    acc = sdot4(w.w, a.w, acc);
    return acc;
}

// Q8_K quantization of 16 consecutive values of one 256-value block held by each of 16 adjacent lanes (lane i of the
// row holds values 16 i .. 16 i + 15). Returns this lane's 16 int8 values, their sum (one bsums entry) and the block
// scale. Results are bit-identical to cpu_quant_matmul_pack_q8_k_block (matmul_quant_pack.c:106-142).
// Fast path: the value of largest magnitude is found from the raw bits (signed integer maximum = largest positive
// float, unsigned maximum = most negative float), which needs no index tracking unless +max and -max tie; the rounding
// is the reference's magic-number add, whose low mantissa byte IS the int8 result when |iscale * x| <= 127 (always,
// for finite input whose maximum does not overflow 127 / max). Blocks that hold NaN / Inf, tiny maxima, or a +/- tie
// take the exact slow path (index tracking and the reference's clamps) for the whole wavefront.
// rot: the lane holds its four 4-value groups in rotated order, v[4 k + e] is value 4 ((rot + k) % 4) + e of the lane's
// 16 (the caller read them that way to avoid LDS bank conflicts and stores word k of q at word (rot + k) % 4).
__device__ __forceinline__ void q8k_quantize16(const float (&v)[16], int lane_in_row, uint4 &q, int &bsum, float &d,
                                               int rot = 0) {
    int pmax = (int)0x80000000;
    uint32_t nmax = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int bits = __float_as_int(v[i]);
        pmax = bits > pmax ? bits : pmax;
        nmax = (uint32_t)bits > nmax ? (uint32_t)bits : nmax;
    }
    pmax = row16_reduce(pmax, [](int a, int b) { return a > b ? a : b; });
    nmax = row16_reduce(nmax, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
    const uint32_t ap = pmax > 0 ? (uint32_t)pmax : 0u;                   // magnitude bits of the largest positive value
    const uint32_t an = nmax >= 0x80000000u ? (nmax & 0x7fffffffu) : 0u;  // ... of the most negative value
    const uint32_t amax = ap > an ? ap : an;
    const bool special = amax >= 0x7f800000u || (amax != 0u && amax < 0x03800000u) || (ap == an && ap != 0u);
    if (__builtin_amdgcn_ballot_w64(special) == 0) {
        q = make_uint4(0, 0, 0, 0);
        bsum = 0;
        d = 0.0f;
        if (amax != 0u) {
            const float mx = ap > an ? __uint_as_float(ap) : __uint_as_float(an | 0x80000000u);
            const float iscale = -127.0f / mx;
            uint32_t b[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                b[i] = __float_as_uint(iscale * v[i] + 12582912.0f);
            }
            uint32_t pk[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t lo = __builtin_amdgcn_perm(b[4 * j + 1], b[4 * j], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm(b[4 * j + 3], b[4 * j + 2], 0x04000c0cu);
                pk[j] = lo | hi;
                bsum = sdot4(pk[j], 0x01010101u, bsum);
            }
            q = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            d = 1.0f / iscale;
        }
        return;
    }
    // exact path: first occurrence of the largest |x| (strict > in index order), the packer's clamps
    float best_abs = 0.0f, best_val = 0.0f;
    int best_idx = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float ax = fabsf(v[i]);
        const int idx = 16 * lane_in_row + 4 * ((rot + (i >> 2)) & 3) + (i & 3);
        const bool gt = ax > best_abs || (ax == best_abs && ax > 0.0f && idx < best_idx);
        best_abs = gt ? ax : best_abs;
        best_val = gt ? v[i] : best_val;
        best_idx = gt ? idx : best_idx;
    }
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
        const float o_abs = __shfl_xor(best_abs, o);
        const float o_val = __shfl_xor(best_val, o);
        const int o_idx = __shfl_xor(best_idx, o);
        const bool take = o_abs > best_abs || (o_abs == best_abs && o_idx < best_idx);
        best_abs = take ? o_abs : best_abs;
        best_val = take ? o_val : best_val;
        best_idx = take ? o_idx : best_idx;
    }
    q = make_uint4(0, 0, 0, 0);
    bsum = 0;
    d = 0.0f;
    if (best_abs > 0.0f) {
        const float iscale = -127.0f / best_val;
        uint32_t pk[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            pk[j] = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int z = nearest_int_clamped(iscale * v[4 * j + i]);
                z = z > 127 ? 127 : z;
                bsum += z;
                pk[j] |= (uint32_t)(z & 0xff) << (8 * i);
            }
        }
        q = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        d = 1.0f / iscale;
    }
}

} // namespace mh

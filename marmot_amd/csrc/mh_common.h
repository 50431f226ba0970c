// Shared declarations of libmarmot_hip: GGUF block layouts, small device helpers, the device object.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <stddef.h>
#include <stdint.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "../../include/marmot_hip.h"

namespace mh {

// ---- GGUF block layouts (include/marmot/quant_block.h:20-125 of the reference)
constexpr int QK = 32;
constexpr int QK_K = 256;
constexpr int Q4_0_BYTES = 18;
constexpr int Q4_1_BYTES = 20;
constexpr int Q5_0_BYTES = 22;
constexpr int Q5_1_BYTES = 24;
constexpr int Q8_0_BYTES = 34;
constexpr int Q8_1_BYTES = 36;
constexpr int Q2_K_BYTES = 84;
constexpr int Q3_K_BYTES = 110;
constexpr int Q4_K_BYTES = 144;
constexpr int Q5_K_BYTES = 176;
constexpr int Q6_K_BYTES = 210;
constexpr int Q8_K_BYTES = 292;

struct __attribute__((packed)) BlockQ4_0 {
    uint16_t scale;
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ4_1 {
    uint16_t scale;
    uint16_t min;
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ5_0 {
    uint16_t scale;
    uint8_t qh[4];  // bit j: fifth bit of value j (32 bits, little endian)
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ5_1 {
    uint16_t scale;
    uint16_t min;
    uint8_t qh[4];
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ8_0 {
    uint16_t scale;
    int8_t qs[32];
};
struct __attribute__((packed)) BlockQ4_K {
    uint16_t d;
    uint16_t dmin;
    uint8_t scales[12];
    uint8_t qs[128];
};
struct __attribute__((packed)) BlockQ8_1 {
    uint16_t scale;
    uint16_t sum;  // f16(sum(q) * scale); not used by the dequantizer or the dots
    int8_t qs[32];
};
struct __attribute__((packed)) BlockQ2_K {
    uint8_t scales[16];  // group g of 16 values: scale in the low nibble, min in the high nibble
    uint8_t qs[64];      // value 128 c + 32 j + l: bits 2 j of qs[32 c + l]
    uint16_t d;
    uint16_t dmin;
};
struct __attribute__((packed)) BlockQ3_K {
    uint8_t hmask[32];   // value 32 t + l: bit t of hmask[l] (set: no -4 offset)
    uint8_t qs[64];      // low two bits, laid out like Q2_K
    uint8_t scales[12];  // 16 six-bit scales (offset 32): low nibbles in bytes 0..7, high pairs in bytes 8..11
    uint16_t d;
};
struct __attribute__((packed)) BlockQ5_K {
    uint16_t d;
    uint16_t dmin;
    uint8_t scales[12];
    uint8_t qh[32];  // fifth bit of value 64 g + l: bit 2 g of qh[l]; of value 64 g + 32 + l: bit 2 g + 1
    uint8_t qs[128];
};
struct __attribute__((packed)) BlockQ6_K {
    uint8_t ql[128];
    uint8_t qh[64];
    int8_t scales[16];
    uint16_t d;
};
struct __attribute__((packed)) BlockQ8_K {
    float d;
    int8_t qs[256];
    int16_t bsums[16];
};
static_assert(sizeof(BlockQ4_0) == Q4_0_BYTES, "Q4_0");
static_assert(sizeof(BlockQ8_0) == Q8_0_BYTES, "Q8_0");
static_assert(sizeof(BlockQ8_1) == Q8_1_BYTES, "Q8_1");
static_assert(sizeof(BlockQ4_1) == Q4_1_BYTES, "Q4_1");
static_assert(sizeof(BlockQ5_0) == Q5_0_BYTES, "Q5_0");
static_assert(sizeof(BlockQ5_1) == Q5_1_BYTES, "Q5_1");
static_assert(sizeof(BlockQ2_K) == Q2_K_BYTES, "Q2_K");
static_assert(sizeof(BlockQ3_K) == Q3_K_BYTES, "Q3_K");
static_assert(sizeof(BlockQ4_K) == Q4_K_BYTES, "Q4_K");
static_assert(sizeof(BlockQ5_K) == Q5_K_BYTES, "Q5_K");
static_assert(sizeof(BlockQ6_K) == Q6_K_BYTES, "Q6_K");
static_assert(sizeof(BlockQ8_K) == Q8_K_BYTES, "Q8_K");

inline size_t block_values(int kind) {
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_0:
    case MARMOT_HIP_KIND_Q4_1:
    case MARMOT_HIP_KIND_Q5_0:
    case MARMOT_HIP_KIND_Q5_1:
    case MARMOT_HIP_KIND_Q8_0:
    case MARMOT_HIP_KIND_Q8_1:
        return QK;
    case MARMOT_HIP_KIND_Q2_K:
    case MARMOT_HIP_KIND_Q3_K:
    case MARMOT_HIP_KIND_Q4_K:
    case MARMOT_HIP_KIND_Q5_K:
    case MARMOT_HIP_KIND_Q6_K:
    case MARMOT_HIP_KIND_Q8_K:
        return QK_K;
    default:
        return 0;
    }
}
inline size_t block_bytes(int kind) {
    switch (kind) {
    case MARMOT_HIP_KIND_Q4_0:
        return Q4_0_BYTES;
    case MARMOT_HIP_KIND_Q4_1:
        return Q4_1_BYTES;
    case MARMOT_HIP_KIND_Q5_0:
        return Q5_0_BYTES;
    case MARMOT_HIP_KIND_Q5_1:
        return Q5_1_BYTES;
    case MARMOT_HIP_KIND_Q8_1:
        return Q8_1_BYTES;
    case MARMOT_HIP_KIND_Q8_0:
        return Q8_0_BYTES;
    case MARMOT_HIP_KIND_Q2_K:
        return Q2_K_BYTES;
    case MARMOT_HIP_KIND_Q3_K:
        return Q3_K_BYTES;
    case MARMOT_HIP_KIND_Q4_K:
        return Q4_K_BYTES;
    case MARMOT_HIP_KIND_Q5_K:
        return Q5_K_BYTES;
    case MARMOT_HIP_KIND_Q6_K:
        return Q6_K_BYTES;
    case MARMOT_HIP_KIND_Q8_K:
        return Q8_K_BYTES;
    default:
        return 0;
    }
}
// weight formats the matmul, QKV, embedding and MoE entry points accept
inline bool is_weight_kind(int kind) {
    return kind == MARMOT_HIP_KIND_Q4_0 || kind == MARMOT_HIP_KIND_Q4_1 || kind == MARMOT_HIP_KIND_Q5_0 ||
           kind == MARMOT_HIP_KIND_Q5_1 || kind == MARMOT_HIP_KIND_Q8_0 || kind == MARMOT_HIP_KIND_Q8_1 ||
           kind == MARMOT_HIP_KIND_Q2_K ||
           kind == MARMOT_HIP_KIND_Q3_K || kind == MARMOT_HIP_KIND_Q4_K || kind == MARMOT_HIP_KIND_Q5_K ||
           kind == MARMOT_HIP_KIND_Q6_K;
}
inline bool is_k_quant(int kind) {
    return block_values(kind) == QK_K;
}

// ---- error plumbing (thread-local text like marmot_set_error, include/marmot/error.h:21-43)
int set_error(int code, const char *fmt, ...);
void set_route(const char *name);
int check_hip(hipError_t e, const char *what);

#define MH_HIP(expr)                                                                                                   \
    do {                                                                                                               \
        int _st = ::mh::check_hip((expr), #expr);                                                                      \
        if (_st != 0)                                                                                                  \
            return _st;                                                                                                \
    } while (0)

#define MH_TRY(expr)                                                                                                   \
    do {                                                                                                               \
        int _st = (expr);                                                                                              \
        if (_st != 0)                                                                                                  \
            return _st;                                                                                                \
    } while (0)

// ---- activation scratch: quantized activations in a structure-of-arrays layout private to the library.
// For N rows of K values (nb = ceil(K/block)):
//   qs    int8  [N][kp]      kp = nb*block, zero padded, 16-byte aligned rows
//   d     float [N][nb]      Q8_K: 1/iscale;  Q8_0: fp16-rounded scale widened to fp32
//   sums  int16 [N][nb*16]   Q8_K: sums of 16 (bsums);  Q8_0: [N][nb] sum of the 32 values
struct ActScratch {
    int8_t *qs = nullptr;
    float *d = nullptr;
    int16_t *sums = nullptr;
    size_t kp = 0;
    size_t nb = 0;
};

} // namespace mh

// Switches read from the environment ONCE, when the device object is created (a process that wants another setting
// creates another device object). Each one turns a route off and leaves the slower general one:
//   MARMOT_HIP_NO_MMQ          small-batch kernels on the int8 matrix cores -> packed matvec
//   MARMOT_HIP_NO_ROW_KERNELS  row-owning kernels (one workgroup per compute unit) -> the streaming kernels
//   MARMOT_HIP_NO_RESIDENT_ROWS the resident-share Q4_K decode kernel (one activation row) -> the ring form of the row kernel
//   MARMOT_HIP_NO_LDS_RING     loader / consumer matvec (weights through an LDS ring) -> register-streaming matvec
//   MARMOT_HIP_NO_FUSED_QUANT  activation quantization inside the matvec -> separate quantization launch
//   MARMOT_HIP_NO_GEMM         fp16 prefill GEMM -> fp16 matvec
//   MARMOT_HIP_NO_GEMM_LOADERS prefill GEMM tile fed by loader wavefronts -> the tile whose wavefronts load for themselves
//   MARMOT_HIP_NO_GEMM_I8      tiled int8 GEMM on Q8_K activations (33 rows and more) -> 32-row passes of the small-batch kernel
//   MARMOT_HIP_MOE_NO_VALIDATE skip the read-back of the expert-id error flag (no stream synchronization per call)
struct marmot_hip_knobs {
    bool no_mmq = false;
    bool no_row_kernels = false;
    bool no_resident_rows = false;
    bool no_attention_mfma = false;  // MARMOT_HIP_NO_ATTENTION_MFMA: paged attention scores on the vector units
    bool no_fp8_update_fused = false;  // MARMOT_HIP_NO_FP8_UPDATE_FUSED: FLOAT8_E4M3 cache update in four launches
    bool no_lds_ring = false;
    bool no_fused_quant = false;
    bool no_gemm = false;
    bool no_gemm_loaders = false;
    bool gemm_wide = false;      // MARMOT_HIP_GEMM_WIDE: the 128 x 128 prefill tile at every token count
    bool no_gemm_wide = false;   // MARMOT_HIP_NO_GEMM_WIDE: never
    bool no_gemm_i8 = false;
    bool moe_no_validate = false;
};

// The device object behind marmot_hip_device_t.
struct marmot_hip_device {
    int device_index = 0;
    marmot_hip_knobs knobs;
    hipStream_t stream = nullptr;
    hipDeviceProp_t props;
    // library-owned workspace, grown on demand (counterpart of the reference's quant workspace slots,
    // src/backends/cpu/ops/matmul/quantized/matmul_quant_dispatch.c:331-371)
    void *workspace = nullptr;
    size_t workspace_bytes = 0;
    bool capturing = false;  // between graph_begin_capture and graph_end_capture
    // Branches (marmot_hip_branch_begin / _next / _join): calls that do not depend on each other go to different
    // streams and may overlap on the device. `stream` above is the stream of the branch that is open (the main stream
    // outside a section and in a section's first branch); a branch other than the first has a workspace of its own,
    // parked in branch_workspace while another branch is open (the fields `workspace` / `workspace_bytes` always belong
    // to the open branch), so calls of different branches never share scratch memory.
    static constexpr int MAX_BRANCHES = MARMOT_HIP_MAX_BRANCHES;
    hipStream_t main_stream = nullptr;
    hipStream_t side_streams[MAX_BRANCHES - 1] = {};
    hipEvent_t fork_event = nullptr;
    hipEvent_t side_done[MAX_BRANCHES - 1] = {};
    struct ParkedWorkspace {
        void *ptr = nullptr;
        size_t bytes = 0;
    } branch_workspace[MAX_BRANCHES];
    int branch = -1;        // -1: no section is open; 0: first branch (main stream); i > 0: side stream i - 1
    int branches_used = 0;  // branches opened in the section so far
    // Executable graphs made by graph_end_capture and not destroyed yet: their kernel arguments hold workspace
    // addresses, so a workspace that is outgrown while any of them lives is retired, not freed.
    size_t live_graphs = 0;
    size_t last_capture_nodes = 0;
    std::vector<void *> retired_workspaces;
    // A statically allocated scratch array of the library as this device sees it (hipGetSymbolAddress at creation)
    // and, while an entry point that must not allocate runs, the switch that makes workspace_reserve hand it out
    // instead of the growing workspace.
    void *static_scratch = nullptr;
    size_t static_scratch_bytes = 0;
    bool use_static_scratch = false;
    std::unordered_set<const void *> large_lds_kernels;  // kernels whose dynamic-LDS limit has been raised (under mu)
    // SpinGuard (mh_rows.h): the device word in which a row-owning kernel records that a wavefront gave up waiting, and
    // the polls a wavefront may spend (MARMOT_HIP_SPIN_LIMIT, read at creation)
    uint32_t *fault_word = nullptr;
    uint32_t spin_limit = 1u << 26;
    // Timeline build only (-DMH_TIMELINE): device buffer of the caller that instrumented kernels write their marks to
    // (marmot_hip_timeline_attach); nullptr = marks off.
    unsigned long long *timeline = nullptr;
    uint32_t timeline_words = 0;
    // allocation accounting
    std::mutex mu;
    std::unordered_map<void *, size_t> allocs;
    size_t current_bytes = 0;
    size_t peak_bytes = 0;
};

namespace mh {

#if defined(__HIPCC__)
// Kernel arguments are fetched through the scalar cache, one 64-byte line per miss, each on first use: a kernel whose
// arguments span several lines pays those misses one after the other along its prologue (and again in its epilogue
// for fields first read there). Touching every line at kernel entry overlaps them into one miss (measured: 0.3-0.5 us
// per launch). BYTES: the explicit arguments to cover. EXPLICIT_SIZE: for a kernel that reads blockDim or gridDim, the
// size of ALL its explicit arguments: the launch dimensions are hidden arguments stored right behind them (block
// counts, then group sizes), usually in a line of their own, and are needed by the first instructions (measured:
// 0.25 us per launch when the explicit arguments grew and pushed them out of a line that was touched anyway).
// Leave EXPLICIT_SIZE at 0 for a kernel that does not read them: its argument segment may end with the explicit ones.
template <int BYTES, int EXPLICIT_SIZE = 0>
__device__ __forceinline__ void warm_kernel_arguments() {
    const uint32_t __attribute__((address_space(4))) *kargs =
        (const uint32_t __attribute__((address_space(4))) *)__builtin_amdgcn_kernarg_segment_ptr();
    uint32_t touched = kargs[(BYTES - 4) / 4];
#pragma unroll
    for (int off = 0; off < BYTES - 4; off += 64) {
        touched ^= kargs[off / 4];
    }
    if (EXPLICIT_SIZE > 0) {
        constexpr int hidden = (EXPLICIT_SIZE + 7) & ~7;  // block counts at +0..11, group sizes at +12..17
        touched ^= kargs[hidden / 4] ^ kargs[(hidden + 16) / 4];
    }
    asm volatile("" ::"s"(touched));
}

// Timeline marks (diagnostic build, -DMH_TIMELINE; the product build compiles them to nothing). MH_MARK(p, slot) keeps
// the wavefront's cycle counter (s_memtime, one scalar instruction, nobody waits for it) in registers; when the
// wavefront leaves, MH_MARK_FLUSH(p) has lane 0 store the marks into words
// (wavefront index in the launch) * MH_TIMELINE_SLOTS + slot of the attached buffer. Slots 0 .. 11 are the kernel's;
// 12 / 13 hold the cycle counter and the 100 MHz constant-rate counter (common to the whole device) at the first
// mark, 14 / 15 the same pair at the flush, which gives the cycle counter's rate and a common time base.
#define MH_TIMELINE_SLOTS 16
#if defined(MH_TIMELINE)
struct TimelineArg {
    unsigned long long *buf;
    uint32_t words;
};
__device__ __forceinline__ void timeline_flush(const TimelineArg &t, unsigned long long (&tm)[MH_TIMELINE_SLOTS]) {
    tm[14] = __builtin_readcyclecounter();
    tm[15] = __builtin_amdgcn_s_memrealtime();
    if (t.buf != nullptr && (threadIdx.x & 63u) == 0) {
        const uint32_t wave = (blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
        const uint32_t base = wave * MH_TIMELINE_SLOTS;
        if (base + MH_TIMELINE_SLOTS <= t.words) {
#pragma unroll
            for (int i = 0; i < MH_TIMELINE_SLOTS; ++i) {
                t.buf[base + i] = tm[i];
            }
        }
    }
}
#define MH_TIMELINE_FIELD ::mh::TimelineArg timeline;
#define MH_TIMELINE_SET(p, dev) ((p).timeline = ::mh::TimelineArg{(dev)->timeline, (dev)->timeline_words})
#define MH_MARK_DECL                                                                                                   \
    unsigned long long mh_tm[MH_TIMELINE_SLOTS] = {};                                                                  \
    mh_tm[12] = __builtin_readcyclecounter();                                                                          \
    mh_tm[13] = __builtin_amdgcn_s_memrealtime();
#define MH_MARK(p, slot) (mh_tm[slot] = __builtin_readcyclecounter())
#define MH_MARK_FLUSH(p) ::mh::timeline_flush((p).timeline, mh_tm)
#else
#define MH_TIMELINE_FIELD
#define MH_TIMELINE_SET(p, dev) ((void)0)
#define MH_MARK_DECL
#define MH_MARK(p, slot) ((void)0)
#define MH_MARK_FLUSH(p) ((void)0)
#endif

// s_waitcnt vmcnt(n) for a run-time n: the immediate must be a constant, and it must be the exact count (a smaller one
// would also wait for loads of the newer steps, i.e. for a full memory latency)
#define MH_VMCNT_CASE(n)                                                             \
    case n:                                                                          \
        __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 15) | (((n) >> 4) << 14));        \
        break;
#define MH_VMCNT_CASE4(n) MH_VMCNT_CASE(n) MH_VMCNT_CASE(n + 1) MH_VMCNT_CASE(n + 2) MH_VMCNT_CASE(n + 3)
#define MH_VMCNT_CASE16(n) MH_VMCNT_CASE4(n) MH_VMCNT_CASE4(n + 4) MH_VMCNT_CASE4(n + 8) MH_VMCNT_CASE4(n + 12)
__device__ __forceinline__ void wait_vmcnt_at_most(int allowed) {
    // the count is the same for every lane; saying so keeps the dispatch on the scalar unit (compares and branches)
    // instead of a tree of execution-mask branches
    switch (__builtin_amdgcn_readfirstlane(allowed > 63 ? 63 : allowed)) {
        MH_VMCNT_CASE16(0)
        MH_VMCNT_CASE16(16)
        MH_VMCNT_CASE16(32)
        MH_VMCNT_CASE16(48)
    default:
        __builtin_amdgcn_s_waitcnt(0x0f70);
        break;
    }
}
#endif

// Looks up this device's address of the library's static scratch array (mh_matmul.hip); called by device_create.
int static_scratch_init(marmot_hip_device *dev);

// Raises a kernel's dynamic-LDS limit to the 160 KiB of a gfx950 compute unit, once per device and kernel.
int allow_large_lds(marmot_hip_device *dev, const void *kernel);

// Returns a workspace of at least `bytes` (256-byte aligned). Growing it synchronizes the stream first.
int workspace_reserve(marmot_hip_device *dev, size_t bytes, void **out);

// Carves the activation scratch for `rows` x `k` out of `base`; returns bytes consumed (256-byte rounded).
size_t act_scratch_layout(int act_kind, size_t rows, size_t k, void *base, ActScratch *out);

// kernels / launchers implemented in the .hip files
int launch_quantize_act_soa(marmot_hip_device *dev, int act_kind, const void *d_x, int in_dtype, size_t rows, size_t k,
                            const ActScratch &dst);
// act == nullptr selects the fused variant: d_x_f32 ([N,K] fp32, N <= 4, K a multiple of the block) is quantized inside
// the matvec kernel; otherwise `act` holds activations packed by launch_quantize_act_soa.
bool matvec_can_fuse_quantization(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *d_x_f32);
int launch_matvec_packed(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, const ActScratch *act,
                         const float *d_x_f32, size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype,
                         void *d_out0, void *d_out1, int out_dtype);
// Up to three weights of one shape [M, K] and one quant kind that share the activations: a single matmul, the
// gate/up pair, the q/k/v triple. One launch streams all of them (the weight index is a grid dimension).
struct WeightSet {
    int count = 1;
    const void *w[3] = {nullptr, nullptr, nullptr};
    const void *bias[3] = {nullptr, nullptr, nullptr};  // per weight, nullptr = none
    void *out[3] = {nullptr, nullptr, nullptr};
    int bias_dtype = 0;
    // fp16 output only. false: f16(f16(dot) + bias), the matmul epilogue adds the bias to the stored value;
    // true: f16(dot + bias), the q/k/v projection starts its fp32 accumulator from the bias (matmul_qkv.c:889-915).
    bool bias_first = false;
};
int launch_matvec_set(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch *act,
                      const float *d_x_f32, size_t N, size_t K, size_t M, int out_dtype);
// Row-owning Q4_K matvec for one or two fp32 activation rows (mh_matvec_rows.hip): one workgroup per compute unit,
// activations quantized once per workgroup. Returns MARMOT_HIP_ERROR_NOT_IMPLEMENTED, error text untouched, for shapes
// it does not cover.
int launch_matvec_rows_q4k(marmot_hip_device *dev, const WeightSet &ws, const float *d_x_f32, size_t N, size_t K,
                           size_t M, int out_dtype);
// Launch plans of the two ring kernels as numbers (no device needed): diagnostics behind marmot_hip_rows_plan_probe
bool rows_plan_probe(uint32_t cus, size_t N, size_t K, size_t M, int nw, uint32_t *out, size_t n_out);
bool mmq_rows_plan_probe(uint32_t cus, size_t N, size_t K, size_t M, int nw, bool packed, uint32_t *out, size_t n_out);
// Resident-share form of the same for ONE weight and ONE activation row (mh_matvec_rows2.hip): the workgroup's rows are
// copied into LDS once, the loaders also fetch the activation row. Same return convention.
int launch_matvec_rows2_q4k(marmot_hip_device *dev, const WeightSet &ws, const float *d_x_f32, size_t N, size_t K,
                            size_t M, int out_dtype);
// Row-owning small-batch Q4_K matmul on the int8 matrix cores for 1..16 activation rows (mh_mmq_rows.hip): fp32 rows
// are quantized inside the kernel (act == nullptr), packed rows are copied into LDS by the kernel's loaders; K is
// split inside the workgroup. Returns
// MARMOT_HIP_ERROR_NOT_IMPLEMENTED, error text untouched, for shapes it does not cover.
bool mmq_rows_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M, int nw, bool packed);
int launch_mmq_rows_q4k(marmot_hip_device *dev, const WeightSet &ws, const float *d_x_f32, const ActScratch *act,
                        size_t N, size_t K, size_t M, int out_dtype);
// quantizes act(gate) * up (SwiGLU or GeGLU) of two fp32 [rows, k] arrays into the activation scratch
int launch_quantize_glu_soa(marmot_hip_device *dev, int act_kind, const float *d_gate, const float *d_up, bool geglu,
                            size_t rows, size_t k, const ActScratch &dst);
int launch_matvec_grouped(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, size_t expert_stride,
                          const ActScratch &act, const uint32_t *d_act_index, const int4 *d_items, const int *d_n_items,
                          size_t max_items, size_t K, size_t M, void *d_out0, void *d_out1);
int launch_matvec_f16(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K, size_t M,
                      const void *d_bias, int bias_dtype, void *d_out, int out_dtype);
// small-batch int8-MFMA matmul (mh_mmq.hip)
bool mmq_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, int weights = 1);
size_t mmq_scratch_bytes(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M, int weights);
int launch_mmq(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, const ActScratch &act, size_t N,
               size_t K, size_t M, const void *d_bias, int bias_dtype, void *d_out0, void *d_out1, int out_dtype,
               void *scratch);
// Tiled int8 GEMM on Q8_K activations (mh_gemm_i8.hip): Q4_K, Q5_K and Q6_K weights; 33 activation rows and more
bool gemm_i8_applies(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *const *weights, int count,
                     const ActScratch &act);
size_t gemm_i8_scratch_bytes(const marmot_hip_device *dev, size_t N, size_t K, size_t M, int weights);
int launch_gemm_i8(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                   size_t M, int out_dtype, void *scratch);
// Tiled int8 GEMM on Q8_0 activations (mh_gemm_i8.hip): Q8_0 and Q4_0 weights, K a multiple of 256, nine rows and more;
// `scratch` holds gemm_i8_scratch_bytes for the K-split partial sums
bool gemm_q23k_applies(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *const *weights, int count,
                       const ActScratch &act);
int launch_gemm_q23k(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                     size_t M, int out_dtype, void *scratch);
size_t gemm_q80_min_rows(int kind);  // activation rows from which the tiled kernel of the format takes over
bool gemm_q80_kind(int kind);  // Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K: formats of the tiled int8 GEMMs from nine rows on
bool gemm_q80_applies(const marmot_hip_device *dev, int kind, size_t N, size_t K, const void *const *weights, int count,
                      const ActScratch &act);
int launch_gemm_q80(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                    size_t M, int out_dtype, void *scratch);
int launch_mmq_set(marmot_hip_device *dev, int kind, const WeightSet &ws, const ActScratch &act, size_t N, size_t K,
                   size_t M, int out_dtype, void *scratch);
bool mmq_grouped_supported(const marmot_hip_device *dev, int kind, size_t K);
int launch_mmq_grouped(marmot_hip_device *dev, int kind, const void *d_w0, const void *d_w1, size_t expert_stride,
                       const ActScratch &act, const uint32_t *d_act_index, const int4 *d_items, const int *d_n_items,
                       size_t max_items, size_t K, size_t M, void *d_out0, void *d_out1, int item_cols);
// sums fp32 partials [splits][N][M] in split order, then bias and output cast (mh_gemm.hip)
int launch_splitk_reduce(marmot_hip_device *dev, const float *partial, int splits, size_t N, size_t M,
                         const void *d_bias, int bias_dtype, void *d_out, int out_dtype, bool bias_first = false);
bool gemm_f16_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M);
int launch_gemm_f16(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K, size_t M,
                    const void *d_bias, int bias_dtype, void *d_out, int out_dtype);
// fp16 activations and every other weight format (mh_gemm_f16_any.hip): 9 rows and more, K a multiple of 128
bool gemm_f16_any_supported(const marmot_hip_device *dev, int kind, size_t N, size_t K, size_t M);
int launch_gemm_f16_any(marmot_hip_device *dev, int kind, const void *d_w, const void *d_x, size_t N, size_t K,
                        size_t M, const void *d_bias, int bias_dtype, void *d_out, int out_dtype);

// ---- device helpers
#if defined(__HIPCC__)
__device__ __forceinline__ float h2f(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}
__device__ __forceinline__ uint16_t f2h(float f) {
    return __half_as_ushort(__float2half_rn(f));
}

// Sum over the 64 lanes of a wavefront; every lane receives the total. DPP within rows of 16, then
// cross-row through readlane.
__device__ __forceinline__ float wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)); // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true)); // row_mirror
    const int iv = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
    return (r0 + r1) + (r2 + r3);
}

// magic-number round-to-nearest-even with the input clamp of the reference's activation packer
// (matmul_quant_pack.c:11-21)
__device__ __forceinline__ int nearest_int_clamped(float value) {
    value = fminf(fmaxf(value, -4194303.0f), 4194303.0f);  // branch-free form of the reference's two-sided clamp
    const float shifted = value + 12582912.0f;
    const int bits = __float_as_int(shifted);
    return (bits & 0x007fffff) - 0x00400000;
}

// Sum over each row of 16 lanes (DPP only); every lane of the row receives the row's total.
__device__ __forceinline__ float row16_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    return v;
}

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}
#endif

} // namespace mh

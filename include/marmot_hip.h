/*
 * marmot_hip.h — C ABI of libmarmot_hip: the MI355X (gfx950) kernels behind marmot's
 * block-quantized GGUF matmul path, plus the device plumbing a MARMOT_BACKEND_HIP needs.
 *
 * Plain pointers and sizes only. All `d_` pointers are device addresses obtained from
 * marmot_hip_alloc (or any hipMalloc in the same process); everything is enqueued on the
 * device object's stream and is asynchronous unless stated. Return values are marmot_error_t
 * codes (0 = success, negative = include/marmot/types.h:210-220 of the reference); the text of
 * the last failure on the calling thread is available from marmot_hip_last_error().
 *
 * Each entry names the reference interface it replaces (paths relative to the reference tree).
 * The marmot_tensor_t-level backend (device vtable, kernel query, bytecode exec table) that sits
 * on top of this ABI is declared in marmot_hip_backend.h.
 *
 * Naming follows the reference: marmot_linear(input[N,K], weight[M,K]) -> out[N,M]; N = tokens,
 * K = reduction dim, M = weight rows (include/marmot/ops/matmul.h:11).
 */
#ifndef MARMOT_HIP_H
#define MARMOT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct marmot_hip_device marmot_hip_device_t;

/* marmot_error_t values (include/marmot/types.h:210-220) */
enum {
    MARMOT_HIP_SUCCESS = 0,
    MARMOT_HIP_ERROR_INVALID_ARGUMENT = -1,
    MARMOT_HIP_ERROR_OUT_OF_MEMORY = -2,
    MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE = -3,
    MARMOT_HIP_ERROR_BACKEND_INIT_FAILED = -4,
    MARMOT_HIP_ERROR_INVALID_OPERATION = -5,
    MARMOT_HIP_ERROR_UNSUPPORTED_DTYPE = -6,
    MARMOT_HIP_ERROR_DIMENSION_MISMATCH = -7,
    MARMOT_HIP_ERROR_NOT_IMPLEMENTED = -8,
};

/* marmot_quant_kind_t values (include/marmot/types.h:372-388). Weight kinds: all but Q8_K, which (like Q8_0) is the
 * format of packed activations. */
enum {
    MARMOT_HIP_KIND_Q4_0 = 1,
    MARMOT_HIP_KIND_Q4_1 = 2,
    MARMOT_HIP_KIND_Q5_0 = 3,
    MARMOT_HIP_KIND_Q5_1 = 4,
    MARMOT_HIP_KIND_Q8_0 = 5,
    MARMOT_HIP_KIND_Q8_1 = 6,
    MARMOT_HIP_KIND_Q2_K = 7,
    MARMOT_HIP_KIND_Q3_K = 8,
    MARMOT_HIP_KIND_Q4_K = 9,
    MARMOT_HIP_KIND_Q5_K = 10,
    MARMOT_HIP_KIND_Q6_K = 11,
    MARMOT_HIP_KIND_Q8_K = 12,
};

/* marmot_dtype_t values (include/marmot/types.h:340-362) */
enum {
    MARMOT_HIP_DTYPE_F32 = 0,
    MARMOT_HIP_DTYPE_F16 = 1,
    MARMOT_HIP_DTYPE_BF16 = 2, /* paged attention (activations and KV cache) and marmot_hip_convert */
    MARMOT_HIP_DTYPE_I32 = 3,  /* position tensors of the rotary epilogue only */
    MARMOT_HIP_DTYPE_U8 = 6,   /* storage type of block-quantized tensors (GGUF reader) */
    MARMOT_HIP_DTYPE_U32 = 8,  /* row indices of marmot_hip_gather_rows */
    MARMOT_HIP_DTYPE_I64 = 11,
    MARMOT_HIP_DTYPE_F8_E4M3 = 14, /* paged attention only: the KV cache with per-block scales */
};

/* marmot_router_weight_policy_t (include/marmot/types.h:283-288), marmot_ffn_type_t (:276-281) */
enum {
    MARMOT_HIP_ROUTER_SOFTMAX_SELECTED = 0,
    MARMOT_HIP_ROUTER_SOFTMAX_SELECTED_SCALED = 1,
    MARMOT_HIP_ROUTER_RENORMALIZE_SELECTED = 2,
};
enum { MARMOT_HIP_FFN_SWIGLU = 0, MARMOT_HIP_FFN_GEGLU = 2 };

/* flags of marmot_hip_matmul_quantized */
enum {
    /* quantize fp16 activations to Q8_0/Q8_K instead of the direct fp16 path
     * (cpu_context_t.force_q8_activations, src/backends/cpu/ops/matmul/quantized/matmul_quant_dispatch.c:438-441) */
    MARMOT_HIP_MATMUL_FORCE_PACK = 1u << 0,
};

/* ------------------------------------------------------------------ device lifecycle and memory
 * Replaces marmot_device_ops_t.{init,destroy,alloc,free,memcpy_to_device,memcpy_from_device,synchronize}
 * (include/marmot/device.h:43-66) at the raw-pointer level. */
int marmot_hip_device_create(int device_index, marmot_hip_device_t **out_dev);
void marmot_hip_device_destroy(marmot_hip_device_t *dev);
int marmot_hip_alloc(marmot_hip_device_t *dev, size_t size, void **out_dptr);
void marmot_hip_free(marmot_hip_device_t *dev, void *dptr);
/* Synchronous with respect to the host buffer: returns after the bytes have left / reached `host`. */
int marmot_hip_memcpy_to_device(marmot_hip_device_t *dev, void *d_dst, const void *host_src, size_t size);
int marmot_hip_memcpy_from_device(marmot_hip_device_t *dev, void *host_dst, const void *d_src, size_t size);
int marmot_hip_memcpy_device(marmot_hip_device_t *dev, void *d_dst, const void *d_src, size_t size);
int marmot_hip_memset(marmot_hip_device_t *dev, void *d_dst, int value, size_t size);
int marmot_hip_synchronize(marmot_hip_device_t *dev);
/* bytes currently held through marmot_hip_alloc, and the high-water mark
 * (marmot_device_ops_t.allocator_usage, include/marmot/allocator.h:27-36) */
int marmot_hip_allocator_usage(marmot_hip_device_t *dev, size_t *current_bytes, size_t *peak_bytes, size_t *n_allocs);
/* The hipStream_t the work of this device object is enqueued on (as void*): the main stream, or inside a branch
 * section (marmot_hip_branch_begin) the stream of the branch that is open. */
void *marmot_hip_stream(marmot_hip_device_t *dev);
const char *marmot_hip_last_error(void);

/* Device facts for marmot_device_caps_t (include/marmot/device_caps.h:14-71) — replaces the per-backend
 * branch of marmot_backend_detect_default_caps (src/core/dispatch/kernel_query.c:88-109). */
typedef struct {
    char name[64];
    char arch[32];           /* e.g. "gfx950" */
    uint32_t num_compute_units;
    uint32_t wavefront_size;
    uint32_t clock_mhz;      /* max engine clock */
    uint32_t mem_clock_mhz;
    uint32_t mem_bus_bits;
    uint32_t l2_cache_kb;
    uint32_t lds_kb_per_cu;
    uint64_t total_mem_bytes;
    float mem_bw_gbps;       /* published HBM peak used for rooflines */
    float peak_tflops_fp16;  /* dense MFMA */
    float peak_tops_int8;    /* dense MFMA */
} marmot_hip_caps_t;
int marmot_hip_get_caps(marmot_hip_device_t *dev, marmot_hip_caps_t *caps);

/* Batched submission: everything enqueued between begin and end is recorded into a HIP graph instead of being
 * executed; launching the returned graph replays the whole batch with one submission. This is the HIP form of
 * marmot_device_ops_t.graph_batch_begin / graph_batch_end(commit) (include/marmot/device.h:57-61), which the graph
 * executor brackets a bytecode program with (src/graph/graph_executor.cpp:895).
 * Rules: a call that needs a larger workspace than any call before it cannot be recorded (it would allocate): run it
 * once eagerly first; the capture returns MARMOT_HIP_ERROR_INVALID_OPERATION otherwise. After a capture the workspace
 * may still grow (an eager call with a larger shape): the old one stays allocated until the last executable graph is
 * destroyed, so earlier graphs stay valid. One graph holds at most MARMOT_HIP_GRAPH_MAX_NODES nodes:
 * graph_end_capture refuses a longer recording (INVALID_OPERATION; split the batch into several graphs). The limit
 * keeps one submission within what a profiler's queue interception handles: a replay of a 2700-kernel graph under
 * `rocprofv3 --kernel-trace` ended in a segmentation fault inside the preloaded interception library, while graphs
 * of 4500 kernels replay without a profiler attached. graph_last_capture_nodes reports the node count of the latest
 * end_capture (also of a refused one), for callers that size their batches. */
#define MARMOT_HIP_GRAPH_MAX_NODES 1024
int marmot_hip_graph_begin_capture(marmot_hip_device_t *dev);
int marmot_hip_graph_end_capture(marmot_hip_device_t *dev, void **out_graph_exec);
int marmot_hip_graph_launch(marmot_hip_device_t *dev, void *graph_exec);
void marmot_hip_graph_destroy(marmot_hip_device_t *dev, void *graph_exec);
size_t marmot_hip_graph_max_nodes(void);
size_t marmot_hip_graph_last_capture_nodes(marmot_hip_device_t *dev);

/* Branches: calls that do not depend on each other may overlap on the device. No counterpart in the reference, whose
 * interpreter runs the instructions of a bytecode program one after the other (marmot_bc_execute_with_hooks,
 * src/core/bytecode/bytecode.c:196-286, called from src/graph/graph_executor.cpp:895);
 * it is for an executor that knows which consecutive instructions are independent (the q, k and v projections of one
 * normalized row; gate and up), because on this device the tail of one linear, the gap to the next launch and the
 * next one's start-up cost 2 - 3 us per linear that nothing else hides.
 *   branch_begin : opens a section; the calls that follow form its first branch
 *   branch_next  : the calls that follow form the next branch; it starts after everything enqueued BEFORE
 *                  branch_begin, and is unordered with respect to the other branches of the section
 *   branch_join  : closes the section; whatever is enqueued afterwards starts after every branch has finished
 * Works the same inside a batched submission (the branches become parallel paths of the HIP graph) and outside one
 * (streams and events). A section holds at most MARMOT_HIP_MAX_BRANCHES branches; sections do not nest; a section
 * opened inside a batched submission must be joined before graph_end_capture, and graph_begin_capture inside a
 * section is refused (all INVALID_OPERATION / INVALID_ARGUMENT). Every branch has a workspace of its own, so calls of
 * different branches share no scratch memory; the caller guarantees that no branch reads or writes what another
 * branch of the same section writes. The first section of a device object makes its side streams and cannot be
 * recorded: run one section outside a batched submission first (INVALID_OPERATION otherwise), as for a workspace
 * that has to grow. marmot_hip_synchronize inside a section waits for all its branches. The entry
 * point that does not allocate may only be called in a section's first branch (its scratch array exists once). */
#define MARMOT_HIP_MAX_BRANCHES 4
int marmot_hip_branch_begin(marmot_hip_device_t *dev);
int marmot_hip_branch_next(marmot_hip_device_t *dev);
int marmot_hip_branch_join(marmot_hip_device_t *dev);

/* DIAGNOSTIC (measurement aid, not an operator), no counterpart in the reference: one launch that only reads `size` bytes at d_src (16-byte loads,
 * nothing is written; d_sink is 1 KiB of device memory the kernel may touch only for a pattern the test data cannot
 * produce). bench.py times it beside the matvec to report the read bandwidth this box delivers to one dependent
 * launch of the same size. size and d_src must be multiples of 16. */
int marmot_hip_read_probe(marmot_hip_device_t *dev, const void *d_src, size_t size, void *d_sink);

/* DIAGNOSTIC (measurement aid, not an operator), no counterpart in the reference: a one-wavefront kernel on the device object's stream that stores the
 * device's constant-rate counter (100 MHz, 10 ns per tick) into the 8 bytes at d_ticks. Unlike a HIP event it can be
 * recorded into a captured graph, so a benchmark can bracket the steps of one graph replay without the submission of
 * the graph in the figure (bench.py does). */
int marmot_hip_timestamp(marmot_hip_device_t *dev, void *d_ticks);

/* DIAGNOSTIC, no counterpart in the reference, no device needed: the launch plan of a ring kernel for a shape as plain
 * numbers, for the host-side model that checks the loader / consumer protocol over the plan space
 * (tests/test_rows_protocol.py). kernel 0 = ring form of the Q4_K decode row kernel (13 values: G, wavefronts, rows per
 * workgroup, K segments, blocks per segment, rows per task, lag, pre, consumers, slots, slot bytes, grid, LDS bytes);
 * kernel 1 = row-owning small-batch kernel (20 values: token slots, wavefronts, rows per workgroup, rows per group,
 * blocks per task, tasks along K, consumers per row group, tasks per K part, row groups per round, rounds, task
 * consumers, consumers, slots, slot bytes, instructions per task, lag, pre, grid, prologue lag, LDS bytes).
 * Returns MARMOT_HIP_ERROR_NOT_IMPLEMENTED (error text untouched) for shapes the kernel does not take. */
int marmot_hip_rows_plan_probe(int kernel, uint32_t compute_units, size_t N, size_t K, size_t M, int weights, int packed,
                               uint32_t *out, size_t n_out);

/* DIAGNOSTIC, no counterpart in the reference: in a library built with `make TIMELINE=1` (-DMH_TIMELINE; it is
 * written to marmot_amd/lib/libmarmot_hip_timeline.so) the instrumented kernels (the row-owning Q4_K matvec, the read
 * probe) store the device's 100 MHz constant-rate counter at marked points: one 8-byte word per wavefront and mark, at
 * word (wavefront index in the launch) * 16 + mark of `d_marks` (device memory of the caller, `bytes` long; later
 * launches overwrite earlier ones; NULL turns the marks off). The product build has no marks in its kernels and
 * returns MARMOT_HIP_ERROR_NOT_IMPLEMENTED. */
int marmot_hip_timeline_attach(marmot_hip_device_t *dev, void *d_marks, size_t bytes);

/* Timing helpers (HIP events on the device object's stream). */
int marmot_hip_event_create(marmot_hip_device_t *dev, void **out_event);
void marmot_hip_event_destroy(marmot_hip_device_t *dev, void *event);
int marmot_hip_event_record(marmot_hip_device_t *dev, void *event);
int marmot_hip_event_elapsed_ms(marmot_hip_device_t *dev, void *start, void *stop, float *out_ms);

/* ------------------------------------------------------------------ block geometry */
size_t marmot_hip_block_values(int kind);
size_t marmot_hip_block_bytes(int kind);
/* bytes of one weight row of k values: ceil(k / block_values) * block_bytes
 * (src/backends/cpu/ops/matmul/quantized/matmul_quant_dispatch.c:423-427) */
size_t marmot_hip_row_bytes(int kind, size_t k);

/* ------------------------------------------------------------------ dequantize (the bit-exact contract)
 * Replaces cpu_dequantize_{q4_0,q8_0,q4_k,q6_k,q8_k} -> cpu_dequantize_blockwise
 * (src/backends/cpu/quantization/ops/quantize_core.c:267-331) with the per-block arithmetic of
 * q4k_gguf.c:133-166, q6k_gguf.c:63-99, q8_gguf.c:189-200, q4_gguf.c:367-394.
 * d_blocks: rows * marmot_hip_row_bytes(kind,k) bytes in native GGUF block layout; d_out: rows*k fp32. */
int marmot_hip_dequantize(marmot_hip_device_t *dev, int kind, const void *d_blocks, size_t rows, size_t k,
                          float *d_out);

/* ------------------------------------------------------------------ activation quantizers
 * Replaces cpu_matmul_quant_pack_q8_0_{f32,f16} / cpu_matmul_quant_pack_q8_k_{f32,f16}
 * (src/backends/cpu/ops/matmul/quantized/matmul_quant_pack.c:23-196) and, for block output, the
 * QUANTIZE schema entries cpu_quantize_q8_0 / cpu_quantize_q8_k. act_kind: Q8_0 or Q8_K.
 * d_x: rows x k activations of in_dtype (row-major, contiguous); d_blocks_out: rows * row_bytes(act_kind,k)
 * bytes of marmot_q8_0_block_t / marmot_q8_k_block_t (include/marmot/quant_block.h:48-52, 121-125). */
int marmot_hip_quantize_activations(marmot_hip_device_t *dev, int act_kind, const void *d_x, int in_dtype,
                                    size_t rows, size_t k, void *d_blocks_out);

/* ------------------------------------------------------------------ K-quant weight quantizers
 * Replaces cpu_quantize_q4_k / cpu_quantize_q5_k / cpu_quantize_q6_k -> cpu_quantize_blockwise
 * (src/backends/cpu/quantization/ops/quantize_core.c:199-265) with the per-block searches of
 * src/backends/cpu/quantization/formats/q4k_gguf.c:35-131, q5k_gguf.c:35-160, q6k_gguf.c:35-61 and
 * src/backends/cpu/quantization/common/kquant_common.h:39-130 (make_qkx2_quants), 150-236 (make_qx_quants),
 * 310-369 (quantize_row_q6_k_ref_single). d_x: [rows, k] fp32, row-major; d_blocks_out: rows x ceil(k / 256) blocks of
 * `kind` (Q4_K, Q5_K or Q6_K), a partial last block quantizes zeros beyond k and zeroes the bytes the reference zeroes.
 * The blocks equal the reference's byte for byte (model preparation: not a per-token path). */
int marmot_hip_quantize_weights(marmot_hip_device_t *dev, int kind, const float *d_x, size_t rows, size_t k,
                                void *d_blocks_out);

/* ------------------------------------------------------------------ quantized linear
 * Replaces cpu_matmul_quantized_{scheme} (every weight scheme of the reference) -> cpu_matmul_quantized_impl
 * (src/backends/cpu/ops/matmul/quantized/matmul_quant_dispatch.c:373-591, 905-929) incl. the bias epilogue
 * (src/backends/cpu/ops/matmul/matmul_epilogue.c). out[n*M + m] = dot(W[m,:], x[n,:]) (+ bias[m]).
 *   d_weight : M rows of marmot_hip_row_bytes(kind,K) bytes, native GGUF blocks
 *   d_input  : [N,K] of in_dtype; F32 -> activations are quantized to Q8_0 (32-value weight blocks) or Q8_K
 *              (K-quants) and integer block dots are used; F16 -> direct dequantized dot unless FORCE_PACK
 *              (NOT_IMPLEMENTED for Q2_K, Q3_K, Q5_K and Q6_K, whose direct dots in the reference do not agree
 *              with its dequantizers: the caller falls back or packs)
 *   d_bias   : NULL or M values of bias_dtype (F32, or F16 when out is F16)
 *   d_out    : [N,M] of out_dtype (F32; F16 allowed only with F16 input)
 * Errors mirror marmot_matmul_validate_quantized (src/core/helpers/matmul.c:68-136). */
int marmot_hip_matmul_quantized(marmot_hip_device_t *dev, int kind, const void *d_weight, const void *d_input,
                                int in_dtype, size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype,
                                void *d_out, int out_dtype, uint32_t flags);

/* marmot_hip_matmul_quantized for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc. No counterpart in the reference. Same arguments, routes, kernels and
 * results (bit for bit) as marmot_hip_matmul_quantized, but the scratch the routes need (quantized activations, K-split
 * partial sums, the prefill GEMM's sub-block sums) comes from a static device array of
 * MARMOT_HIP_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends; the call allocates
 * and frees nothing. A shape that needs more returns MARMOT_HIP_ERROR_INVALID_ARGUMENT with the two sizes in the error
 * text. Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two device objects, two threads)
 * race, and the array keeps the last call's contents (no kernel of these routes reads scratch it has not written). */
#define MARMOT_HIP_NOALLOC_SCRATCH_BYTES (8u << 20)
int marmot_hip_matmul_quantized_noalloc(marmot_hip_device_t *dev, int kind, const void *d_weight, const void *d_input,
                                        int in_dtype, size_t N, size_t K, size_t M, const void *d_bias,
                                        int bias_dtype, void *d_out, int out_dtype, uint32_t flags);

/* Replaces cpu_matmul_quantized_dual_output (matmul_quant_dispatch.c:593-856): two weights of the same
 * kind and shape applied to one input with a single activation quantization (gate/up projections). */
int marmot_hip_matmul_quantized_dual(marmot_hip_device_t *dev, int kind, const void *d_weight_a,
                                     const void *d_weight_b, const void *d_input, int in_dtype, size_t N, size_t K,
                                     size_t M, void *d_out_a, void *d_out_b, int out_dtype, uint32_t flags);

/* Fused Q/K/V projection, separate weights. Replaces cpu_matmul_qkv_run_separate_quantized_impl
 * (src/backends/cpu/ops/matmul/qkv/matmul_qkv.c:749-947), reached through cpu_matmul_qkv_{q4_k,q6_k,q8_0}
 * (matmul_qkv.c:1498-1532) for marmot_matmul_qkv with MARMOT_QKV_LAYOUT_SEPARATE (include/marmot/ops/matmul.h:74-95).
 * Three weights of one kind and one shape [M,K] are applied to one input [N,K]; the activations are quantized once
 * (Q8_0 for Q4_0/Q8_0 weights, Q8_K for K-quants: F16 input is packed too, there is no direct F16 route here) and
 * out_x[n*M + m] = (float)bias_x[m] + dot(Wx[m,:], act[n,:]), one rounding to the output type at the store.
 *   d_input          : [N,K] of in_dtype (F32 or F16), row-major
 *   d_bq, d_bk, d_bv : each NULL or M values of bias_dtype (F32 or F16)
 *   d_out_*          : [N,M] of out_dtype, which must equal in_dtype (matmul_qkv.c:769-772)
 * The rotary epilogue of the reference op (rope_params) is the _rope variant below. */
int marmot_hip_matmul_qkv_quantized(marmot_hip_device_t *dev, int kind, const void *d_wq, const void *d_wk,
                                    const void *d_wv, const void *d_input, int in_dtype, size_t N, size_t K, size_t M,
                                    const void *d_bq, const void *d_bk, const void *d_bv, int bias_dtype,
                                    void *d_out_q, void *d_out_k, void *d_out_v, int out_dtype);

/* Rotary epilogue of the Q/K/V projection: cpu_matmul_qkv_apply_rope_row / cpu_matmul_qkv_rotate_row_f32_headed
 * (matmul_qkv.c:700-747, matmul_qkv_rope.h:50-70, 123-138). q and/or k rows are rotated in FLOAT32 before the one
 * rounding of the store: per head of head_dim values and pair i, angle = (float)position[n] * freqs[i],
 * (even, odd) -> (even*c - odd*s, even*s + odd*c) with c = cos(angle)*attn_scale, s = sin(angle)*attn_scale;
 * pairs are (2i, 2i+1) for rope_type 0 (NORM) and (i, i + head_dim/2) for 1 (NEOX). */
typedef struct marmot_hip_rope {
    const void *d_positions; /* N values of positions_dtype: F32, I32 or I64 (cpu_backend_internal.h:567-578) */
    int positions_dtype;
    const float *d_freqs;    /* head_dim / 2 angular frequencies in device memory (marmot_hip_rope_frequencies) */
    float attn_scale;
    uint32_t head_dim;       /* even, divides M (after cpu_matmul_qkv_resolve_head_dim, matmul_qkv_rope.h:14-23) */
    int rope_type;
    int apply_to_q, apply_to_k;
} marmot_hip_rope_t;

/* marmot_hip_matmul_qkv_quantized followed by the rotary epilogue; rope == NULL or neither apply flag set is the
 * plain projection. */
int marmot_hip_matmul_qkv_rope_quantized(marmot_hip_device_t *dev, int kind, const void *d_wq, const void *d_wk,
                                         const void *d_wv, const void *d_input, int in_dtype, size_t N, size_t K,
                                         size_t M, const void *d_bq, const void *d_bk, const void *d_bv,
                                         int bias_dtype, void *d_out_q, void *d_out_k, void *d_out_v, int out_dtype,
                                         const marmot_hip_rope_t *rope);

/* Host-side: the head_dim/2 angular frequencies and the attention scale of marmot_rope_freq_cache_ensure
 * (src/core/helpers/rope.c:61-127, 143-200) for marmot_rope_params_t fields (include/marmot/ops_types.h:98-112);
 * scaling_type as marmot_rope_scaling_type_t (include/marmot/types.h:254-261). head_dim is resolved against M as
 * cpu_matmul_qkv_resolve_head_dim does and returned in *head_dim_out. freqs_out: host array of at least M/2 floats.
 * Includes the YaRN ramp (a non-zero extrapolation factor with a valid original context: correction range
 * rope.c:38-59, ramp :28-36, attention scale :95-99). */
int marmot_hip_rope_frequencies(int scaling_type, float theta, float freq_scale, float ext_factor,
                                float attn_factor, float beta_fast, float beta_slow, uint32_t orig_ctx_len,
                                uint32_t head_dim, size_t M, float *freqs_out, float *attn_scale_out,
                                uint32_t *head_dim_out);

/* ------------------------------------------------------------------ quantized embedding gather
 * Replaces cpu_embedding_gather_scalar for block-quantized tables (cpu_embedding_run_worker and
 * cpu_embedding_copy_row_quantized, src/backends/cpu/ops/embedding/scalar/embedding_scalar.c:241-303, 381-447;
 * descriptor marmot_embedding_gather_desc_t, include/marmot/ops_types.h:160-170).
 *   d_table : vocab rows of marmot_hip_row_bytes(kind, dim) bytes (any weight kind)
 *   d_ids   : n token ids of ids_dtype (MARMOT_HIP_DTYPE_I32 or _I64)
 *   d_out   : [n, dim] of out_dtype (F32 or F16): decoded value * scale, one rounding for F16
 * A token equal to padding_id (when padding_id >= 0) gives a zero row. A token outside [0, vocab) gives a zero row,
 * or MARMOT_HIP_ERROR_INVALID_ARGUMENT when bounds_check is non-zero (the ids are then read back and checked on the
 * host before the launch; not possible, and skipped, while a graph is being captured). Q4_0 and Q4_1 tables are
 * decoded in the embedding path's interleaved nibble order (value i = nibble i % 2 of byte i / 2,
 * embedding_scalar.c:221-240), the other kinds bit-exactly like marmot_hip_dequantize. */
int marmot_hip_embedding_gather_quantized(marmot_hip_device_t *dev, int kind, const void *d_table, size_t vocab,
                                          size_t dim, const void *d_ids, int ids_dtype, size_t n, void *d_out,
                                          int out_dtype, float scale, int32_t padding_id, int bounds_check);

/* ------------------------------------------------------------------ pre-packed activations
 * The reference packs (quantizes) a tile of activations once and then runs the row kernels against the packed
 * tile: cpu_quant_matmul_pack_column (matmul_quant_dispatch.c:270-302) followed by
 * cpu_quant_matmul_dispatch_quant_tile (matmul_quant_compute.c:1958-1990). These three entry points expose the
 * same split, so that several weights sharing one input (q/k/v, gate/up) pay for one quantization.
 * The packed buffer has a library-private layout; only its size is public. */
size_t marmot_hip_packed_activation_bytes(int weight_kind, size_t N, size_t K);
/* Where the parts of a packed buffer lie, for tests and tools that inspect or build one on the host. Row n holds
 * values_per_row int8 values at values_offset + n*values_per_row (the row padded with zeros to whole blocks),
 * blocks_per_row fp32 block scales at scales_offset + 4*n*blocks_per_row, and blocks_per_row*sums_per_block int16
 * sums at sums_offset (Q8_K: the 16 sums of 16 values, marmot_q8_k_block_t.bsums; Q8_0: the sum of the block's 32
 * values). The layout may change between versions of the library; the packed size is total_bytes. */
typedef struct marmot_hip_packed_layout {
    int act_kind; /* MARMOT_HIP_KIND_Q8_0 or MARMOT_HIP_KIND_Q8_K */
    size_t total_bytes;
    size_t values_offset, values_per_row;
    size_t scales_offset, blocks_per_row;
    size_t sums_offset, sums_per_block;
} marmot_hip_packed_layout_t;
int marmot_hip_packed_activation_layout(int weight_kind, size_t N, size_t K, marmot_hip_packed_layout_t *layout);
int marmot_hip_pack_activations(marmot_hip_device_t *dev, int weight_kind, const void *d_input, int in_dtype,
                                size_t N, size_t K, void *d_packed);
int marmot_hip_matmul_prepacked(marmot_hip_device_t *dev, int kind, const void *d_weight, const void *d_packed,
                                size_t N, size_t K, size_t M, const void *d_bias, int bias_dtype, void *d_out,
                                int out_dtype);

/* ------------------------------------------------------------------ ops between the linears
 * The fp32 operations a decoder layer runs between its quantized linears, and the fused forms that hand the next
 * linear its activations already packed (marmot_hip_matmul_prepacked and the prepacked forms of the q/k/v and gate/up
 * projections then start without a quantization launch).
 *
 * marmot_hip_rms_norm replaces cpu_rmsnorm_impl (weight_offset 0) and cpu_rmsnorm_gemma_impl (weight_offset 1)
 * for fp32 tensors (src/backends/cpu/ops/normalization/normalization_dispatch.c:129-181, 240-246;
 * scalar/normalization_scalar.c:469-510, 780-791): per row of `cols` values,
 *   v = x (+ residual);  out = v * (1 / sqrt(mean(v^2) + eps)) * (weight + weight_offset)
 * d_residual and d_weight may be null (no residual; no scaling). The mean of squares is summed by 256 threads, not
 * sequentially: results agree with the scalar CPU loop to a few units in the last place.
 * marmot_hip_rms_norm_pack writes the same rows as packed activations for a linear of weight_kind (layout and size
 * of marmot_hip_pack_activations) and, when d_out is not null, as fp32 too; the packed rows are bit-identical to
 * marmot_hip_pack_activations applied to the fp32 output. */
int marmot_hip_rms_norm(marmot_hip_device_t *dev, const float *d_x, const float *d_residual, const float *d_weight,
                        float weight_offset, float eps, size_t rows, size_t cols, float *d_out);
int marmot_hip_rms_norm_pack(marmot_hip_device_t *dev, const float *d_x, const float *d_residual,
                             const float *d_weight, float weight_offset, float eps, size_t rows, size_t cols,
                             int weight_kind, float *d_out, void *d_packed);
/* Replaces cpu_swiglu_f32_scalar / cpu_geglu_f32_scalar (src/backends/cpu/ops/elementwise/scalar/
 * elementwise_f32_scalar.c:11-20, 147-214): out = silu(gate) * up, or gelu_tanh(gate) * up for MARMOT_HIP_FFN_GEGLU
 * (the tanh form; the MoE expert body uses the erf form, moe_ops.c:321-324). Row strides in elements.
 * marmot_hip_swiglu_pack writes silu(gate) * up of contiguous rows as packed activations for a linear of weight_kind. */
int marmot_hip_glu(marmot_hip_device_t *dev, int ffn_type, const float *d_gate, const float *d_up, size_t rows,
                   size_t cols, size_t gate_stride, size_t up_stride, size_t out_stride, float *d_out);
int marmot_hip_swiglu_pack(marmot_hip_device_t *dev, const float *d_gate, const float *d_up, size_t rows, size_t cols,
                           int weight_kind, void *d_packed);
/* Replaces cpu_add for contiguous fp32 tensors of equal shape (the residual add). */
int marmot_hip_add(marmot_hip_device_t *dev, const float *d_a, const float *d_b, size_t n, float *d_out);
/* Replaces cpu_rope (src/backends/cpu/ops/rope/rope_dispatch.c:145-372; validation :18-88) for FLOAT32 and FLOAT16
 * rows: d_x and d_out hold `rows` rows of `dim` values at row strides (in elements) >= dim; row r is rotated by
 * positions[r]: angle_i = (float)position * freq_i, cos and sin times attn_scale, pairs (2i, 2i+1) for rope_type 0
 * and (i, i + dim/2) for 1; arithmetic in fp32, one rounding at a FLOAT16 store. rope->d_freqs holds the dim/2
 * frequencies of marmot_hip_rope_frequencies for head_dim == dim (rope->head_dim must say so); the apply flags are
 * not read. d_out == d_x rotates in place; other overlaps are not supported. Errors in the reference's order: odd dim
 * DIMENSION_MISMATCH, empty input INVALID_ARGUMENT, positions type UNSUPPORTED_DTYPE, a stride below dim
 * DIMENSION_MISMATCH. */
int marmot_hip_rope(marmot_hip_device_t *dev, const void *d_x, int dtype, size_t rows, size_t dim,
                    size_t x_row_stride, size_t out_row_stride, const marmot_hip_rope_t *rope, void *d_out);

/* ------------------------------------------------------------------ tensor operations around the linears
 * The nodes a GGUF model graph places between its quantized linears besides the ones above (graph_builder.cpp:555-1140),
 * so that a graph's values can stay on the device from the embedding to the logits. */
enum {
    MARMOT_HIP_UNARY_GELU = 0,      /* x * 0.5 * (1 + erf(x / sqrt 2)) */
    MARMOT_HIP_UNARY_GELU_TANH = 1, /* 0.5 * x * (1 + tanh(sqrt(2 / pi) * (x + 0.044715 x^3))) */
    MARMOT_HIP_UNARY_SILU = 2,      /* x / (1 + exp(-x)) */
};
/* Replaces cpu_unary_gelu / _gelu_tanh / _silu for FLOAT32 and FLOAT16 values (gelu_scalar, gelu_tanh_scalar,
 * silu_scalar_fn, src/backends/cpu/ops/unary/scalar/unary_scalar.c:201-218): n contiguous values of `dtype`, fp32
 * arithmetic in the reference's expression order, FLOAT16 rounded once at the store. d_out may be d_x. */
int marmot_hip_unary(marmot_hip_device_t *dev, int op, const void *d_x, int dtype, size_t n, void *d_out);
/* Replaces cpu_softmax_impl for FLOAT32 (src/backends/cpu/ops/softmax/softmax_dispatch.c:67-103 ->
 * softmax_f32_scalar.c:30-83): a contiguous tensor seen as [outer, axis, inner], normalized along `axis`
 * (marmot_softmax_prepare, src/core/helpers/norm.c:123-179, yields the three sizes): maximum, exp(x - max) with
 * differences at or below -88 giving exactly 0, sum, one multiplication by 1 / sum. d_out may be d_x. */
int marmot_hip_softmax(marmot_hip_device_t *dev, const float *d_x, size_t outer, size_t axis, size_t inner,
                       float *d_out);
/* The same for a tensor of `dtype` FLOAT32, FLOAT16 or BFLOAT16 (input and output of one type). The 16-bit types follow
 * softmax_f16_scalar / softmax_bf16_scalar (src/backends/cpu/ops/softmax/scalar/softmax_misc_scalar.c:4-62, 64-122):
 * maximum and sum in FLOAT32, each exponential rounded to the type when stored (the sum takes the unrounded value),
 * and the stored value times 1 / sum rounded again. d_out may be d_x. */
int marmot_hip_softmax_typed(marmot_hip_device_t *dev, int dtype, const void *d_x, size_t outer, size_t axis,
                             size_t inner, void *d_out);
/* Replaces cpu_convert_{f32,f16,bf16}_to_{f32,f16,bf16} (src/backends/cpu/ops/convert/dtype_convert.c:17-130 and the
 * bridges through FLOAT32, src/utils/dtype_ref.c:106-114): n contiguous values; to FLOAT16 and to BFLOAT16 round to
 * nearest even (the reference's vector body; its scalar tail of n % 8 values truncates FLOAT16, dtype_ref.c:14-50,
 * which is not reproduced). Equal types copy. */
int marmot_hip_convert(marmot_hip_device_t *dev, void *d_dst, int dst_dtype, const void *d_src, int src_dtype,
                       size_t n);
/* Replaces cpu_gather_rows (src/backends/cpu/ops/tensor_ops/tensor_ops.c:464-547): out row r = x row idx[r * idx_stride]
 * for r < rows_out <= 65535; rows of row_bytes bytes at the given byte strides; indices MARMOT_HIP_DTYPE_I32 or _U32.
 * An index outside [0, rows_in) returns MARMOT_HIP_ERROR_INVALID_ARGUMENT "gather_rows index out of range" (device
 * flag read back: one stream synchronization, skipped while a graph is being captured, where such rows are zeroed). */
int marmot_hip_gather_rows(marmot_hip_device_t *dev, const void *d_x, size_t rows_in, size_t row_bytes,
                           size_t in_stride_bytes, const void *d_idx, int idx_dtype, size_t idx_stride, size_t rows_out,
                           void *d_out, size_t out_stride_bytes);
/* Replaces cpu_slice (tensor_ops.c:401-462): the box [starts, starts + sizes) of a contiguous tensor of shape
 * in_shape (ndim <= 8 dimensions, elements of 1, 2, 4 or 8 bytes) copied into a contiguous tensor of shape sizes.
 * The three arrays are host memory and are read before the call returns. */
int marmot_hip_slice(marmot_hip_device_t *dev, const void *d_x, size_t elem_size, int ndim, const size_t *in_shape,
                     const size_t *starts, const size_t *sizes, void *d_out);

/* ------------------------------------------------------------------ paged attention
 * Replaces cpu_paged_attention_impl (src/backends/cpu/ops/paged_attention/paged_attention_ref.c:573-1082; descriptor
 * marmot_paged_attention_desc_t, include/marmot/ops/paged_attention.h:32-57) for FLOAT32 / FLOAT16 / BFLOAT16
 * activations and FLOAT32 / FLOAT16 / BFLOAT16 / FLOAT8_E4M3 KV caches. The tensors of the descriptor
 * arrive as device pointers with their strides in elements:
 *   d_token_meta  [token_count, 4] uint32: seq_slot, pos, kv_slot, flags (flags are not read)
 *   d_q, d_out    [tokens, num_q_heads, head_dim], d_k_new, d_v_new [tokens, num_kv_heads, head_dim] of act_dtype
 *   d_kv_k, d_kv_v [kv_blocks, kv_layers, num_kv_heads, block_size, head_dim] of kv_dtype, updated in place
 *   d_block_table [max_seqs, max_blocks_per_seq] uint32, 0xFFFFFFFF = no block
 * First every token's new key / value rows are stored at its kv_slot (block = kv_slot / block_size, same storage
 * type: the same bits, otherwise one conversion through FLOAT32), then out[t, h] = softmax(scale * q[t, h] . K) V over
 * positions 0 .. pos of the token's sequence read through the block table (positions without a block are skipped, a
 * token with no position gives zeros); FLOAT32 arithmetic, one rounding at the store. head_dim up to 256.
 * validate_meta != 0: seq_slot and kv_slot ranges are checked on the device before anything is written and
 * MARMOT_HIP_ERROR_DIMENSION_MISMATCH is returned (one stream synchronization; skipped while a graph is being
 * captured). Without the check, tokens with an out-of-range slot are skipped. */
typedef struct marmot_hip_paged_attention {
    uint32_t token_count, layer_idx, num_q_heads, num_kv_heads, head_dim, block_size;
    float scale;
    int act_dtype, kv_dtype;
    const uint32_t *d_token_meta;
    size_t meta_stride[2];
    const void *d_q, *d_k_new, *d_v_new;
    size_t q_stride[3], k_stride[3], v_stride[3];
    void *d_kv_k, *d_kv_v;
    size_t kv_stride[5];
    size_t kv_blocks, kv_layers;
    const uint32_t *d_block_table;
    size_t table_stride[2];
    size_t max_seqs, max_blocks_per_seq;
    void *d_out;
    size_t out_stride[3];
    /* kv_dtype == MARMOT_HIP_DTYPE_F8_E4M3 (paged_attention_ref.c:825-989): fp32 scales [kv_blocks, kv_layers,
     * num_kv_heads] for keys and for values at scale_stride, read and updated. A block's scale becomes the largest
     * magnitude among its rows below the first offset this call writes (decoded with the old scale) and the new rows,
     * divided by 240; rows already in the block are re-encoded when the scale changes; bytes and scales equal the
     * reference's bit for bit (its e4m3: bias 7, exponent field 15 = NaN, src/utils/dtype_ref.c:118-212). */
    float *d_kv_k_scale, *d_kv_v_scale;
    size_t scale_stride[3];
} marmot_hip_paged_attention_t;
int marmot_hip_paged_attention(marmot_hip_device_t *dev, const marmot_hip_paged_attention_t *args, int validate_meta);

/* ------------------------------------------------------------------ MoE
 * Replaces cpu_topk_impl (src/backends/cpu/ops/moe/moe_ops.c:789-889): top-k over the last axis of
 * fp32 x[rows,cols], ties to the lower index; values fp32 [rows,k], indices int32 [rows,k]. */
int marmot_hip_topk(marmot_hip_device_t *dev, const float *d_x, size_t rows, size_t cols, size_t k,
                    float *d_values, int32_t *d_indices);
/* Softmax over each row of k selected logits (router policy SOFTMAX_SELECTED*,
 * src/graph/gguf/graph_builder.cpp:2276-2316). */
int marmot_hip_softmax_rows(marmot_hip_device_t *dev, const float *d_x, size_t rows, size_t k, float *d_out);

/* Replaces cpu_moe_experts_impl for fp32 activations and block-quantized experts
 * (src/backends/cpu/ops/moe/moe_ops.c:891-1049, 506-568, 1069-1178).
 *   d_hidden [T,H] fp32; d_gate/d_up: E slices of [F rows, H] blocks of kind_gate_up;
 *   d_down: E slices of [H rows, F] blocks of kind_down; d_topk_ids int32 [T,k]; d_topk_weights fp32 [T,k];
 *   d_out [T,H] fp32 (fully overwritten). */
int marmot_hip_moe_experts(marmot_hip_device_t *dev, const float *d_hidden, size_t T, size_t H, size_t F, size_t E,
                           size_t k_per_token, int kind_gate_up, int kind_down, const void *d_gate, const void *d_up,
                           const void *d_down, const int32_t *d_topk_ids, const float *d_topk_weights,
                           float weights_scale, int router_weight_policy, int ffn_type, float *d_out);

/* DIAGNOSTIC (test hook, not an operator; no counterpart in the reference's backend interface). The same call with its
 * stages observable, for parity tests that check each stage of cpu_moe_experts_impl
 * (moe_ops.c:951-1042: gate/up projections, the quantized GLU product, down projection + combine) against a CPU
 * restatement instead of only the final sum. Every pointer may be null. Outputs are in expert-sorted route order
 * (moe_ops.c:929-943); d_route_pos[t*k + j] is the sorted position of token t's j-th route, -1 if it was dropped.
 *   d_sorted_tokens uint32 [T*k]; d_gate_out / d_up_out fp32 [T*k, F];
 *   d_fused_packed: the packed activations of [T*k, F] the down projection reads, in the layout and size of
 *     marmot_hip_pack_activations (see marmot_hip_packed_activation_layout) for kind_down;
 *   d_fused_override: packed activations in the same layout that REPLACE them before the down projection.
 * Not capturable into a graph (it copies with the runtime's copy engine). */
typedef struct marmot_hip_moe_probe {
    uint32_t *d_sorted_tokens;
    int32_t *d_route_pos;
    float *d_gate_out;
    float *d_up_out;
    void *d_fused_packed;
    const void *d_fused_override;
} marmot_hip_moe_probe_t;
int marmot_hip_moe_experts_probe(marmot_hip_device_t *dev, const float *d_hidden, size_t T, size_t H, size_t F,
                                 size_t E, size_t k_per_token, int kind_gate_up, int kind_down, const void *d_gate,
                                 const void *d_up, const void *d_down, const int32_t *d_topk_ids,
                                 const float *d_topk_weights, float weights_scale, int router_weight_policy,
                                 int ffn_type, float *d_out, const marmot_hip_moe_probe_t *probe);

/* ------------------------------------------------------------------ GGUF files
 * Replaces, for the weights of this path, marmot_gguf_load / marmot_gguf_find_tensor (src/graph/gguf/loader.cpp:577-770,
 * 808-818) and the tensor views they build (set_tensor_data_views, :492-575): the file is mapped read-only, the
 * key/value table is skipped except general.alignment, every tensor becomes a view into the mapping. Shapes follow the
 * loader: matrices are [rows, cols] = [ne1, ne0], other ranks keep the file's order (expert stacks [cols, rows,
 * experts]); ggml types map to quant kinds as in map_ggml_type (:300-490), dense F32 / F16 / I32 tensors have kind 0.
 * The views are host memory: the tensor-level backend mirrors a view on first use (the residency table), and
 * marmot_hip_gguf_upload copies one tensor into a fresh device allocation for callers of this raw-pointer ABI
 * (counterpart of the upload in ExecutionSession, src/graph/execution_session.cpp:315-320; free with
 * marmot_hip_free). Views stay valid until marmot_hip_gguf_close. */
#define MARMOT_HIP_GGUF_MAX_DIMS 4
typedef struct marmot_hip_gguf marmot_hip_gguf_t;
typedef struct {
    const char *name;
    uint32_t ggml_type;
    int kind;           /* MARMOT_HIP_KIND_*, 0 for a dense tensor */
    int dtype;          /* MARMOT_HIP_DTYPE_U8 for quantized tensors, else F32 / F16 / I32 */
    uint32_t ndim;
    uint64_t shape[MARMOT_HIP_GGUF_MAX_DIMS];
    const void *data;   /* inside the mapping */
    size_t nbytes;
} marmot_hip_gguf_tensor_t;
int marmot_hip_gguf_open(const char *path, marmot_hip_gguf_t **out);
void marmot_hip_gguf_close(marmot_hip_gguf_t *g);
size_t marmot_hip_gguf_tensor_count(const marmot_hip_gguf_t *g);
size_t marmot_hip_gguf_alignment(const marmot_hip_gguf_t *g);
int marmot_hip_gguf_tensor(const marmot_hip_gguf_t *g, size_t index, marmot_hip_gguf_tensor_t *out);
int marmot_hip_gguf_find(const marmot_hip_gguf_t *g, const char *name, marmot_hip_gguf_tensor_t *out);
int marmot_hip_gguf_upload(marmot_hip_device_t *dev, const marmot_hip_gguf_t *g, size_t index, void **d_out);

/* Key/value metadata of the file (marmot_gguf_find_kv, include/marmot/graph/gguf_loader.h:165; the value kinds of
 * marmot_gguf_value_type_t :72-86). Entries are views into the mapping, valid until marmot_hip_gguf_close:
 *   type      GGUF value type (0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string, 9 array, 10 u64,
 *             11 i64, 12 f64); elem_type: element type of an array, else 0
 *   count     elements of an array, else 1
 *   data      scalar: its little-endian bytes (unaligned); string: its characters (not NUL-terminated); array of
 *             scalars: the elements; array of strings: the first length-prefixed string
 *   nbytes    bytes of that payload
 * The typed readers take an element index (0 for a scalar or a plain string): _int for the integer and bool types,
 * _float for every numeric type, _string for a string or an element of a string array. */
typedef struct {
    const char *key;    /* NUL-terminated */
    uint32_t type;
    uint32_t elem_type;
    uint64_t count;
    const void *data;
    size_t nbytes;
} marmot_hip_gguf_kv_t;
size_t marmot_hip_gguf_kv_count(const marmot_hip_gguf_t *g);
int marmot_hip_gguf_kv(const marmot_hip_gguf_t *g, size_t index, marmot_hip_gguf_kv_t *out);
int marmot_hip_gguf_find_kv(const marmot_hip_gguf_t *g, const char *key, marmot_hip_gguf_kv_t *out);
int marmot_hip_gguf_kv_int(const marmot_hip_gguf_kv_t *kv, uint64_t index, int64_t *out);
int marmot_hip_gguf_kv_float(const marmot_hip_gguf_kv_t *kv, uint64_t index, double *out);
int marmot_hip_gguf_kv_string(const marmot_hip_gguf_kv_t *kv, uint64_t index, const char **chars, size_t *length);

/* ------------------------------------------------------------------ introspection
 * Name of the kernel route the last marmot_hip_matmul_quantized call on this thread took
 * (counterpart of the reference's MARMOT_METAL_LOG_MATMUL_QUANT route log,
 * src/backends/metal/ops/matmul_quant_dispatch.mm:30-70). */
const char *marmot_hip_last_route(void);
const char *marmot_hip_version(void);

#ifdef __cplusplus
}
#endif

#endif /* MARMOT_HIP_H */

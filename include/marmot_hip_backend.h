/*
 * marmot_hip_backend.h — the marmot_tensor_t-level face of MARMOT_BACKEND_HIP.
 *
 * marmot has no plugin loader: a backend is compiled into libmarmot and reached through four tables
 * (paths relative to the reference tree):
 *   1. the device vtable      marmot_device_ops_t            include/marmot/device.h:43-66
 *   2. the kernel query       marmot_<backend>_query_kernel  src/core/dispatch/kernel_query.c:35-52
 *   3. the bytecode tables    marmot_bc_get_tables           src/core/bytecode/bytecode_compile.c:128-156
 *   4. the impl functions the generated dispatch shims call  src/backends/cpu/kernels/matmul_quantized_scalar.def:3-19,
 *                                                            src/backends/cpu/kernels/moe.def:3-73
 * This header declares the HIP backend's entry for each of them. The functions sit on top of the raw-pointer
 * C ABI of marmot_hip.h and live in the same shared library.
 *
 * Types. Inside the marmot tree, define MARMOT_HIP_IN_TREE before including this header: the real marmot
 * headers are used. Outside (this repository's tests and harness), the header declares the subset of marmot's
 * public types the backend touches, with the same names, member order and enumerator values, so that objects
 * built either way are ABI-compatible. Every mirrored type cites the definition it follows.
 */
#ifndef MARMOT_HIP_BACKEND_H
#define MARMOT_HIP_BACKEND_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef MARMOT_HIP_IN_TREE
#include "marmot/marmot.h"
#include "core/bytecode/bytecode.h"
#include "core/bytecode/bytecode_compile.h"
#include "core/dispatch/kernel_query.h"
#else

#ifdef __cplusplus
extern "C" {
#endif

/* include/marmot/types.h:18 */
enum { MARMOT_MAX_DIMS = 8 };

/* include/marmot/types.h:210-220 */
typedef enum {
    MARMOT_SUCCESS = 0,
    MARMOT_ERROR_INVALID_ARGUMENT = -1,
    MARMOT_ERROR_OUT_OF_MEMORY = -2,
    MARMOT_ERROR_DEVICE_NOT_AVAILABLE = -3,
    MARMOT_ERROR_BACKEND_INIT_FAILED = -4,
    MARMOT_ERROR_INVALID_OPERATION = -5,
    MARMOT_ERROR_UNSUPPORTED_DTYPE = -6,
    MARMOT_ERROR_DIMENSION_MISMATCH = -7,
    MARMOT_ERROR_NOT_IMPLEMENTED = -8,
} marmot_error_t;

/* include/marmot/types.h:222-228; HIP takes the next free value */
typedef enum {
    MARMOT_BACKEND_CPU = 0,
    MARMOT_BACKEND_METAL = 1,
    MARMOT_BACKEND_CUDA = 2,
} marmot_backend_type_t;

/* include/marmot/types.h:230-234 */
typedef enum {
    MARMOT_ROUTING_ALWAYS_CPU = 0,
    MARMOT_ROUTING_ALWAYS_GPU = 1,
    MARMOT_ROUTING_AUTO = 2,
} marmot_routing_policy_t;

/* include/marmot/types.h:281-293 */
typedef enum {
    MARMOT_FFN_SWIGLU = 0,
    MARMOT_FFN_GELU = 1,
    MARMOT_FFN_GEGLU = 2,
    MARMOT_FFN_COUNT,
} marmot_ffn_type_t;

typedef enum {
    MARMOT_ROUTER_WEIGHT_POLICY_SOFTMAX_SELECTED = 0,
    MARMOT_ROUTER_WEIGHT_POLICY_SOFTMAX_SELECTED_SCALED = 1,
    MARMOT_ROUTER_WEIGHT_POLICY_RENORMALIZE_SELECTED = 2,
    MARMOT_ROUTER_WEIGHT_POLICY_COUNT,
} marmot_router_weight_policy_t;

/* include/marmot/types.h:344-364 */
typedef enum {
    MARMOT_DTYPE_FLOAT32 = 0,
    MARMOT_DTYPE_FLOAT16 = 1,
    MARMOT_DTYPE_BFLOAT16 = 2,
    MARMOT_DTYPE_INT32 = 3,
    MARMOT_DTYPE_INT16 = 4,
    MARMOT_DTYPE_INT8 = 5,
    MARMOT_DTYPE_UINT8 = 6,
    MARMOT_DTYPE_UINT16 = 7,
    MARMOT_DTYPE_UINT32 = 8,
    MARMOT_DTYPE_UINT64 = 9,
    MARMOT_DTYPE_FLOAT64 = 10,
    MARMOT_DTYPE_INT64 = 11,
    MARMOT_DTYPE_INT4 = 12,
    MARMOT_DTYPE_UINT4 = 13,
    MARMOT_DTYPE_FLOAT8_E4M3 = 14,
    MARMOT_DTYPE_FLOAT8_E5M2 = 15,
    MARMOT_DTYPE_COUNT,
} marmot_dtype_t;

/* include/marmot/types.h:366-370 */
typedef enum {
    MARMOT_QUANT_LAYOUT_GENERIC = 0,
    MARMOT_QUANT_LAYOUT_GGUF = 1,
    MARMOT_QUANT_LAYOUT_COUNT,
} marmot_quant_layout_t;

/* include/marmot/types.h:372-388 */
typedef enum {
    MARMOT_QUANT_KIND_GENERIC = 0,
    MARMOT_QUANT_KIND_Q4_0 = 1,
    MARMOT_QUANT_KIND_Q4_1 = 2,
    MARMOT_QUANT_KIND_Q5_0 = 3,
    MARMOT_QUANT_KIND_Q5_1 = 4,
    MARMOT_QUANT_KIND_Q8_0 = 5,
    MARMOT_QUANT_KIND_Q8_1 = 6,
    MARMOT_QUANT_KIND_Q2_K = 7,
    MARMOT_QUANT_KIND_Q3_K = 8,
    MARMOT_QUANT_KIND_Q4_K = 9,
    MARMOT_QUANT_KIND_Q5_K = 10,
    MARMOT_QUANT_KIND_Q6_K = 11,
    MARMOT_QUANT_KIND_Q8_K = 12,
    MARMOT_QUANT_KIND_COUNT,
} marmot_quant_kind_t;

/* include/marmot/types.h:392-409: only the size of the enumeration matters to the backend */
typedef enum {
    MARMOT_CPU_UNKNOWN = 0,
} marmot_cpu_microarch_t;

/* include/marmot/types.h:415-425 */
typedef struct {
    size_t ndim;
    size_t shape[MARMOT_MAX_DIMS];
    size_t strides[MARMOT_MAX_DIMS];
} marmot_shape_t;

typedef struct {
    float scale;
    float zero_point;
    size_t block_size;
} marmot_quant_params_t;

/* include/marmot/tensor.h:10-38 */
struct marmot_context;
typedef struct marmot_context marmot_context_t;

typedef enum marmot_memory_location {
    MARMOT_MEMORY_HOST = 0,
    MARMOT_MEMORY_DEVICE = 1,
    MARMOT_MEMORY_UNIFIED = 2,
    MARMOT_MEMORY_UNKNOWN = 3
} marmot_memory_location_t;

struct marmot_tensor {
    marmot_shape_t shape;
    marmot_dtype_t dtype;
    void *data;
    size_t capacity_bytes;
    bool owns_data;
    marmot_quant_params_t *quant_params;
    marmot_quant_kind_t quant_kind;
    marmot_quant_layout_t quant_layout;
    marmot_backend_type_t backend;
    marmot_context_t *ctx;
    marmot_memory_location_t memory_location;
    bool needs_sync;
    void *packed_data;
    const void *packed_src_data;
    size_t packed_bytes;
    size_t packed_row_bytes;
    size_t packed_rows;
};
typedef struct marmot_tensor marmot_tensor_t;

/* include/marmot/allocator.h:27-36 */
typedef struct {
    size_t current_bytes;
    size_t peak_bytes;
    size_t pooled_bytes;
    size_t active_allocations;
    size_t peak_allocations;
    uint64_t total_allocations;
    uint64_t pool_hits;
    uint64_t pool_misses;
} marmot_allocator_usage_t;

/* include/marmot/device.h:20-36 */
typedef enum {
    MARMOT_QUANT_ACTIVATION_AUTO = 0,
    MARMOT_QUANT_ACTIVATION_FORCE_DIRECT = 1,
} marmot_quant_activation_mode_t;

typedef struct {
    marmot_dtype_t embedding_quant_output_dtype;
    marmot_quant_activation_mode_t quant_activation_mode;
    uint32_t variant_flags_mask;
    bool embedding_prefer_gpu_private;
    bool embedding_allow_quant_decode_on_the_fly;
    bool matmul_requires_temp_tensors;
    bool matmul_prefer_packed_weights;
} marmot_context_policy_t;

/* include/marmot/device.h:43-66 */
struct marmot_device_ops {
    marmot_error_t (*init)(void **device_ctx);
    void (*destroy)(const void *device_ctx);
    marmot_error_t (*configure)(const void *device_ctx, const marmot_context_t *ctx);
    marmot_error_t (*alloc)(const void *device_ctx, size_t size, void **ptr);
    void (*free)(const void *device_ctx, void *ptr);
    marmot_error_t (*memcpy_to_device)(const void *device_ctx, void *dst, const void *src, size_t size);
    marmot_error_t (*memcpy_from_device)(const void *device_ctx, void *dst, const void *src, size_t size);
    marmot_error_t (*synchronize)(const void *device_ctx);
    marmot_error_t (*allocator_usage)(const void *device_ctx, marmot_allocator_usage_t *usage);
    marmot_error_t (*graph_batch_begin)(void *device_ctx);
    marmot_error_t (*graph_batch_end)(void *device_ctx, bool commit);
    void (*on_host_ptr_freed)(void *device_ctx, const void *ptr);
    void (*on_host_range_freed)(void *device_ctx, const void *start, size_t length);
};
typedef struct marmot_device_ops marmot_device_ops_t;

/* include/marmot/ops_types.h:114-118 */
struct marmot_matmul_epilogue {
    const marmot_tensor_t *bias;
    bool enable_output_cast;
    marmot_dtype_t output_dtype;
};
typedef struct marmot_matmul_epilogue marmot_matmul_epilogue_t;

/* include/marmot/ops_types.h:195-214 */
struct marmot_topk_desc {
    const marmot_tensor_t *x;
    marmot_tensor_t *values_out;
    marmot_tensor_t *indices_out;
    int32_t axis;
    uint32_t k;
};
typedef struct marmot_topk_desc marmot_topk_desc_t;

/* include/marmot/ops_types.h:189-193 */
struct marmot_softmax_desc {
    const marmot_tensor_t *x;
    marmot_tensor_t *out;
    int32_t axis;
};
typedef struct marmot_softmax_desc marmot_softmax_desc_t;

/* include/marmot/ops_types.h:90-96 */
struct marmot_activation_params {
    const marmot_tensor_t *parameter_tensor;
    const marmot_tensor_t *bias;
    float alpha;
    float beta;
    float gamma;
};
typedef struct marmot_activation_params marmot_activation_params_t;

/* include/marmot/ops_types.h:181-187 */
struct marmot_rmsnorm_desc {
    const marmot_tensor_t *x;
    const marmot_tensor_t *residual;
    const marmot_tensor_t *weight;
    marmot_tensor_t *out;
    float eps;
};
typedef struct marmot_rmsnorm_desc marmot_rmsnorm_desc_t;

struct marmot_moe_experts_desc {
    const marmot_tensor_t *hidden_states;
    const marmot_tensor_t *gate_exps;
    const marmot_tensor_t *up_exps;
    const marmot_tensor_t *down_exps;
    const marmot_tensor_t *topk_ids;
    const marmot_tensor_t *topk_weights;
    marmot_tensor_t *out;
    marmot_ffn_type_t ffn_type;
    float weights_scale;
    marmot_router_weight_policy_t router_weight_policy;
};
typedef struct marmot_moe_experts_desc marmot_moe_experts_desc_t;

/* include/marmot/types.h:254-267 */
typedef enum {
    MARMOT_ROPE_SCALING_UNSPECIFIED = -1,
    MARMOT_ROPE_SCALING_NONE = 0,
    MARMOT_ROPE_SCALING_LINEAR = 1,
    MARMOT_ROPE_SCALING_YARN = 2,
    MARMOT_ROPE_SCALING_LONGROPE = 3,
    MARMOT_ROPE_SCALING_MAX_VALUE = MARMOT_ROPE_SCALING_LONGROPE,
} marmot_rope_scaling_type_t;

typedef enum {
    MARMOT_ROPE_TYPE_NORM = 0,
    MARMOT_ROPE_TYPE_NEOX = 1,
    MARMOT_ROPE_TYPE_MAX_VALUE = MARMOT_ROPE_TYPE_NEOX,
} marmot_rope_type_t;

/* include/marmot/ops_types.h:98-112 */
typedef struct marmot_rope_params {
    const marmot_tensor_t *positions;
    marmot_rope_scaling_type_t scaling_type;
    marmot_rope_type_t rope_type;
    float theta;
    float freq_scale;
    float ext_factor;
    float attn_factor;
    float beta_fast;
    float beta_slow;
    uint32_t orig_ctx_len;
    uint32_t head_dim;
    bool apply_to_q;
    bool apply_to_k;
} marmot_rope_params_t;

/* include/marmot/ops/matmul.h:63-95 */
typedef enum {
    MARMOT_QKV_LAYOUT_UNSPECIFIED = 0,
    MARMOT_QKV_LAYOUT_FUSED = 1,
    MARMOT_QKV_LAYOUT_SEPARATE = 2,
} marmot_matmul_qkv_layout_t;

typedef struct marmot_matmul_qkv_fused {
    const marmot_tensor_t *weight;
    const marmot_tensor_t *bias;
} marmot_matmul_qkv_fused_t;

typedef struct marmot_matmul_qkv_separate {
    const marmot_tensor_t *wq;
    const marmot_tensor_t *wk;
    const marmot_tensor_t *wv;
    const marmot_tensor_t *bq;
    const marmot_tensor_t *bk;
    const marmot_tensor_t *bv;
} marmot_matmul_qkv_separate_t;

typedef struct marmot_matmul_qkv_desc {
    const marmot_tensor_t *input;
    marmot_matmul_qkv_layout_t layout;
    union {
        marmot_matmul_qkv_fused_t fused;
        marmot_matmul_qkv_separate_t separate;
    };
    const marmot_matmul_epilogue_t *epilogue;
    marmot_tensor_t *out_q;
    marmot_tensor_t *out_k;
    marmot_tensor_t *out_v;
    const marmot_rope_params_t *rope_params;
} marmot_matmul_qkv_desc_t;

/* include/marmot/types.h:236-240 */
typedef enum {
    MARMOT_PREFERENCE_DEFAULT = 0,
    MARMOT_PREFERENCE_ENABLE = 1,
    MARMOT_PREFERENCE_DISABLE = 2,
} marmot_preference_t;

/* include/marmot/ops_types.h:160-170 */
struct marmot_embedding_gather_desc {
    const marmot_tensor_t *weights;
    const marmot_tensor_t *token_ids;
    marmot_tensor_t *out;
    marmot_dtype_t dtype_out;
    float scale;
    int32_t padding_id;
    bool bounds_check;
    marmot_preference_t prefer_gpu_private;
    marmot_preference_t allow_quant_decode_on_the_fly;
};
typedef struct marmot_embedding_gather_desc marmot_embedding_gather_desc_t;

/* include/marmot/ops/paged_attention.h:14-19, 32-57 */
#define MARMOT_PAGED_ATTENTION_DESC_VERSION 1
#define MARMOT_PAGED_ATTENTION_KV_SCALE_EXT_VERSION 1
typedef struct {
    uint32_t struct_size;
    uint32_t struct_version;
    const marmot_tensor_t *kv_k_scale;
    const marmot_tensor_t *kv_v_scale;
} marmot_paged_attention_kv_scale_ext_t;
typedef struct {
    uint32_t struct_size;
    uint32_t struct_version;
    uint64_t flags;
    uint32_t token_count;
    uint32_t layer_idx;
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    uint32_t block_size;
    float scale;
    const marmot_tensor_t *token_meta;
    const marmot_tensor_t *q;
    const marmot_tensor_t *k_new;
    const marmot_tensor_t *v_new;
    const marmot_tensor_t *kv_k;
    const marmot_tensor_t *kv_v;
    const marmot_tensor_t *block_table;
    marmot_tensor_t *out;
    const void *pnext;
    uint64_t reserved[4];
} marmot_paged_attention_desc_t;

/* include/marmot/traits_ids.gen.h:40-107 (the operations this backend answers for), :111-116, :120-133 */
typedef enum {
    MARMOT_OP_INVALID = 0,
    MARMOT_OP_QKV_PROJECTION = 191,
    MARMOT_OP_DEQUANTIZE = 210,
    MARMOT_OP_GATHER_ROWS = 244,
    MARMOT_OP_RESHAPE = 258,
    MARMOT_OP_MOE_EXPERTS = 263,
    MARMOT_OP_SWIGLU = 331,
    MARMOT_OP_SILU = 352,
    MARMOT_OP_GEGLU = 410,
    MARMOT_OP_RMS_NORM_GEMMA = 447,
    MARMOT_OP_MATMUL = 498,
    MARMOT_OP_VIEW = 502,
    MARMOT_OP_PAGED_ATTENTION = 503,
    MARMOT_OP_QUANTIZE = 524,
    MARMOT_OP_GELU = 621,
    MARMOT_OP_GELU_TANH = 642,
    MARMOT_OP_LINEAR = 708,
    MARMOT_OP_QKV_SHARED_INPUT = 771,
    MARMOT_OP_QKV_ROPE = 778,
    MARMOT_OP_SLICE = 809,
    MARMOT_OP_ROPE = 843,
    MARMOT_OP_EMBEDDING = 853,
    MARMOT_OP_ADD = 876,
    MARMOT_OP_TOPK = 901,
    MARMOT_OP_RMS_NORM = 929,
    MARMOT_OP_CONVERT = 932,
    MARMOT_OP_SOFTMAX = 994,
    MARMOT_OP_COUNT = 995,
} marmot_op_id_t;

typedef enum {
    MARMOT_PROFILE_INVALID = 0,
    MARMOT_PROFILE_ACCELERATE = 1,
    MARMOT_PROFILE_AVX2 = 2,
    MARMOT_PROFILE_NEON = 3,
    MARMOT_PROFILE_SCALAR = 4,
    MARMOT_PROFILE_COUNT,
} marmot_profile_id_t;

typedef enum {
    MARMOT_QSCHEME_NONE = 0,
    MARMOT_QSCHEME_Q4_0 = 1,
    MARMOT_QSCHEME_Q4_1 = 2,
    MARMOT_QSCHEME_Q5_0 = 3,
    MARMOT_QSCHEME_Q5_1 = 4,
    MARMOT_QSCHEME_Q8_0 = 5,
    MARMOT_QSCHEME_Q2_K = 6,
    MARMOT_QSCHEME_Q3_K = 7,
    MARMOT_QSCHEME_Q4_K = 8,
    MARMOT_QSCHEME_Q5_K = 9,
    MARMOT_QSCHEME_Q6_K = 10,
    MARMOT_QSCHEME_Q8_K = 11,
    MARMOT_QSCHEME_Q8_1 = 12,
    MARMOT_QSCHEME_COUNT,
} marmot_qscheme_id_t;

/* include/marmot/traits_ids.gen.h:136-2103: generated, one id per kernel of every backend. The ids of the HIP
 * kernels are assigned by the code generator once the .def files of this backend are part of the tree; outside
 * the tree the backend numbers them from MARMOT_KERNEL_HIP_BASE. */
typedef enum {
    MARMOT_KERNEL_INVALID = 0,
    MARMOT_KERNEL_HIP_BASE = 0x4000,
} marmot_kernel_id_t;

/* include/marmot/matmul_types.h:10-22 */
typedef struct {
    size_t N;
    size_t K;
    size_t M;
} marmot_matmul_dims_t;

typedef enum {
    MARMOT_MATMUL_LAYOUT_INVALID = 0,
    MARMOT_MATMUL_LAYOUT_NN = 1,
    MARMOT_MATMUL_LAYOUT_NT = 2,
    MARMOT_MATMUL_LAYOUT_TN = 3,
    MARMOT_MATMUL_LAYOUT_TT = 4,
} marmot_matmul_layout_t;

/* include/marmot/ops_types.h:40-61: only the size of the enumeration matters to the backend */
typedef enum {
    MARMOT_DEVICE_UNARY_IDENTITY = 0,
} marmot_device_unary_op_t;

/* include/marmot/graph/op_signature.h:14-92 */
typedef enum {
    MARMOT_WEIGHT_LAYOUT_INVALID = 0,
    MARMOT_WEIGHT_LAYOUT_SEPARATE = 1,
} marmot_weight_layout_t;

typedef enum {
    MARMOT_STRIDE_MODE_ANY = 0,
    MARMOT_STRIDE_MODE_CONTIGUOUS = 1,
    MARMOT_STRIDE_MODE_ROW_STRIDED = 2,
    MARMOT_STRIDE_MODE_STRIDED = 3,
} marmot_stride_mode_t;

typedef enum {
    MARMOT_EPILOGUE_NONE = 0,
    MARMOT_EPILOGUE_BIAS = 1u << 0,
    MARMOT_EPILOGUE_ACTIVATION = 1u << 1,
    MARMOT_EPILOGUE_RESIDUAL = 1u << 2,
    MARMOT_EPILOGUE_ROPE = 1u << 3,
} marmot_epilogue_flags_t;

typedef struct {
    uint32_t block_size;
    uint32_t group_size;
    marmot_dtype_t scale_dtype;
    marmot_dtype_t zero_point_dtype;
} marmot_quant_block_t;

typedef struct {
    uint32_t n;
    uint32_t d;
} marmot_layernorm_dims_t;

typedef struct {
    uint32_t seq_len;
    uint32_t n_rot;
} marmot_rope_dims_t;

typedef struct {
    uint32_t n_elems;
} marmot_elementwise_dims_t;

typedef struct {
    uint32_t axis_size;
    uint32_t inner_stride;
    uint32_t outer_size;
    uint32_t row_count;
} marmot_softmax_dims_t;

typedef union {
    marmot_matmul_dims_t matmul;
    marmot_layernorm_dims_t layernorm;
    marmot_rope_dims_t rope;
    marmot_elementwise_dims_t elementwise;
    marmot_softmax_dims_t softmax;
} marmot_op_signature_dims_t;

typedef struct {
    marmot_op_id_t op_id;
    marmot_profile_id_t profile_id;
    marmot_matmul_layout_t matmul_layout;
    marmot_dtype_t input_dtype;
    marmot_dtype_t weight_dtype;
    marmot_dtype_t output_dtype;
    marmot_dtype_t accum_dtype;
    marmot_qscheme_id_t qscheme_id;
    marmot_quant_block_t quant_block;
    marmot_weight_layout_t weight_layout;
    marmot_stride_mode_t stride_mode;
    uint32_t epilogue_flags;
    marmot_device_unary_op_t activation;
    uint32_t variant_flags;
    marmot_op_signature_dims_t dims;
} marmot_op_signature_t;

/* include/marmot/graph/kernel_selection.h:14-27 */
typedef struct {
    bool supported;
    marmot_kernel_id_t kernel_id;
    uint16_t op_index;
    double estimated_us;
    double est_comm_us;
    double est_workspace_mb;
    float confidence;
    const char *fallback_reason;
    uint32_t shardable_axes;
    uint32_t device_affinity;
} marmot_kernel_selection_t;

#define MARMOT_KERNEL_OP_INDEX_INVALID UINT16_MAX

/* include/marmot/device_caps.h:14-71 */
typedef struct {
    float peak_flops_tflops_fp32;
    float peak_flops_tflops_fp16;
    float mem_bw_gbps;
    float launch_overhead_us;
    float edge_penalty_alpha;
    uint32_t l1_cache_kb;
    uint32_t l2_cache_kb;
    uint32_t l3_cache_mb;
    uint32_t num_compute_units;
    uint32_t simd_width;
    bool has_fma;
    bool has_fp16_compute;
    bool has_bf16_compute;
    bool has_tensor_cores;
    bool has_simdgroup_mm;
    float h2d_bw_gbps;
    float d2h_bw_gbps;
    float d2d_bw_gbps;
    float d2d_lat_us;
    uint32_t copy_engines;
    uint32_t max_streams;
    float calib_dequant_us_q4k;
    float calib_dequant_us_q5k;
    float calib_dequant_us_q6k;
    float calib_dequant_us_q8_0;
    float calib_epilogue_scale;
    union {
        struct {
            bool has_amx;
            uint32_t neural_engine_tops;
            bool has_arm_bf16;
            bool has_arm_dotprod;
            bool has_arm_sve;
            marmot_cpu_microarch_t cpu_microarch;
        } apple;
        struct {
            uint32_t sm_count;
            uint32_t shared_mem_kb;
            uint32_t compute_capability;
        } cuda;
    } backend;
    struct {
        uint32_t total_cores;
        uint32_t p_cores;
        uint32_t e_cores;
        bool is_hybrid;
    } topology;
} marmot_device_caps_t;

/* src/core/dispatch/kernel_query.h:13-16 */
typedef struct {
    marmot_context_policy_t policy;
    marmot_routing_policy_t routing_policy;
} marmot_backend_preferences_t;

/* src/core/bytecode/bytecode.h:20-62 */
#define MARMOT_BC_END 0
#define MARMOT_BC_INVALID_OFFSET UINT32_MAX
#define MARMOT_BC_REG_INVALID UINT16_MAX

typedef enum {
    MARMOT_BC_SCHEMA_INVALID = 0,
    MARMOT_BC_SCHEMA_UNARY,
    MARMOT_BC_SCHEMA_BINARY,
    MARMOT_BC_SCHEMA_TERNARY,
    MARMOT_BC_SCHEMA_REDUCTION,
    MARMOT_BC_SCHEMA_SOFTMAX,
    MARMOT_BC_SCHEMA_TOPK,
    MARMOT_BC_SCHEMA_MOE_EXPERTS,
    MARMOT_BC_SCHEMA_LAYERNORM,
    MARMOT_BC_SCHEMA_RMS_NORM,
    MARMOT_BC_SCHEMA_PAGED_ATTENTION,
    MARMOT_BC_SCHEMA_ROPE,
    MARMOT_BC_SCHEMA_MATMUL,
    MARMOT_BC_SCHEMA_QKV,
    MARMOT_BC_SCHEMA_RESHAPE,
    MARMOT_BC_SCHEMA_VIEW,
    MARMOT_BC_SCHEMA_CONTIGUOUS,
    MARMOT_BC_SCHEMA_TRANSPOSE,
    MARMOT_BC_SCHEMA_CONCAT,
    MARMOT_BC_SCHEMA_SLICE,
    MARMOT_BC_SCHEMA_GATHER_ROWS,
    MARMOT_BC_SCHEMA_QUANTIZE,
    MARMOT_BC_SCHEMA_DEQUANTIZE,
    MARMOT_BC_SCHEMA_COMPUTE_QPARAMS,
    MARMOT_BC_SCHEMA_EMBEDDING,
    MARMOT_BC_SCHEMA_CONVERT,
    MARMOT_BC_SCHEMA_VEC_DOT,
} marmot_bc_schema_id_t;

typedef struct marmot_bc_exec_ctx {
    const marmot_context_t *ctx;
    const void *device_ctx;
} marmot_bc_exec_ctx_t;

typedef marmot_error_t (*marmot_bc_exec_fn)(const void *backend_exec_ctx, marmot_tensor_t **regs, const uint8_t *imm,
                                            const uint8_t *const_pool);

/* src/core/bytecode/bytecode_compile.h:23-28 */
typedef struct marmot_bc_tables {
    const uint16_t *imm_size;
    const marmot_bc_exec_fn *exec_table;
    const marmot_bc_schema_id_t *schema_id;
    uint16_t op_count;
} marmot_bc_tables_t;

#ifdef __cplusplus
}
#endif

#endif /* MARMOT_HIP_IN_TREE */

#ifdef __cplusplus
extern "C" {
#endif

/* The value MARMOT_BACKEND_HIP takes in marmot_backend_type_t (next free after MARMOT_BACKEND_CUDA = 2,
 * include/marmot/types.h:222-228; MARMOT_BACKEND_COUNT becomes 4). */
#define MARMOT_BACKEND_HIP_VALUE 3

/* ------------------------------------------------------------------ 1. device vtable
 * Counterpart of marmot_get_cpu_ops / marmot_get_metal_ops (include/marmot/device.h:112-116), selected in
 * marmot_init (src/core/context/context.c:86-108).
 *
 * Ownership. Every marmot_tensor_t owns or views a host buffer. The core calls memcpy_to_device(ctx, p, p, n)
 * with dst == src == a host pointer to say "the host copy is newer" (src/core/tensor/transfer.c:22) and
 * memcpy_from_device(ctx, p, p, n) to say "make the host copy current" (transfer.c:49-55). The backend keeps a
 * residency table keyed by host address range: a device mirror per range, created on first use by a kernel,
 * re-uploaded when the host copy was declared newer, copied back on request when a kernel wrote it. Views into
 * a mirrored range (an expert slice, a tensor inside a mapped GGUF file) resolve to an offset in the same
 * mirror. Kernels set memory_location = MARMOT_MEMORY_DEVICE and needs_sync = true on their outputs, as the
 * Metal backend does (src/backends/metal/internal/metal_memory.mm:1582-1588).
 * With dst != src, memcpy_to_device / memcpy_from_device are plain copies to / from memory from alloc(). */
const marmot_device_ops_t *marmot_get_hip_ops(void);

/* ------------------------------------------------------------------ 2. kernel query
 * Hooked into marmot_backend_query_kernel_impl, marmot_backend_detect_default_caps and
 * marmot_backend_get_default_preferences (src/core/dispatch/kernel_query.c:35-52, 88-109, 111-132).
 * Matching rules follow the generated queries (scripts/codegen/templates/backend_query.c.j2:60-104): profile is
 * a wildcard; matmul needs layout NT, input F32 or F16, output F32 (or F16 with F16 input), accumulation F32,
 * weight layout SEPARATE, contiguous strides, epilogue flags within {BIAS}, no variant flags, and a weight
 * scheme of Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K or Q6_K. */
marmot_kernel_selection_t marmot_hip_query_kernel(const marmot_op_signature_t *sig, const marmot_device_caps_t *caps);
marmot_device_caps_t marmot_hip_detect_default_caps(void);
bool marmot_hip_default_preferences(const marmot_device_caps_t *caps, marmot_backend_preferences_t *prefs_out);

/* ------------------------------------------------------------------ 3. bytecode tables
 * What marmot_bc_get_tables returns for MARMOT_BACKEND_HIP (src/core/bytecode/bytecode_compile.c:128-156; CPU
 * analogues src/backends/cpu/dispatch/bytecode_exec_cpu.gen.h:14-16). Opcode 0 is MARMOT_BC_END. Immediates
 * are little-endian and unaligned:
 *   MATMUL      u16 input, u16 weight, u16 bias (0xFFFF none), u32 epilogue const offset (0xFFFFFFFF none),
 *               u16 output                                             (bytecode_compile.c:628-669)
 *   MOE_EXPERTS u16 hidden, gate, up, down, topk_ids, topk_weights, out; u32 ffn_type; f32 weights_scale;
 *               u32 router_weight_policy                               (bytecode_compile.c:480-504)
 *   TOPK        u16 input, values_out, indices_out; u32 axis; u32 k    (bytecode_compile.c:459-479)
 *   QKV         u16 input, wq, wk, wv, bq, bk, bv (0xFFFF none); u32 epilogue const offset; u32 rope-params const
 *               offset (0xFFFFFFFF none); u16 out_q, out_k, out_v      (bytecode_compile.c:670-715)
 *   EMBEDDING   u16 weights, token_ids, out; u32 dtype_out; f32 scale; u32 padding_id; u8 bounds_check,
 *               prefer_gpu_private, allow_quant_decode_on_the_fly       (bytecode_compile.c:989-1018)
 *   QUANTIZE    u16 input; u32 quant-params const offset; u16 output; u32 kind; u32 layout   (:912-941)
 *   DEQUANTIZE  u16 input; u16 output; u32 kind; u32 layout            (bytecode_compile.c:942-962)
 *   RMS_NORM    u16 input, weight, residual (0xFFFF none), output; f32 eps      (bytecode_compile.c:530-552)
 *   BINARY      u16 input_a, input_b, output                            (bytecode_compile.c:357-375)
 *   ROPE        u16 input, output, positions (0xFFFF: the parameters' own tensor); u32 rope-params const offset;
 *               u32 n_past; u32 n_rot                                   (bytecode_compile.c:598-623)
 *   PAGED_ATTENTION u16 token_meta, q, k_new, v_new, kv_k, kv_v, block_table, kv_k_scale, kv_v_scale (0xFFFF none),
 *               out; u32 token_count, layer_idx, num_q_heads, num_kv_heads, head_dim, block_size; f32 scale
 *                                                                       (bytecode_compile.c:553-597)
 *   UNARY       u16 input, output; u32 activation-params const offset (0xFFFFFFFF none)  (bytecode_compile.c:331-356)
 *   SOFTMAX     u16 input, output; u32 axis (two's complement)          (bytecode_compile.c:440-458)
 *   RESHAPE     u16 input, output; u32 const offset of new_ndim size_t values; u64 new_ndim   (:718-745)
 *   VIEW        u16 input, output; u64 byte offset                      (bytecode_compile.c:746-763)
 *   SLICE       u16 input, output; u32 const offset of starts; u32 const offset of sizes (size_t per dimension of
 *               the output)                                              (bytecode_compile.c:863-892)
 *   GATHER_ROWS u16 input, indices, output                              (bytecode_compile.c:893-911)
 *   CONVERT     u32 const offset of the destination pointer; u32 const offset of the source pointer (host addresses
 *               stored in the const pool); u64 n; u32 dst dtype; u32 src dtype   (bytecode_compile.c:1020-1043) */
enum {
    MARMOT_HIP_BC_OP_END = 0,
    MARMOT_HIP_BC_OP_MATMUL_Q4_0 = 1,
    MARMOT_HIP_BC_OP_MATMUL_Q8_0 = 2,
    MARMOT_HIP_BC_OP_MATMUL_Q4_K = 3,
    MARMOT_HIP_BC_OP_MATMUL_Q6_K = 4,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q4_0 = 5,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q8_0 = 6,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q4_K = 7,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q6_K = 8,
    MARMOT_HIP_BC_OP_TOPK_F32 = 9,
    MARMOT_HIP_BC_OP_QUANTIZE_BLOCK = 10,
    MARMOT_HIP_BC_OP_DEQUANTIZE_BLOCK = 11,
    MARMOT_HIP_BC_OP_QKV_Q4_0 = 12,
    MARMOT_HIP_BC_OP_QKV_Q8_0 = 13,
    MARMOT_HIP_BC_OP_QKV_Q4_K = 14,
    MARMOT_HIP_BC_OP_QKV_Q6_K = 15,
    MARMOT_HIP_BC_OP_EMBEDDING_Q4_0 = 16,
    MARMOT_HIP_BC_OP_EMBEDDING_Q8_0 = 17,
    MARMOT_HIP_BC_OP_EMBEDDING_Q4_K = 18,
    MARMOT_HIP_BC_OP_EMBEDDING_Q6_K = 19,
    MARMOT_HIP_BC_OP_MATMUL_Q5_K = 20,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q5_K = 21,
    MARMOT_HIP_BC_OP_QKV_Q5_K = 22,
    MARMOT_HIP_BC_OP_EMBEDDING_Q5_K = 23,
    /* kinds added later take four consecutive ops each: MATMUL, MOE_EXPERTS, QKV, EMBEDDING */
    MARMOT_HIP_BC_OP_MATMUL_Q4_1 = 24,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q4_1 = 25,
    MARMOT_HIP_BC_OP_QKV_Q4_1 = 26,
    MARMOT_HIP_BC_OP_EMBEDDING_Q4_1 = 27,
    MARMOT_HIP_BC_OP_MATMUL_Q5_0 = 28,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q5_0 = 29,
    MARMOT_HIP_BC_OP_QKV_Q5_0 = 30,
    MARMOT_HIP_BC_OP_EMBEDDING_Q5_0 = 31,
    MARMOT_HIP_BC_OP_MATMUL_Q5_1 = 32,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q5_1 = 33,
    MARMOT_HIP_BC_OP_QKV_Q5_1 = 34,
    MARMOT_HIP_BC_OP_EMBEDDING_Q5_1 = 35,
    MARMOT_HIP_BC_OP_MATMUL_Q2_K = 36,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q2_K = 37,
    MARMOT_HIP_BC_OP_QKV_Q2_K = 38,
    MARMOT_HIP_BC_OP_EMBEDDING_Q2_K = 39,
    MARMOT_HIP_BC_OP_MATMUL_Q3_K = 40,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q3_K = 41,
    MARMOT_HIP_BC_OP_QKV_Q3_K = 42,
    MARMOT_HIP_BC_OP_EMBEDDING_Q3_K = 43,
    MARMOT_HIP_BC_OP_MATMUL_Q8_1 = 44,
    MARMOT_HIP_BC_OP_MOE_EXPERTS_Q8_1 = 45,
    MARMOT_HIP_BC_OP_QKV_Q8_1 = 46,
    MARMOT_HIP_BC_OP_EMBEDDING_Q8_1 = 47,
    /* the FLOAT32 ops between the linears */
    MARMOT_HIP_BC_OP_RMS_NORM_F32 = 48,
    MARMOT_HIP_BC_OP_RMS_NORM_GEMMA_F32 = 49,
    MARMOT_HIP_BC_OP_SWIGLU_F32 = 50,
    MARMOT_HIP_BC_OP_GEGLU_F32 = 51,
    MARMOT_HIP_BC_OP_ADD_F32 = 52,
    /* rotary embedding of FLOAT32 or FLOAT16 rows */
    MARMOT_HIP_BC_OP_ROPE = 53,
    /* paged attention: cache write + attention through the block table */
    MARMOT_HIP_BC_OP_PAGED_ATTENTION = 54,
    /* the remaining nodes of a GGUF model graph: activations, router softmax, conversions, row gather, views */
    MARMOT_HIP_BC_OP_GELU = 55,
    MARMOT_HIP_BC_OP_GELU_TANH = 56,
    MARMOT_HIP_BC_OP_SILU = 57,
    MARMOT_HIP_BC_OP_SOFTMAX_F32 = 58,
    MARMOT_HIP_BC_OP_RESHAPE = 59,
    MARMOT_HIP_BC_OP_VIEW = 60,
    MARMOT_HIP_BC_OP_SLICE = 61,
    MARMOT_HIP_BC_OP_GATHER_ROWS = 62,
    MARMOT_HIP_BC_OP_CONVERT = 63,
    MARMOT_HIP_BC_OP_COUNT = 64,
};
bool marmot_hip_bc_get_tables(marmot_bc_tables_t *out);

/* ------------------------------------------------------------------ 4. impl functions
 * The functions the generated dispatch shims call for the HIP kernel families
 * (cf. cpu_matmul_quantized_{scheme}, src/backends/cpu/dispatch/matmul_dispatch_cpu.gen.c:955-965;
 * cpu_moe_experts_impl and cpu_topk_impl, src/backends/cpu/ops/moe/moe_ops.c:1069-1178, 789-889;
 * cpu_quantize_q8_0 / cpu_quantize_q8_k / cpu_dequantize_{scheme},
 * src/backends/cpu/cpu_backend_internal.h:925-939). Validation and error codes follow
 * marmot_matmul_validate_quantized (src/core/helpers/matmul.c:68-136). */
marmot_error_t hip_matmul_quantized_q4_0(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q8_0(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q4_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q4_1(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q5_0(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q5_1(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q2_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q3_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q8_1(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q5_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
marmot_error_t hip_matmul_quantized_q6_k(const void *device_ctx, const marmot_tensor_t *input,
                                         const marmot_tensor_t *weight, const marmot_matmul_epilogue_t *epilogue,
                                         marmot_tensor_t *out);
/* marmot_matmul_qkv with MARMOT_QKV_LAYOUT_SEPARATE and block-quantized weights of one kind and shape
 * (cf. cpu_matmul_qkv_{q4_k,q6_k,q8_0}, src/backends/cpu/ops/matmul/qkv/matmul_qkv.c:1498-1532; validation as
 * cpu_matmul_qkv_validate_desc, :1230-1300), including the rotary epilogue (rope_params applied to q and/or k with
 * FLOAT32, INT32 or INT64 positions; frequencies as marmot_rope_freq_cache_ensure, src/core/helpers/rope.c). The fused
 * layout and dense weights return MARMOT_ERROR_NOT_IMPLEMENTED. */
marmot_error_t hip_matmul_qkv_q4_0(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q8_0(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q4_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q4_1(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q5_0(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q5_1(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q2_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q3_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q8_1(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q5_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
marmot_error_t hip_matmul_qkv_q6_k(const void *device_ctx, const marmot_matmul_qkv_desc_t *desc);
/* marmot_embedding_gather with a block-quantized table [vocab, dim] (cf. cpu_embedding_gather,
 * src/backends/cpu/ops/embedding/embedding_dispatch.c:4-16 -> embedding_scalar.c:460-591): token ids INT32 or INT64 of
 * any shape, output FLOAT32 or FLOAT16 viewed as [tokens, dim]; weights->quant_kind selects Q4_0, Q4_1, Q5_0,
 * Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K or Q6_K. */
marmot_error_t hip_embedding_gather(const void *device_ctx, const marmot_embedding_gather_desc_t *desc);
marmot_error_t hip_moe_experts_impl(const void *device_ctx, const marmot_moe_experts_desc_t *desc);
marmot_error_t hip_topk_impl(const void *device_ctx, const marmot_topk_desc_t *desc);
/* The FLOAT32 ops between the linears: cpu_rmsnorm_impl / cpu_rmsnorm_gemma_impl
 * (src/backends/cpu/ops/normalization/normalization_dispatch.c:240-246; any rank, normalized over the last dimension,
 * optional residual and weight), cpu_swiglu_f32_scalar / cpu_geglu_f32_scalar and the elementwise add
 * (src/backends/cpu/ops/elementwise/scalar/elementwise_f32_scalar.c; contiguous or, for the gated products,
 * row-strided 2-D tensors). A normalization of nine rows or more also leaves its output packed for the linears that
 * read it, and a linear that packs an fp32 input of nine rows or more keeps the packed rows for the linears that
 * share it (see activation_packs / activation_pack_hits below): no quantization launch per linear. */
marmot_error_t hip_rmsnorm_impl(const void *device_ctx, const marmot_rmsnorm_desc_t *desc);
marmot_error_t hip_rmsnorm_gemma_impl(const void *device_ctx, const marmot_rmsnorm_desc_t *desc);
marmot_error_t hip_swiglu_f32(const void *device_ctx, const marmot_tensor_t *a, const marmot_tensor_t *b,
                              marmot_tensor_t *out);
marmot_error_t hip_geglu_f32(const void *device_ctx, const marmot_tensor_t *a, const marmot_tensor_t *b,
                             marmot_tensor_t *out);
marmot_error_t hip_add_f32(const void *device_ctx, const marmot_tensor_t *a, const marmot_tensor_t *b,
                           marmot_tensor_t *out);
/* marmot_rope (cf. cpu_rope, src/backends/cpu/ops/rope/rope_dispatch.c:145-372): the last dimension of x, FLOAT32 or
 * FLOAT16, is rotated into out (same shape and type; out == x rotates in place), one position per row from
 * params->positions (FLOAT32, INT32 or INT64, as many values as x has rows); frequencies and attention scale as
 * marmot_rope_freq_cache_ensure for the rotated dimension (src/core/helpers/rope.c:143-200), all scaling types.
 * Contiguous tensors, or rows at one stride >= their length; FLOAT64 and BFLOAT16 are declined NOT_IMPLEMENTED. */
/* marmot_paged_attention (cf. cpu_paged_attention_impl, src/backends/cpu/ops/paged_attention/paged_attention_ref.c:
 * 573-1082): every token's k_new / v_new rows go into the paged cache at its kv_slot, then every token attends over
 * positions 0 .. pos of its sequence through the block table. q / k_new / v_new / out of one type among FLOAT32,
 * FLOAT16, BFLOAT16 and the cache of one of these types or FLOAT8_E4M3 (then with FLOAT32 scale tensors [blocks,
 * layers, kv heads] in pnext, read and written like the cache), any strides; validation, codes and messages in the
 * reference's order. Declined with NOT_IMPLEMENTED: head dimensions beyond 256, key and value caches (or scales) of
 * different strides. The cache tensors are read and written: their mirrors are brought up to date first and the
 * device copy is the current one afterwards. */
marmot_error_t hip_paged_attention_impl(const void *device_ctx, const marmot_paged_attention_desc_t *desc);
marmot_error_t hip_rope(const void *device_ctx, const marmot_tensor_t *x, const marmot_rope_params_t *params,
                        marmot_tensor_t *out);
/* The remaining nodes of a GGUF model graph (src/graph/gguf/graph_builder.cpp:555-1140).
 * hip_gelu / hip_gelu_tanh / hip_silu (cf. cpu_unary_gelu_f32 and friends, src/backends/cpu/ops/unary/scalar/
 * unary_scalar.c:201-218, 387-396): contiguous FLOAT32 or FLOAT16 tensors of equal shape; activation parameters with a
 * bias or a parameter tensor are declined NOT_IMPLEMENTED.
 * hip_softmax_impl (cf. cpu_softmax_impl, src/backends/cpu/ops/softmax/softmax_dispatch.c:67-103; validation as
 * marmot_softmax_prepare, src/core/helpers/norm.c:123-179): contiguous FLOAT32 tensors, any axis.
 * hip_reshape / hip_view (cf. cpu_reshape, cpu_view, src/backends/cpu/ops/tensor_ops/tensor_ops.c:29-158): metadata
 * only, no device work: the output aliases the input's host range, which the residency table resolves to the same
 * mirror; an output buffer the tensor owned is released (and its mirror dropped) as the reference does.
 * hip_slice (cf. cpu_slice, tensor_ops.c:401-462): contiguous tensors of up to 8 dimensions.
 * hip_gather_rows (cf. cpu_gather_rows, tensor_ops.c:464-547): 2-D tensors with unit column stride.
 * hip_convert (cf. cpu_convert_dispatch, src/backends/cpu/ops/convert/): n values between FLOAT32, FLOAT16 and
 * BFLOAT16 at host addresses known to (or made known to) the residency table. */
marmot_error_t hip_gelu(const void *device_ctx, const marmot_tensor_t *x, const marmot_activation_params_t *params,
                        marmot_tensor_t *out);
marmot_error_t hip_gelu_tanh(const void *device_ctx, const marmot_tensor_t *x, const marmot_activation_params_t *params,
                             marmot_tensor_t *out);
marmot_error_t hip_silu(const void *device_ctx, const marmot_tensor_t *x, const marmot_activation_params_t *params,
                        marmot_tensor_t *out);
marmot_error_t hip_softmax_impl(const void *device_ctx, const marmot_softmax_desc_t *desc);
marmot_error_t hip_reshape(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out,
                           const size_t *new_shape, size_t new_ndim);
marmot_error_t hip_view(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out, size_t byte_offset);
marmot_error_t hip_slice(const void *device_ctx, const marmot_tensor_t *x, marmot_tensor_t *out, const size_t *starts,
                         const size_t *sizes);
marmot_error_t hip_gather_rows(const void *device_ctx, const marmot_tensor_t *input, const marmot_tensor_t *indices,
                               marmot_tensor_t *out);
marmot_error_t hip_convert(const void *device_ctx, marmot_dtype_t dst_dtype, void *dst, marmot_dtype_t src_dtype,
                           const void *src, size_t n);
/* output->quant_kind selects the block format: the activation formats Q8_0 and Q8_K (FLOAT32 or FLOAT16 input) or the
 * weight formats Q4_K, Q5_K and Q6_K (FLOAT32 input; cf. cpu_quantize_q4_k / _q5_k / _q6_k, quantize_core.c:199-265) */
marmot_error_t hip_quantize_block(const void *device_ctx, const marmot_tensor_t *input, marmot_tensor_t *output);
/* input->quant_kind selects the weight block format: Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K,
 * Q6_K or Q8_K */
marmot_error_t hip_dequantize_block(const void *device_ctx, const marmot_tensor_t *input, marmot_tensor_t *output);

/* ------------------------------------------------------------------ error text and introspection
 * Inside the marmot tree errors go to marmot_set_error (include/marmot/error.h:21-43). Outside, the last code
 * and text set by this layer on the calling thread are kept here. */
marmot_error_t marmot_hip_backend_last_error(const char **detail_out);
/* Residency-table facts for tests: number of mirrors, bytes mirrored, uploads and downloads so far. */
typedef struct {
    size_t mirrors;
    size_t mirrored_bytes;
    uint64_t uploads;
    uint64_t upload_bytes;
    uint64_t downloads;
    uint64_t download_bytes;
    uint64_t activation_packs;     /* packed copies of fp32 activation tensors made (by a normalization or a linear) */
    uint64_t activation_pack_hits; /* linears that found their input already packed */
} marmot_hip_residency_stats_t;
void marmot_hip_backend_residency_stats(const void *device_ctx, marmot_hip_residency_stats_t *out);

#ifdef __cplusplus
}
#endif

#endif /* MARMOT_HIP_BACKEND_H */

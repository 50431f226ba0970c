/* Prints "name value" lines: sizes, member offsets and enumerator values of every marmot type the HIP backend
 * touches. Built twice by make_abi_layout.py / test_backend_abi.py: against the reference's own headers
 * (-DABI_PROBE_REFERENCE, include paths into the reference tree) and against the mirror in marmot_hip_backend.h.
 * The two outputs must be identical. */
#include <stddef.h>
#include <stdio.h>

#ifdef ABI_PROBE_REFERENCE
#include "marmot/device.h"
#include "marmot/graph/kernel_selection.h"
#include "marmot/graph/op_signature.h"
#include "marmot/ops_types.h"
#include "marmot/ops/matmul.h"
#include "marmot/ops/paged_attention.h"
#include "core/bytecode/bytecode.h"
#include "core/bytecode/bytecode_compile.h"
#include "core/dispatch/kernel_query.h"
#else
#include "marmot_hip_backend.h"
#endif

#define SZ(T) printf("sizeof(" #T ") %zu\n", sizeof(T))
#define OFF(T, m) printf("offsetof(" #T "," #m ") %zu\n", offsetof(T, m))
#define VAL(e) printf(#e " %lld\n", (long long)(e))

int main(void) {
    SZ(marmot_error_t); SZ(marmot_dtype_t); SZ(marmot_quant_kind_t); SZ(marmot_quant_layout_t);
    SZ(marmot_backend_type_t); SZ(marmot_memory_location_t); SZ(marmot_cpu_microarch_t);
    SZ(marmot_device_unary_op_t); SZ(marmot_op_id_t); SZ(marmot_kernel_id_t); SZ(marmot_bc_schema_id_t);
    VAL(MARMOT_MAX_DIMS);
    VAL(MARMOT_SUCCESS); VAL(MARMOT_ERROR_INVALID_ARGUMENT); VAL(MARMOT_ERROR_OUT_OF_MEMORY);
    VAL(MARMOT_ERROR_DEVICE_NOT_AVAILABLE); VAL(MARMOT_ERROR_BACKEND_INIT_FAILED);
    VAL(MARMOT_ERROR_INVALID_OPERATION); VAL(MARMOT_ERROR_UNSUPPORTED_DTYPE);
    VAL(MARMOT_ERROR_DIMENSION_MISMATCH); VAL(MARMOT_ERROR_NOT_IMPLEMENTED);
    VAL(MARMOT_BACKEND_CPU); VAL(MARMOT_BACKEND_METAL); VAL(MARMOT_BACKEND_CUDA);
    VAL(MARMOT_DTYPE_FLOAT32); VAL(MARMOT_DTYPE_FLOAT16); VAL(MARMOT_DTYPE_INT32); VAL(MARMOT_DTYPE_INT8);
    VAL(MARMOT_DTYPE_UINT8); VAL(MARMOT_DTYPE_COUNT);
    VAL(MARMOT_QUANT_LAYOUT_GGUF);
    VAL(MARMOT_QUANT_KIND_Q4_0); VAL(MARMOT_QUANT_KIND_Q8_0); VAL(MARMOT_QUANT_KIND_Q4_K);
    VAL(MARMOT_QUANT_KIND_Q4_1); VAL(MARMOT_QUANT_KIND_Q5_0); VAL(MARMOT_QUANT_KIND_Q5_1);
    VAL(MARMOT_QUANT_KIND_Q5_K); VAL(MARMOT_QUANT_KIND_Q6_K); VAL(MARMOT_QUANT_KIND_Q8_K); VAL(MARMOT_QUANT_KIND_COUNT);
    VAL(MARMOT_MEMORY_HOST); VAL(MARMOT_MEMORY_DEVICE);
    VAL(MARMOT_FFN_SWIGLU); VAL(MARMOT_FFN_GEGLU);
    VAL(MARMOT_ROUTER_WEIGHT_POLICY_SOFTMAX_SELECTED); VAL(MARMOT_ROUTER_WEIGHT_POLICY_SOFTMAX_SELECTED_SCALED);
    VAL(MARMOT_ROUTER_WEIGHT_POLICY_RENORMALIZE_SELECTED);
    VAL(MARMOT_ROUTING_ALWAYS_GPU);
    VAL(MARMOT_OP_MATMUL); VAL(MARMOT_OP_LINEAR); VAL(MARMOT_OP_MOE_EXPERTS); VAL(MARMOT_OP_TOPK);
    VAL(MARMOT_OP_QUANTIZE); VAL(MARMOT_OP_DEQUANTIZE);
    VAL(MARMOT_OP_QKV_PROJECTION); VAL(MARMOT_OP_QKV_SHARED_INPUT); VAL(MARMOT_OP_QKV_ROPE);
    VAL(MARMOT_QKV_LAYOUT_FUSED); VAL(MARMOT_QKV_LAYOUT_SEPARATE);
    VAL(MARMOT_ROPE_SCALING_NONE); VAL(MARMOT_ROPE_SCALING_YARN); VAL(MARMOT_ROPE_TYPE_NORM); VAL(MARMOT_ROPE_TYPE_NEOX);
    VAL(MARMOT_EPILOGUE_ROPE); VAL(MARMOT_BC_SCHEMA_QKV);
    VAL(MARMOT_OP_EMBEDDING); VAL(MARMOT_BC_SCHEMA_EMBEDDING); VAL(MARMOT_DTYPE_INT64);
    VAL(MARMOT_PREFERENCE_ENABLE); VAL(MARMOT_PREFERENCE_DISABLE);
    VAL(MARMOT_QSCHEME_Q4_0); VAL(MARMOT_QSCHEME_Q8_0); VAL(MARMOT_QSCHEME_Q4_K); VAL(MARMOT_QSCHEME_Q6_K);
    VAL(MARMOT_QSCHEME_Q8_K); VAL(MARMOT_QSCHEME_Q5_K);
    VAL(MARMOT_QSCHEME_Q4_1); VAL(MARMOT_QSCHEME_Q5_0); VAL(MARMOT_QSCHEME_Q5_1);
    VAL(MARMOT_QSCHEME_Q2_K); VAL(MARMOT_QSCHEME_Q3_K); VAL(MARMOT_QUANT_KIND_Q2_K); VAL(MARMOT_QUANT_KIND_Q3_K);
    VAL(MARMOT_QSCHEME_Q8_1); VAL(MARMOT_QUANT_KIND_Q8_1);
    VAL(MARMOT_MATMUL_LAYOUT_NT); VAL(MARMOT_WEIGHT_LAYOUT_SEPARATE); VAL(MARMOT_STRIDE_MODE_CONTIGUOUS);
    VAL(MARMOT_EPILOGUE_BIAS); VAL(MARMOT_KERNEL_INVALID);
    VAL(MARMOT_BC_SCHEMA_TOPK); VAL(MARMOT_BC_SCHEMA_MOE_EXPERTS); VAL(MARMOT_BC_SCHEMA_MATMUL);
    VAL(MARMOT_BC_SCHEMA_QUANTIZE); VAL(MARMOT_BC_SCHEMA_DEQUANTIZE);
    VAL(MARMOT_BC_REG_INVALID); VAL(MARMOT_BC_INVALID_OFFSET); VAL(MARMOT_BC_END);
    VAL(MARMOT_OP_RMS_NORM); VAL(MARMOT_OP_RMS_NORM_GEMMA); VAL(MARMOT_OP_SWIGLU); VAL(MARMOT_OP_GEGLU); VAL(MARMOT_OP_ADD);
    VAL(MARMOT_BC_SCHEMA_RMS_NORM); VAL(MARMOT_BC_SCHEMA_BINARY);
    VAL(MARMOT_OP_ROPE); VAL(MARMOT_BC_SCHEMA_ROPE);
    VAL(MARMOT_OP_PAGED_ATTENTION); VAL(MARMOT_BC_SCHEMA_PAGED_ATTENTION); VAL(MARMOT_DTYPE_BFLOAT16);
    VAL(MARMOT_DTYPE_UINT32); VAL(MARMOT_DTYPE_FLOAT8_E4M3); VAL(MARMOT_PAGED_ATTENTION_DESC_VERSION);
    VAL(MARMOT_PAGED_ATTENTION_KV_SCALE_EXT_VERSION);
    VAL(MARMOT_OP_GELU); VAL(MARMOT_OP_GELU_TANH); VAL(MARMOT_OP_SILU); VAL(MARMOT_OP_SOFTMAX); VAL(MARMOT_OP_RESHAPE);
    VAL(MARMOT_OP_VIEW); VAL(MARMOT_OP_SLICE); VAL(MARMOT_OP_GATHER_ROWS); VAL(MARMOT_OP_CONVERT);
    VAL(MARMOT_BC_SCHEMA_UNARY); VAL(MARMOT_BC_SCHEMA_SOFTMAX); VAL(MARMOT_BC_SCHEMA_RESHAPE); VAL(MARMOT_BC_SCHEMA_VIEW);
    VAL(MARMOT_BC_SCHEMA_SLICE); VAL(MARMOT_BC_SCHEMA_GATHER_ROWS); VAL(MARMOT_BC_SCHEMA_CONVERT);

    SZ(marmot_shape_t); OFF(marmot_shape_t, ndim); OFF(marmot_shape_t, shape); OFF(marmot_shape_t, strides);
    SZ(marmot_quant_params_t);
    SZ(marmot_tensor_t);
    OFF(marmot_tensor_t, shape); OFF(marmot_tensor_t, dtype); OFF(marmot_tensor_t, data);
    OFF(marmot_tensor_t, capacity_bytes); OFF(marmot_tensor_t, owns_data); OFF(marmot_tensor_t, quant_params);
    OFF(marmot_tensor_t, quant_kind); OFF(marmot_tensor_t, quant_layout); OFF(marmot_tensor_t, backend);
    OFF(marmot_tensor_t, ctx); OFF(marmot_tensor_t, memory_location); OFF(marmot_tensor_t, needs_sync);
    OFF(marmot_tensor_t, packed_data); OFF(marmot_tensor_t, packed_src_data); OFF(marmot_tensor_t, packed_bytes);
    OFF(marmot_tensor_t, packed_row_bytes); OFF(marmot_tensor_t, packed_rows);
    SZ(marmot_allocator_usage_t); OFF(marmot_allocator_usage_t, active_allocations);
    OFF(marmot_allocator_usage_t, pool_misses);
    SZ(marmot_context_policy_t); OFF(marmot_context_policy_t, matmul_requires_temp_tensors);
    SZ(marmot_backend_preferences_t); OFF(marmot_backend_preferences_t, routing_policy);
    SZ(marmot_device_ops_t);
    OFF(marmot_device_ops_t, init); OFF(marmot_device_ops_t, destroy); OFF(marmot_device_ops_t, configure);
    OFF(marmot_device_ops_t, alloc); OFF(marmot_device_ops_t, free); OFF(marmot_device_ops_t, memcpy_to_device);
    OFF(marmot_device_ops_t, memcpy_from_device); OFF(marmot_device_ops_t, synchronize);
    OFF(marmot_device_ops_t, allocator_usage); OFF(marmot_device_ops_t, graph_batch_begin);
    OFF(marmot_device_ops_t, graph_batch_end); OFF(marmot_device_ops_t, on_host_ptr_freed);
    OFF(marmot_device_ops_t, on_host_range_freed);
    SZ(marmot_matmul_epilogue_t); OFF(marmot_matmul_epilogue_t, bias);
    OFF(marmot_matmul_epilogue_t, enable_output_cast); OFF(marmot_matmul_epilogue_t, output_dtype);
    SZ(marmot_rope_params_t); OFF(marmot_rope_params_t, positions); OFF(marmot_rope_params_t, scaling_type);
    OFF(marmot_rope_params_t, rope_type); OFF(marmot_rope_params_t, theta); OFF(marmot_rope_params_t, beta_slow);
    OFF(marmot_rope_params_t, orig_ctx_len); OFF(marmot_rope_params_t, head_dim);
    OFF(marmot_rope_params_t, apply_to_q); OFF(marmot_rope_params_t, apply_to_k);
    SZ(marmot_matmul_qkv_desc_t); OFF(marmot_matmul_qkv_desc_t, input); OFF(marmot_matmul_qkv_desc_t, layout);
    OFF(marmot_matmul_qkv_desc_t, fused); OFF(marmot_matmul_qkv_desc_t, separate);
    OFF(marmot_matmul_qkv_desc_t, epilogue); OFF(marmot_matmul_qkv_desc_t, out_q);
    OFF(marmot_matmul_qkv_desc_t, out_k); OFF(marmot_matmul_qkv_desc_t, out_v);
    OFF(marmot_matmul_qkv_desc_t, rope_params);
    SZ(marmot_matmul_qkv_separate_t); OFF(marmot_matmul_qkv_separate_t, wv); OFF(marmot_matmul_qkv_separate_t, bq);
    SZ(marmot_embedding_gather_desc_t); OFF(marmot_embedding_gather_desc_t, out);
    OFF(marmot_embedding_gather_desc_t, dtype_out); OFF(marmot_embedding_gather_desc_t, scale);
    OFF(marmot_embedding_gather_desc_t, padding_id); OFF(marmot_embedding_gather_desc_t, bounds_check);
    OFF(marmot_embedding_gather_desc_t, prefer_gpu_private);
    OFF(marmot_embedding_gather_desc_t, allow_quant_decode_on_the_fly);
    SZ(marmot_paged_attention_desc_t); OFF(marmot_paged_attention_desc_t, struct_size);
    OFF(marmot_paged_attention_desc_t, struct_version); OFF(marmot_paged_attention_desc_t, flags);
    OFF(marmot_paged_attention_desc_t, token_count); OFF(marmot_paged_attention_desc_t, layer_idx);
    OFF(marmot_paged_attention_desc_t, num_q_heads); OFF(marmot_paged_attention_desc_t, num_kv_heads);
    OFF(marmot_paged_attention_desc_t, head_dim); OFF(marmot_paged_attention_desc_t, block_size);
    OFF(marmot_paged_attention_desc_t, scale); OFF(marmot_paged_attention_desc_t, token_meta);
    OFF(marmot_paged_attention_desc_t, q); OFF(marmot_paged_attention_desc_t, k_new);
    OFF(marmot_paged_attention_desc_t, v_new); OFF(marmot_paged_attention_desc_t, kv_k);
    OFF(marmot_paged_attention_desc_t, kv_v); OFF(marmot_paged_attention_desc_t, block_table);
    OFF(marmot_paged_attention_desc_t, out); OFF(marmot_paged_attention_desc_t, pnext);
    OFF(marmot_paged_attention_desc_t, reserved);
    SZ(marmot_paged_attention_kv_scale_ext_t); OFF(marmot_paged_attention_kv_scale_ext_t, struct_size);
    OFF(marmot_paged_attention_kv_scale_ext_t, struct_version); OFF(marmot_paged_attention_kv_scale_ext_t, kv_k_scale);
    OFF(marmot_paged_attention_kv_scale_ext_t, kv_v_scale);
    SZ(marmot_topk_desc_t); OFF(marmot_topk_desc_t, axis); OFF(marmot_topk_desc_t, k);
    SZ(marmot_softmax_desc_t); OFF(marmot_softmax_desc_t, out); OFF(marmot_softmax_desc_t, axis);
    SZ(marmot_activation_params_t); OFF(marmot_activation_params_t, bias); OFF(marmot_activation_params_t, alpha);
    OFF(marmot_activation_params_t, gamma);
    SZ(marmot_rmsnorm_desc_t); OFF(marmot_rmsnorm_desc_t, residual); OFF(marmot_rmsnorm_desc_t, weight);
    OFF(marmot_rmsnorm_desc_t, out); OFF(marmot_rmsnorm_desc_t, eps);
    SZ(marmot_moe_experts_desc_t); OFF(marmot_moe_experts_desc_t, out); OFF(marmot_moe_experts_desc_t, ffn_type);
    OFF(marmot_moe_experts_desc_t, weights_scale); OFF(marmot_moe_experts_desc_t, router_weight_policy);
    SZ(marmot_matmul_dims_t); SZ(marmot_quant_block_t); SZ(marmot_op_signature_dims_t);
    SZ(marmot_op_signature_t);
    OFF(marmot_op_signature_t, op_id); OFF(marmot_op_signature_t, profile_id);
    OFF(marmot_op_signature_t, matmul_layout); OFF(marmot_op_signature_t, input_dtype);
    OFF(marmot_op_signature_t, weight_dtype); OFF(marmot_op_signature_t, output_dtype);
    OFF(marmot_op_signature_t, accum_dtype); OFF(marmot_op_signature_t, qscheme_id);
    OFF(marmot_op_signature_t, quant_block); OFF(marmot_op_signature_t, weight_layout);
    OFF(marmot_op_signature_t, stride_mode); OFF(marmot_op_signature_t, epilogue_flags);
    OFF(marmot_op_signature_t, activation); OFF(marmot_op_signature_t, variant_flags);
    OFF(marmot_op_signature_t, dims);
    SZ(marmot_kernel_selection_t);
    OFF(marmot_kernel_selection_t, supported); OFF(marmot_kernel_selection_t, kernel_id);
    OFF(marmot_kernel_selection_t, op_index); OFF(marmot_kernel_selection_t, estimated_us);
    OFF(marmot_kernel_selection_t, est_comm_us); OFF(marmot_kernel_selection_t, est_workspace_mb);
    OFF(marmot_kernel_selection_t, confidence); OFF(marmot_kernel_selection_t, fallback_reason);
    OFF(marmot_kernel_selection_t, shardable_axes); OFF(marmot_kernel_selection_t, device_affinity);
    SZ(marmot_device_caps_t);
    OFF(marmot_device_caps_t, peak_flops_tflops_fp16); OFF(marmot_device_caps_t, mem_bw_gbps);
    OFF(marmot_device_caps_t, launch_overhead_us); OFF(marmot_device_caps_t, l2_cache_kb);
    OFF(marmot_device_caps_t, num_compute_units); OFF(marmot_device_caps_t, simd_width);
    OFF(marmot_device_caps_t, has_fma); OFF(marmot_device_caps_t, has_tensor_cores);
    OFF(marmot_device_caps_t, h2d_bw_gbps); OFF(marmot_device_caps_t, max_streams);
    OFF(marmot_device_caps_t, calib_epilogue_scale); OFF(marmot_device_caps_t, backend);
    OFF(marmot_device_caps_t, topology);
    SZ(marmot_bc_exec_ctx_t); OFF(marmot_bc_exec_ctx_t, ctx); OFF(marmot_bc_exec_ctx_t, device_ctx);
    SZ(marmot_bc_tables_t); OFF(marmot_bc_tables_t, imm_size); OFF(marmot_bc_tables_t, exec_table);
    OFF(marmot_bc_tables_t, schema_id); OFF(marmot_bc_tables_t, op_count);
    return 0;
}

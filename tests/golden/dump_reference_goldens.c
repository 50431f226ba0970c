/*
 * Fixture generator (runs only where the reference checkout is present).
 *
 * Includes the golden-vector headers that the reference's own tests hold
 * (tests/backend/golden_quant_llama.h, golden_vec_dot_llama.h, golden_matmul_llama.h,
 * matmul_quantized_golden_cases.h) directly from the reference tree at build time and
 * writes their arrays as a flat binary container on stdout:
 *     repeat { u32 name_len, name bytes, u32 dtype_len, dtype bytes, u64 nbytes, data }
 * make_fixtures.py turns that stream into an .npz of plain arrays (data only).
 */
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "marmot/quant_block.h"
#include "marmot/types.h"

#include "backend/matmul_quantized_golden_cases.h"
#include "backend/golden_vec_dot_llama.h"
/* the conversion goldens of tests/backend/test_backend_conversions.c: FLOAT8_E4M3 codes and round trips */
#define MARMOT_ENABLE_FP8 1
#include "backend/golden_data.h"

static void emit(const char *name, const char *dtype, const void *data, size_t nbytes) {
    uint32_t nl = (uint32_t)strlen(name);
    uint32_t dl = (uint32_t)strlen(dtype);
    uint64_t nb = (uint64_t)nbytes;
    fwrite(&nl, 4, 1, stdout);
    fwrite(name, 1, nl, stdout);
    fwrite(&dl, 4, 1, stdout);
    fwrite(dtype, 1, dl, stdout);
    fwrite(&nb, 8, 1, stdout);
    fwrite(data, 1, nbytes, stdout);
}

#define EMIT(arr, dtype) emit(#arr, dtype, arr, sizeof(arr))
#define EMIT_SCALAR(v, dtype) emit(#v, dtype, &v, sizeof(v))

int main(void) {
    /* quantizer goldens */
    EMIT(g_llama_test_input, "f4");
    EMIT(g_llama_q4_0, "u1");
    EMIT(g_llama_q4_0_dequant, "f4");
    EMIT(g_llama_q4_1, "u1");
    EMIT(g_llama_q4_1_dequant, "f4");
    EMIT(g_llama_q5_0, "u1");
    EMIT(g_llama_q5_0_dequant, "f4");
    EMIT(g_llama_q5_1, "u1");
    EMIT(g_llama_q5_1_dequant, "f4");
    EMIT(g_llama_q8_1, "u1");
    EMIT(g_llama_q8_1_dequant, "f4");
    EMIT(g_llama_q8_0, "u1");
    EMIT(g_llama_q8_0_dequant, "f4");
    EMIT(g_llama_q2_k, "u1");
    EMIT(g_llama_q2_k_dequant, "f4");
    EMIT(g_llama_q3_k, "u1");
    EMIT(g_llama_q3_k_dequant, "f4");
    EMIT(g_llama_q4_k, "u1");
    EMIT(g_llama_q4_k_dequant, "f4");
    EMIT(g_llama_q5_k, "u1");
    EMIT(g_llama_q5_k_dequant, "f4");
    EMIT(g_llama_q6_k, "u1");
    EMIT(g_llama_q6_k_dequant, "f4");
    EMIT(g_llama_q8_k, "u1");
    EMIT(g_llama_q8_k_dequant, "f4");

    /* block-dot goldens */
    EMIT(g_vec_dot_test_vec1, "f4");
    EMIT(g_vec_dot_test_vec2, "f4");
    EMIT(g_vec_dot_q8_0_activations, "u1");
    EMIT(g_vec_dot_q8_k_activations, "u1");
    EMIT(g_vec_dot_q4_0_weights, "u1");
    EMIT(g_vec_dot_q8_0_weights, "u1");
    EMIT(g_vec_dot_q8_1_weights, "u1");
    EMIT(g_vec_dot_q4_1_weights, "u1");
    EMIT(g_vec_dot_q5_0_weights, "u1");
    EMIT(g_vec_dot_q5_1_weights, "u1");
    EMIT(g_vec_dot_q2_k_weights, "u1");
    EMIT(g_vec_dot_q3_k_weights, "u1");
    EMIT(g_vec_dot_q4_k_weights, "u1");
    EMIT(g_vec_dot_q5_k_weights, "u1");
    EMIT(g_vec_dot_q6_k_weights, "u1");
    EMIT_SCALAR(g_vec_dot_q4_0_q8_0_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q8_0_q8_0_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q8_1_q8_0_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q4_1_q8_0_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q5_0_q8_0_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q5_1_q8_0_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q2_k_q8_k_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q3_k_q8_k_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q4_k_q8_k_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q5_k_q8_k_expected, "f4");
    EMIT_SCALAR(g_vec_dot_q6_k_q8_k_expected, "f4");

    /* whole-matmul goldens for the formats on the path */
    const size_t ncases = sizeof(g_matmul_quant_goldens) / sizeof(g_matmul_quant_goldens[0]);
    for (size_t i = 0; i < ncases; ++i) {
        const matmul_golden_case_t *c = &g_matmul_quant_goldens[i];
        if (c->kind != MARMOT_QUANT_KIND_Q4_0 && c->kind != MARMOT_QUANT_KIND_Q8_0 &&
            c->kind != MARMOT_QUANT_KIND_Q4_K && c->kind != MARMOT_QUANT_KIND_Q5_K &&
            c->kind != MARMOT_QUANT_KIND_Q6_K && c->kind != MARMOT_QUANT_KIND_Q4_1 &&
            c->kind != MARMOT_QUANT_KIND_Q5_0 && c->kind != MARMOT_QUANT_KIND_Q5_1 &&
            c->kind != MARMOT_QUANT_KIND_Q2_K && c->kind != MARMOT_QUANT_KIND_Q3_K &&
            c->kind != MARMOT_QUANT_KIND_Q8_1) {
            continue;
        }
        char name[128];
        int64_t dims[4] = {(int64_t)c->kind, (int64_t)c->N, (int64_t)c->K, (int64_t)c->M};
        snprintf(name, sizeof(name), "matmul_%s_dims", c->name);
        emit(name, "i8", dims, sizeof(dims));
        snprintf(name, sizeof(name), "matmul_%s_weight", c->name);
        emit(name, "u1", c->weights, c->weight_bytes);
        snprintf(name, sizeof(name), "matmul_%s_input_f32", c->name);
        emit(name, "f4", c->input_f32, c->N * c->K * 4);
        snprintf(name, sizeof(name), "matmul_%s_input_f16", c->name);
        emit(name, "u2", c->input_f16, c->N * c->K * 2);
        snprintf(name, sizeof(name), "matmul_%s_expected_f32", c->name);
        emit(name, "f4", c->expected_f32, c->N * c->M * 4);
        snprintf(name, sizeof(name), "matmul_%s_expected_f16", c->name);
        emit(name, "f4", c->expected_f16, c->N * c->M * 4);
    }
    /* e4m3 conversion goldens (g_conv_fp8, g_conv_fp8_half_bridge, tests/backend/golden_data.h:1859-1893) */
    emit("g_conv_fp8_src", "f4", g_conv_fp8.src, sizeof(g_conv_fp8.src));
    emit("g_conv_fp8_e4m3_bits", "u1", g_conv_fp8.e4m3_bits, sizeof(g_conv_fp8.e4m3_bits));
    emit("g_conv_fp8_e4m3_roundtrip", "f4", g_conv_fp8.e4m3_roundtrip, sizeof(g_conv_fp8.e4m3_roundtrip));
    emit("g_conv_fp8_half_bridge_src", "f4", g_conv_fp8_half_bridge.src, sizeof(g_conv_fp8_half_bridge.src));
    emit("g_conv_fp8_half_bridge_f16_bits", "u2", g_conv_fp8_half_bridge.f16_bits, sizeof(g_conv_fp8_half_bridge.f16_bits));
    emit("g_conv_fp8_half_bridge_fp8_bits", "u1", g_conv_fp8_half_bridge.fp8_bits, sizeof(g_conv_fp8_half_bridge.fp8_bits));
    emit("g_conv_fp8_half_bridge_roundtrip", "f4", g_conv_fp8_half_bridge.roundtrip, sizeof(g_conv_fp8_half_bridge.roundtrip));
    /* the goldens of the tensor operations around the linears (tests/backend/golden_data.h): activations :449-476,
     * softmax :521-545, slice :998-1040, FLOAT16 / BFLOAT16 conversions :1811-1858 */
#define EMIT_FIELD(obj, field, dtype) emit(#obj "_" #field, dtype, obj.field, sizeof(obj.field))
    EMIT_FIELD(g_activation, input, "f4");
    EMIT_FIELD(g_activation, gelu, "f4");
    EMIT_FIELD(g_activation, silu, "f4");
    EMIT_FIELD(g_activation, gelu_tanh, "f4");
    EMIT_FIELD(g_softmax, shape, "u8");
    EMIT_FIELD(g_softmax, input, "f4");
    EMIT_FIELD(g_softmax, expected_axis_last, "f4");
    EMIT_FIELD(g_softmax, expected_axis0, "f4");
    EMIT_FIELD(g_tensor_slice3d, shape_src, "u8");
    EMIT_FIELD(g_tensor_slice3d, starts, "u8");
    EMIT_FIELD(g_tensor_slice3d, sizes, "u8");
    EMIT_FIELD(g_tensor_slice3d, src, "f4");
    EMIT_FIELD(g_tensor_slice3d, expected, "f4");
    EMIT_FIELD(g_conv_f16, src, "f4");
    EMIT_FIELD(g_conv_f16, f16_bits, "u2");
    EMIT_FIELD(g_conv_f16, roundtrip, "f4");
    EMIT_FIELD(g_conv_bf16, src, "f4");
    EMIT_FIELD(g_conv_bf16, bf16_bits, "u2");
    EMIT_FIELD(g_conv_bf16, roundtrip, "f4");
    EMIT_FIELD(g_conv_f16_bf16_bridge, src, "f4");
    EMIT_FIELD(g_conv_f16_bf16_bridge, f16_bits, "u2");
    EMIT_FIELD(g_conv_f16_bf16_bridge, bf16_bits, "u2");
    EMIT_FIELD(g_conv_f16_bf16_bridge, bf16_from_f16_bits, "u2");
    EMIT_FIELD(g_conv_f16_bf16_bridge, f16_from_bf16_bits, "u2");
    return 0;
}

/*
 * marmot_oracle — TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, CPU-only restatement of the arithmetic of marmot's CPU backend for
 * block-quantized (GGUF) weight x float activation matmul.  It exists to check
 * the HIP kernels and to be timed as the CPU baseline; nothing in the product
 * library links, loads or calls it.
 *
 * Every function names the reference file:line whose behaviour it restates
 * (paths relative to the reference checkout).  The restatement follows the
 * reference's *scalar* configuration (no NEON/AVX2 paths, no FMA contraction),
 * which fixes rounding: Q8_0 uses roundf (half away from zero), K-quants use
 * the magic-number round-to-nearest-even.
 *
 * Pinned by (see tests/test_oracle_*.py):
 *   - the reference's own golden vectors for quantizer bytes, dequantized
 *     values, block dot products and whole matmuls;
 *   - a shared library compiled from the reference's own leaf sources
 *     (oracle/_ref) on seeded Gaussian rows, byte- and bit-exact;
 *   - float64 brute force and closed-form special cases.
 * "parity unpinned": none of the functions below; the MoE driver and top-k are
 * pinned by brute force against dense math and the reference tests' tie cases
 * only (the reference holds no golden vector for them).
 */
#ifndef MARMOT_ORACLE_H
#define MARMOT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* quant kinds: numeric values of marmot_quant_kind_t (include/marmot/types.h:372-388) */
enum {
    MO_KIND_Q4_0 = 1,
    MO_KIND_Q4_1 = 2,
    MO_KIND_Q5_0 = 3,
    MO_KIND_Q5_1 = 4,
    MO_KIND_Q8_0 = 5,
    MO_KIND_Q8_1 = 6,
    MO_KIND_Q2_K = 7,
    MO_KIND_Q3_K = 8,
    MO_KIND_Q4_K = 9,
    MO_KIND_Q5_K = 10,
    MO_KIND_Q6_K = 11,
    MO_KIND_Q8_K = 12,
};

/* dtype ids: numeric values of marmot_dtype_t (include/marmot/types.h:340-362) */
enum {
    MO_DTYPE_F32 = 0,
    MO_DTYPE_F16 = 1,
    MO_DTYPE_BF16 = 2,
    MO_DTYPE_I32 = 3,
    MO_DTYPE_I64 = 11,
    MO_DTYPE_F8_E4M3 = 14,
};

enum {
    MO_ROUTER_SOFTMAX_SELECTED = 0,
    MO_ROUTER_SOFTMAX_SELECTED_SCALED = 1,
    MO_ROUTER_RENORMALIZE_SELECTED = 2,
};

enum { MO_FFN_SWIGLU = 0, MO_FFN_GEGLU = 2 };

/* block geometry (include/marmot/quant_block.h:20-125) */
size_t mo_block_values(int kind);
size_t mo_block_bytes(int kind);
size_t mo_row_bytes(int kind, size_t k);

/* fp16 <-> fp32: exact widening, round-to-nearest-even narrowing
 * (the reference uses a native _Float16 cast, cpu_backend_internal.h:600-606) */
float mo_f16_to_f32(uint16_t h);
uint16_t mo_f32_to_f16(float f);

/* weight quantizers: `rows` rows of `k` floats -> rows * mo_row_bytes(kind,k) bytes.
 * Tails are zero-padded per block (ops/quantize_core.c:199-265). Returns 0 on success. */
int mo_quantize_rows(int kind, const float *x, size_t rows, size_t k, void *out);

/* dequantizers (the bit-exact contract). Returns 0 on success. */
int mo_dequantize_rows(int kind, const void *blocks, size_t rows, size_t k, float *out);

/* activation packers (matmul_quant_pack.c:23-196). in_dtype: MO_DTYPE_F32/F16. */
void mo_pack_q8_0(const void *x, int in_dtype, size_t k, void *blocks_out);
void mo_pack_q8_k(const void *x, int in_dtype, size_t k, void *blocks_out);

/* integer block dots (vec_dot_impl.h) over `nblocks` consecutive blocks */
float mo_vec_dot_q8_0_q8_0(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q4_0_q8_0(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q4_1_q8_0(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q8_1_q8_0(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q5_0_q8_0(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q5_1_q8_0(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q2_k_q8_k(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q3_k_q8_k(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q4_k_q8_k(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q5_k_q8_k(const void *w, const void *a, size_t nblocks);
float mo_vec_dot_q6_k_q8_k(const void *w, const void *a, size_t nblocks);

/* fp16-activation direct dots (vec_dot_impl.h:220-250, 419-450, 973-1023) */
float mo_vec_dot_f16(int kind, const void *w, const uint16_t *a, size_t nblocks, size_t k);

/*
 * marmot_linear for a quantized weight: out[n*M + m] = dot(W[m,:], x[n,:]) (+ bias[m]).
 *   in_dtype F32  -> packed path (Q8_0 for Q4_0/Q8_0 weights, Q8_K for K-quants)
 *   in_dtype F16  -> direct path unless force_pack != 0
 *   out_dtype F32 or F16 (F16 only allowed with F16 input)
 *   bias: NULL or M floats (fp32 bias; applied after the store like the reference)
 *   threads: weight rows are split over this many worker threads (>=1)
 * Returns 0, or a negative marmot_error_t value on invalid arguments.
 */
int mo_matmul_quantized(
    int kind, const void *weight, const void *input, int in_dtype, size_t N, size_t K, size_t M, const float *bias,
    void *out, int out_dtype, int force_pack, int threads
);

/*
 * marmot_matmul_qkv, separate block-quantized weights (src/backends/cpu/ops/matmul/qkv/matmul_qkv.c:749-947):
 * three weights of one kind and shape [M,K], one input [N,K] of in_dtype (F32 or F16), outputs [N,M] of the same
 * dtype. Per input row the activations are packed once (Q8_0 or Q8_K, also for F16 input), then for every m
 * acc = (float)bias[m] + dot(w_row, act, all blocks of the row) and the store rounds once to the output dtype.
 * wq/wk/wv weights; bias[i]: NULL or M values of bias_dtype (F32 or F16); out[i]: N*M values of in_dtype.
 * The rotary epilogue (rope_params) is not restated.
 */
int mo_matmul_qkv_separate(
    int kind, const void *const weights[3], const void *input, int in_dtype, size_t N, size_t K, size_t M,
    const void *const bias[3], int bias_dtype, void *const out[3]
);

/* marmot_rope_params_t without the positions tensor (include/marmot/ops_types.h:98-112) */
typedef struct {
    int scaling_type; /* -1 unspecified, 0 none, 1 linear, 2 yarn, 3 longrope (include/marmot/types.h:254-261) */
    int rope_type;    /* 0 norm: pairs (2i, 2i+1); 1 neox: pairs (i, i + head_dim/2) */
    float theta, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
    uint32_t orig_ctx_len, head_dim;
    int apply_to_q, apply_to_k;
} mo_rope_params;

/* cpu_matmul_qkv_resolve_head_dim (matmul_qkv_rope.h:14-23) */
size_t mo_rope_resolve_head_dim(size_t dim, uint32_t head_dim);

/*
 * marmot_rope_freq_cache_ensure without the cache (src/core/helpers/rope.c:61-127, 143-200): head_dim/2 angular
 * frequencies theta^(-2i/head_dim) * scale and the attention scale, including the YaRN ramp (ext_factor != 0 after
 * rope_scaling_prepare: correction range rope.c:38-59, ramp :28-36, attention scale :95-99).
 */
int mo_rope_frequencies(const mo_rope_params *p, size_t head_dim, float *freqs_out, float *attn_scale_out);

/* cpu_matmul_qkv_rotate_row_f32_headed (matmul_qkv_rope.h:50-70, 123-138): in-place rotation of one fp32 row */
void mo_rope_rotate_row(float *row, size_t dim, size_t head_dim, float position, const float *freqs, float attn_scale,
                        int rope_type);

/*
 * marmot_rope on rows (cpu_rope, src/backends/cpu/ops/rope/rope_dispatch.c:145-372, scalar path): x and out hold
 * `rows` rows of `dim` values of dtype (MO_DTYPE_F32 or MO_DTYPE_F16) at the given row strides (in elements, >= dim);
 * row r is rotated by positions[r] with the frequencies of mo_rope_frequencies(rope, dim); rope->head_dim and the
 * apply flags play no part. x == out is allowed. Pinned by the closed form and the inputs of the reference's own test
 * (tests/backend/test_rope.c:5-42, 44-118).
 */
int mo_rope(
    const void *x, int dtype, size_t rows, size_t dim, size_t x_row_stride, size_t out_row_stride,
    const mo_rope_params *rope, const void *positions, int pos_dtype, void *out
);

/*
 * mo_matmul_qkv_separate with the rotary epilogue (matmul_qkv.c:812-822, 829-831, 917-925, 700-747): q and/or k rows
 * are rotated in fp32 before the store. positions: N values of pos_dtype (MO_DTYPE_F32, MO_DTYPE_I32 or
 * MO_DTYPE_I64), converted to float as cpu_rope_position_as_f32 does (cpu_backend_internal.h:567-578).
 */
int mo_matmul_qkv_separate_rope(
    int kind, const void *const weights[3], const void *input, int in_dtype, size_t N, size_t K, size_t M,
    const void *const bias[3], int bias_dtype, void *const out[3], const mo_rope_params *rope, const void *positions,
    int pos_dtype
);

/*
 * marmot_embedding_gather with a block-quantized table (cpu_embedding_gather_scalar ->
 * cpu_embedding_run_worker / cpu_embedding_copy_row_quantized, src/backends/cpu/ops/embedding/scalar/
 * embedding_scalar.c:241-303, 381-447): weights = vocab rows of row_bytes(kind, dim); ids: n values of ids_dtype
 * (MO_DTYPE_I32 or MO_DTYPE_I64); out: [n, dim] of out_dtype (F32 or F16), value = decoded * scale (one rounding for
 * F16). A token equal to padding_id (when padding_id >= 0) gives a zero row; a token outside [0, vocab) gives a zero
 * row, or MO_ERR_INVALID_ARGUMENT when bounds_check is set (*error_index receives the position). Q4_0 rows are decoded
 * in the table's interleaved nibble order (value i = nibble i % 2 of byte i / 2, :221-229), the other kinds with
 * their block dequantizers.
 */
int mo_embedding_gather_quantized(
    int kind, const void *weights, size_t vocab, size_t dim, const void *ids, int ids_dtype, size_t n, void *out,
    int out_dtype, float scale, int32_t padding_id, int bounds_check, size_t *error_index
);

/* top-k over the last axis, ties -> lower index (moe_ops.c:789-889) */
int mo_topk(const float *x, size_t rows, size_t cols, size_t k, float *values_out, int32_t *indices_out);

/* router: softmax over the k selected logits (graph_builder.cpp:2276-2316) */
void mo_softmax_rows(const float *x, size_t rows, size_t k, float *out);

/* RMS normalization of fp32 rows, scalar path (normalization_scalar.c:469-510, 780-791); weight_offset 1 is the Gemma
 * variant. residual / weight may be NULL. */
int mo_rms_norm(const float *x, const float *residual, const float *weight, float weight_offset, float eps,
                size_t rows, size_t cols, float *out);
/* silu(gate) * up, or gelu_tanh(gate) * up when geglu != 0 (elementwise_f32_scalar.c:11-20, 147-214) */
int mo_glu(const float *gate, const float *up, size_t n, int geglu, float *out);

/* act(gate[i]) * up[i] as the expert body computes it between the projections (moe_ops.c:548-559);
 * out may alias gate. */
int mo_moe_glu(const float *gate, const float *up, size_t n, int ffn_type, float *out);

/*
 * marmot_moe_experts, fp32 activations, block-quantized experts (moe_ops.c:891-1049, 622-787).
 * gate/up: E slices of [F, H] rows; down: E slices of [H, F]. kind_gate_up / kind_down are quant kinds.
 * force_grouped != 0 disables the <=4-token decode path.
 */
int mo_moe_experts(
    const float *hidden, size_t T, size_t H, size_t F, size_t E, size_t k_per_token, int kind_gate_up, int kind_down,
    const void *gate, const void *up, const void *down, const int32_t *topk_ids, const float *topk_weights,
    float weights_scale, int policy, int ffn_type, int force_grouped, int threads, float *out
);

/* row grain used to split weight rows over threads (matmul_quant_compute.c:1222-1240) */
size_t mo_row_grain(size_t row_count, size_t cols_in_tile, size_t thread_cap);

/* ======================= paged attention ======================= */
/* cpu_paged_attention_impl (src/backends/cpu/ops/paged_attention/paged_attention_ref.c:573-1082) for FLOAT32 / FLOAT16 /
 * BFLOAT16 activations and KV caches (the FP8 cache of MARMOT_ENABLE_FP8 builds is not restated): first every token's
 * k_new / v_new rows are written into the paged cache at the token's kv_slot (:346-373), then every token attends over
 * positions 0 .. pos of its sequence through the block table with an online softmax in blocks of block_n positions
 * (:398-569; scalar kernels paged_attention/scalar). All strides are in elements.
 *   token_meta  [token_count, 4] uint32: seq_slot, pos, kv_slot, flags (flags are not read)
 *   q, out      [tokens, num_q_heads, head_dim], k_new, v_new [tokens, num_kv_heads, head_dim] of act_dtype
 *   kv_k, kv_v  [blocks, layers, num_kv_heads, block_size, head_dim] of kv_dtype (updated in place)
 *   block_table [max_seqs, max_blocks_per_seq] uint32, 0xFFFFFFFF = no block */
typedef struct {
    uint32_t token_count, layer_idx, num_q_heads, num_kv_heads, head_dim, block_size;
    float scale;
    int act_dtype, kv_dtype;
    const uint32_t *token_meta;
    size_t meta_stride[2];
    const void *q, *k_new, *v_new;
    size_t q_stride[3], k_stride[3], v_stride[3];
    void *kv_k, *kv_v;
    size_t kv_stride[5];
    size_t kv_blocks, kv_layers;
    const uint32_t *block_table;
    size_t table_stride[2];
    size_t max_seqs, max_blocks_per_seq;
    void *out;
    size_t out_stride[3];
    /* kv_dtype == MO_DTYPE_F8_E4M3 (paged_attention_ref.c:825-989): one fp32 scale per (block, layer, kv head) for keys
     * and for values, [blocks, layers, kv heads] at scale_stride, read and updated: a block's scale is the largest
     * magnitude among its rows below the first offset written by this call (decoded with the old scale) and the new
     * rows, divided by 240; rows already in the block are re-encoded when the scale changes. */
    float *kv_k_scale, *kv_v_scale;
    size_t scale_stride[3];
} mo_paged_attention_args;

int mo_paged_attention(const mo_paged_attention_args *a);

/* marmot_f32_to_fp8_e4m3_ref / marmot_fp8_e4m3_to_f32_ref (src/utils/dtype_ref.c:118-212): 1-4-3 bits, bias 7, exponent
 * field 15 is NaN, largest finite value 240, round to nearest even, saturating. */
uint8_t mo_f32_to_fp8_e4m3(float value);
float mo_fp8_e4m3_to_f32(uint8_t bits);

/* ---- tensor operations around the linears ----
 * Pinned by tests/test_oracle_tensor_ops.py: the reference's conversion goldens (g_conv_f16, g_conv_bf16,
 * g_conv_f16_bf16_bridge, tests/backend/golden_data.h:1814-1858), numpy's IEEE conversions on every FLOAT16 bit pattern
 * and on seeded values around the rounding ties, the identity gelu(x) - gelu(-x) = x and float64 erf / tanh / exp
 * closed forms, softmax rows that sum to one, are shift invariant and flush at -88, and numpy indexing for the gather
 * and the slice. */
/* op: 0 GELU (erf), 1 GELU (tanh), 2 SiLU; dtype MO_DTYPE_F32 or MO_DTYPE_F16 */
int mo_unary(int op, const void *x, int dtype, size_t n, void *out);
int mo_softmax(const float *x, size_t outer, size_t axis, size_t inner, float *out);
/* the same for FLOAT16 / BFLOAT16 tensors (bit patterns in uint16): exponentials rounded to the type when stored,
 * scaled from the stored value and rounded again (softmax_misc_scalar.c:4-122); pinned by the reference's g_softmax
 * vector at the reference's own tolerances for these types (tests/backend/test_backend_softmax.c:53-54) and by a numpy
 * model of the two roundings */
int mo_softmax_typed(int dtype, const void *x, size_t outer, size_t axis, size_t inner, void *out);
int mo_convert(void *dst, int dst_dtype, const void *src, int src_dtype, size_t n);
int mo_gather_rows(const void *x, size_t rows_in, size_t cols, size_t elem_size, size_t in_stride0, const void *idx,
                   int idx_is_signed, size_t idx_stride, size_t rows_out, void *out, size_t out_stride0,
                   size_t *bad_row);
int mo_slice(const void *x, void *out, size_t elem_size, size_t ndim, const size_t *in_shape, const size_t *out_shape,
             const size_t *starts, const size_t *sizes);

#ifdef __cplusplus
}
#endif

#endif

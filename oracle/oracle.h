/* CPU oracle for the quantized FULLY_CONNECTED path.
 *
 * TEST INFRASTRUCTURE ONLY. This library restates, on the CPU, the arithmetic
 * of the reference's FULLY_CONNECTED kernels so that the HIP path can be
 * checked against it. Nothing in the shipped product (the C-ABI library, the
 * delegate, the Python host mirror) links, loads or calls it: only tests, the
 * smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Every function names the reference file:line it follows. Functions whose
 * result no reference vector, reference build or mathematical identity pins
 * say "parity unpinned" here.
 *
 * Build: `make -C oracle` (g++ -O2 -ffp-contract=off, no fast-math: the
 * reference's x86-64 baseline build has no FMA, and several float steps below
 * are sensitive to contraction).
 */
#ifndef LITERT_AMD_ORACLE_H_
#define LITERT_AMD_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Fused activation codes: TfLiteFusedActivation,
 * tflite/converter/core/c/builtin_op_data.h:79-87. */
enum {
  ORC_ACT_NONE = 0,
  ORC_ACT_RELU = 1,
  ORC_ACT_RELU_N1_TO_1 = 2,
  ORC_ACT_RELU6 = 3,
  ORC_ACT_TANH = 4,
  ORC_ACT_SIGN_BIT = 5,
  ORC_ACT_SIGMOID = 6,
};

/* Which build of the activation quantizer to mimic
 * (tflite/kernels/internal/optimized/sse_tensor_utils.h:286-305 dispatch). */
enum {
  ORC_QUANT_PORTABLE = 0,    /* reference/portable_tensor_utils.cc:41-119 (normative) */
  ORC_QUANT_NEON_V8 = 1,     /* optimized/neon_tensor_utils.cc:2412-2552, __ARM_ARCH >= 8 */
  ORC_QUANT_NEON_LEGACY = 2, /* same file, RoundToNearest fallback :2351-2357 */
};

/* ---- scalar quantization math ------------------------------------------ */

/* tflite/kernels/internal/quantization_util.cc:53-104 (non-emulated, double rounding build). */
void orc_quantize_multiplier(double real_multiplier, int32_t* quantized_multiplier, int* shift);

/* gemmlowp fixedpoint.h @16e8662c (not vendored in the reference): published
 * SaturatingRoundingDoublingHighMul / RoundingDivideByPOT, as called from
 * tflite/kernels/internal/common.cc:83-89. */
int32_t orc_srdhm(int32_t a, int32_t b);
int32_t orc_rounding_divide_by_pot(int32_t x, int exponent);

/* tflite/kernels/internal/common.cc:80-90 (TFLITE_SINGLE_ROUNDING undefined). */
int32_t orc_mbqm(int32_t x, int32_t quantized_multiplier, int shift);
/* tflite/kernels/internal/common.cc:33-47 (TFLITE_SINGLE_ROUNDING build). */
int32_t orc_mbqm_single_rounding(int32_t x, int32_t quantized_multiplier, int shift);

/* tflite/kernels/kernel_util.cc:343-412 for an int8 output tensor. Returns 0
 * on success, 1 when the reference would fail its overflow check. */
int orc_activation_range_int8(int activation, float out_scale, int32_t out_zero_point,
                              int32_t* act_min, int32_t* act_max);

/* IEEE binary16 -> binary32 including subnormals, inf and NaN; stands in for
 * Eigen::half -> float used at tflite/kernels/fully_connected.cc:1030-1036. */
float orc_half_to_float(uint16_t h);

/* tflite/kernels/internal/portable_tensor_utils.cc:96-127, bit_width 4, signed. */
void orc_unpack_int4(const int8_t* src, int num_elements, int8_t* dst);

/* tflite/kernels/internal/portable_tensor_utils.cc:128-163, bit_width 2, signed: four values
 * per byte, the first in bits 0-1; a last partial byte gives num_elements % 4 values. */
void orc_unpack_int2(const int8_t* src, int num_elements, int8_t* dst);

/* ---- Prepare-time derivations ------------------------------------------ */

/* tflite/kernels/fully_connected.cc:552-564. Returns 0. */
int orc_fc_prepare_per_channel(float input_scale, const float* filter_scales, int num_channels,
                               float output_scale, int32_t* multipliers, int32_t* shifts);

/* tflite/kernels/fully_connected.cc:566-573 with kernel_util.cc:291-341.
 * Returns 0 on success, 1 when the bias-scale sanity check or the
 * non-negative-scale check fails. */
int orc_fc_prepare_per_tensor(float input_scale, float filter_scale, int has_bias,
                              float bias_scale, float output_scale, int32_t* multiplier,
                              int32_t* shift);

/* ---- full-integer int8 FULLY_CONNECTED --------------------------------- */

/* reference/integer_ops/fully_connected.h:35-77 (multiplier form, normative).
 * input [batches, depth], filter [out_depth, depth], output [batches, out_depth].
 * bias may be NULL. */
void orc_fc_int8_per_channel(const int8_t* input, const int8_t* filter, const int32_t* bias,
                             const int32_t* multipliers, const int32_t* shifts, int8_t* output,
                             int batches, int depth, int out_depth, int32_t input_offset,
                             int32_t output_offset, int32_t act_min, int32_t act_max);

/* Same loop with the single-rounding multiplier, to report mismatch counts. */
void orc_fc_int8_per_channel_single_rounding(const int8_t* input, const int8_t* filter,
                                             const int32_t* bias, const int32_t* multipliers,
                                             const int32_t* shifts, int8_t* output, int batches,
                                             int depth, int out_depth, int32_t input_offset,
                                             int32_t output_offset, int32_t act_min,
                                             int32_t act_max);

/* reference/integer_ops/fully_connected.h:83-132 (float-scale form used by
 * Register_FULLY_CONNECTED_REF, call site fully_connected.cc:1401-1411). */
void orc_fc_int8_per_channel_float_scale(const int8_t* input, const int8_t* filter,
                                         const int32_t* bias, const float* filter_scales,
                                         float input_scale, float output_scale, int8_t* output,
                                         int batches, int depth, int out_depth,
                                         int32_t input_offset, int32_t output_offset,
                                         int32_t act_min, int32_t act_max);

/* reference/integer_ops/fully_connected.h:136-180 (per-tensor, multiplier form). */
void orc_fc_int8_per_tensor(const int8_t* input, const int8_t* filter, const int32_t* bias,
                            int32_t multiplier, int shift, int8_t* output, int batches, int depth,
                            int out_depth, int32_t input_offset, int32_t filter_offset,
                            int32_t output_offset, int32_t act_min, int32_t act_max);

/* The legacy uint8 kernel, tflite/kernels/internal/reference/fully_connected.h:118-166
 * (multiplier form: what the op computes unless built with the reference kernel type, whose
 * float-scale form :68-116 the reference's test vectors do not tell apart). Offsets are the
 * negated zero points of the uint8 tensors. */
void orc_fc_uint8_per_tensor(const uint8_t* input, const uint8_t* filter, const int32_t* bias,
                             int32_t multiplier, int shift, uint8_t* output, int batches, int depth,
                             int out_depth, int32_t input_offset, int32_t filter_offset,
                             int32_t output_offset, int32_t act_min, int32_t act_max);

/* CalculateActivationRangeQuantized for a uint8 output (kernel_util.cc:354-412 with the limits
 * 0 and 255). Returns 1 where the quantized bound leaves int32. */
int orc_activation_range_uint8(int activation, float out_scale, int32_t out_zero_point,
                               int32_t* act_min, int32_t* act_max);

/* reference/integer_ops/fully_connected.h:186-233 (per-tensor, float-scale form). */
void orc_fc_int8_per_tensor_float_scale(const int8_t* input, const int8_t* filter,
                                        const int32_t* bias, float input_scale,
                                        float filter_scale, float output_scale, int8_t* output,
                                        int batches, int depth, int out_depth,
                                        int32_t input_offset, int32_t filter_offset,
                                        int32_t output_offset, int32_t act_min, int32_t act_max);

/* ---- activation quantization ------------------------------------------- */

/* AsymmetricQuantizeFloats, one row. variant = ORC_QUANT_*. */
void orc_asymmetric_quantize_floats(const float* values, int size, int8_t* quantized,
                                    float* scaling_factor, int32_t* offset, int variant);
/* SymmetricQuantizeFloats, one row. */
void orc_symmetric_quantize_floats(const float* values, int size, int8_t* quantized,
                                   float* scaling_factor, int variant);
/* tflite/kernels/internal/portable_tensor_utils.h:158-176. */
void orc_batch_quantize_floats(const float* values, int n_batch, int n_data, int8_t* quantized,
                               float* scaling_factors, int32_t* zero_points, int do_asymmetric,
                               int variant);

/* ---- hybrid (float activations, int8 weights) -------------------------- */

/* The same product as the reference's optimized x86 build computes it
 * (optimized/sse_tensor_utils.cc:308-379, SSE branch), in oracle_sse.cc; row_sums must be
 * filled when input_offset is given. orc_have_sse() is 0 on other hosts (the function is
 * then a no-op). */
int orc_have_sse(void);
void orc_matrix_batch_vector_multiply_accumulate_sse(
    const int8_t* matrix, int m_rows, int m_cols, const int8_t* vectors,
    const float* scaling_factors, int n_batch, float* result, const float* per_channel_scale,
    const int32_t* input_offset, const int32_t* row_sums);

/* reference/portable_tensor_utils.cc:165-206 (+ :140-163 when input_offset is
 * NULL). row_sums is recomputed when compute_row_sums is non-zero. */
void orc_matrix_batch_vector_multiply_accumulate(const int8_t* matrix, int m_rows, int m_cols,
                                                 const int8_t* vectors,
                                                 const float* scaling_factors, int n_batch,
                                                 float* result, const float* per_channel_scale,
                                                 const int32_t* input_offset, int32_t* row_sums,
                                                 int compute_row_sums);

/* tflite/kernels/internal/tensor_utils.h:58-77 for None/Relu/ReluN1To1/Relu6/SignBit
 * (portable_tensor_utils.cc:41-70). Returns 1 for tanh/sigmoid (Eigen: not restated). */
int orc_apply_activation(float* data, int size, int activation);

/* tflite/kernels/fully_connected.cc:763-858 (EvalHybridDense), int8 filter.
 * per_channel_scales == NULL means per-tensor with filter_scale. bias may be
 * NULL. q_out/sf_out/zp_out (each may be NULL) receive the quantized
 * activations. Returns 0, or 1 for an unsupported activation. */
int orc_fc_hybrid(const float* input, int batches, int depth, const int8_t* filter, int out_depth,
                  const float* per_channel_scales, float filter_scale, const float* bias,
                  int asymmetric_quantize_inputs, int activation, int quant_variant,
                  float* output, int8_t* q_out, float* sf_out, int32_t* zp_out);

/* Same, with the row sums kept by the caller as the op keeps them in a persistent
 * temporary (fully_connected.cc:700-708): computed when compute_row_sums != 0,
 * reused otherwise. This is the form the CPU-baseline timing uses. */
int orc_fc_hybrid_cached(const float* input, int batches, int depth, const int8_t* filter,
                         int out_depth, const float* per_channel_scales, float filter_scale,
                         const float* bias, int asymmetric_quantize_inputs, int activation,
                         int quant_variant, float* output, int8_t* q_out, float* sf_out,
                         int32_t* zp_out, int32_t* row_sums, int compute_row_sums);

/* ---- blockwise int4 weights -------------------------------------------- */

/* BATCH_MATMUL, float x int8 (hybrid): tflite/kernels/batch_matmul.cc:454-520 over the
 * kernel of tflite/kernels/internal/reference/batch_matmul.h:111-210. lhs: lhs_batches x rows
 * x depth floats; weights: weight_matrices x units x depth int8 (the op's RHS after its
 * transposition); per_channel_scales [units] or NULL (then filter_scale); output batch b =
 * lhs batch lhs_batch_index[b] x weight matrix rhs_batch_index[b], [out_batches, rows, units].
 * The reference's own vectors for it (batch_matmul_test.cc:504-985) are tolerance-class; at
 * the bit level it is pinned by reduction to orc_fc_hybrid wherever the float detour of its
 * zero-point correction is exact, and by a numpy float32 replay of that detour where it is
 * not (tests/test_oracle_batch_matmul.py). */
void orc_batch_matmul_hybrid(const float* lhs, int lhs_batches, int rows, int depth,
                             const int8_t* weights, int weight_matrices, int units,
                             const float* per_channel_scales, float filter_scale,
                             int asymmetric_quantize_inputs, int quant_variant,
                             const int* lhs_batch_index, const int* rhs_batch_index,
                             int out_batches, float* output);

/* tflite/kernels/fully_connected.cc:1014-1086 (EvalBlockwise4Bit), float ops
 * in source order and uncontracted. packed_filter holds out_depth rows of
 * ceil_even(depth)/2 bytes, low nibble = even k. scales_f16 [out_depth,
 * depth/blocksize]. bias may be NULL. PARITY UNPINNED at bit level: the
 * reference holds no vectors for this function and its float chain may be
 * FMA-contracted by the reference's compiler; checked here only through the
 * identities in tests/test_oracle_blockwise.py. */
void orc_fc_blockwise_int4(const float* input, int batches, int depth,
                           const uint8_t* packed_filter, int out_depth,
                           const uint16_t* scales_f16, int blocksize, const float* bias,
                           int quant_variant, float* output);

/* EvalHybridDense4Bit (per-channel int4 weights, symmetric activations); see oracle.cc. */
void orc_fc_hybrid_int4_per_channel(const float* input, int batches, int depth,
                                    const uint8_t* packed_filter, int out_depth,
                                    const float* filter_scales, const float* bias,
                                    int activation, float* output);

/* ---- EMBEDDING_LOOKUP from quantized tables ------------------------------ */

/* IEEE binary32 -> binary16, round to nearest even (tflite/types/half.h:69, :129). */
uint16_t orc_float_to_half(float f);

/* tflite/kernels/embedding_lookup.cc:194-307 (EvalBlockwise, Int4 table, fp16 block scales
 * [rows, cols/blocksize]). output: float32 or (out_f16) binary16 [count, cols]. Returns 0,
 * -(position+1) of the first lookup outside [0, rows), or 1 when blocksize does not divide cols. */
int orc_embedding_lookup_blockwise_int4(const int32_t* lookup, int count, const uint8_t* table,
                                        int rows, int cols, const uint16_t* scales_f16,
                                        int blocksize, int out_f16, void* output);

/* tflite/kernels/embedding_lookup.cc:309-395 (EvalHybrid) for value_bits 8 or 4; one scale or
 * row_scales[rows]. */
int orc_embedding_lookup_hybrid(const int32_t* lookup, int count, const void* table, int value_bits,
                                int rows, int cols, float scale, const float* row_scales,
                                int out_f16, void* output);

#ifdef __cplusplus
}
#endif
#endif /* LITERT_AMD_ORACLE_H_ */

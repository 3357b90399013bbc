/* litert_amd_fc.h — C ABI of the MI355X (gfx950) quantized FULLY_CONNECTED kernels.
 *
 * This is the thin layer between the TfLiteDelegate / LiteRT accelerator host
 * code and the hand-written HIP kernels. Every entry point takes plain
 * pointers and sizes. Unless a parameter says "host", data pointers are DEVICE
 * pointers and `stream` is a hipStream_t passed as void* (NULL = the default
 * stream). Calls are asynchronous with respect to the host: they enqueue work
 * on `stream` and return. Every function returns 0 on success and a non-zero
 * LrtFcStatus otherwise; lrtfc_last_error() then describes the failure for the
 * calling thread.
 *
 * Tensor conventions are the reference's: input [batches, depth] row-major,
 * filter [out_depth, depth] row-major, output [batches, out_depth] row-major
 * (tflite/kernels/internal/reference/integer_ops/fully_connected.h:57-76).
 */
#ifndef LITERT_AMD_FC_H_
#define LITERT_AMD_FC_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: lrtfc_int4_group_node gained nibble_filter, lrtfc_int4_group_launch gained form. */
#define LRTFC_ABI_VERSION 2

typedef enum LrtFcStatus {
  LRTFC_OK = 0,
  LRTFC_INVALID_ARGUMENT = 1, /* shape, alignment or NULL-pointer contract broken */
  LRTFC_NO_DEVICE = 2,        /* no gfx950 device visible to HIP */
  LRTFC_HIP_ERROR = 3,        /* a HIP runtime call failed */
  LRTFC_UNSUPPORTED = 4,      /* valid request this build does not implement */
} LrtFcStatus;

/* Fused activation, numbered as TfLiteFusedActivation
 * (tflite/converter/core/c/builtin_op_data.h:79-87). */
typedef enum LrtFcActivation {
  LRTFC_ACT_NONE = 0,
  LRTFC_ACT_RELU = 1,
  LRTFC_ACT_RELU_N1_TO_1 = 2,
  LRTFC_ACT_RELU6 = 3,
  /* 4 (tanh) and 6 (sigmoid) go through Eigen in the reference and are not offered. */
  LRTFC_ACT_SIGN_BIT = 5, /* float outputs only: 1.0f where the sign bit is set, else 0.0f
                             (tflite/kernels/internal/portable_tensor_utils.cc:65-71) */
} LrtFcActivation;

/* Which build of the reference's activation quantizer to reproduce bit for bit
 * (dispatch: tflite/kernels/internal/optimized/sse_tensor_utils.h:286-305). */
typedef enum LrtFcQuantVariant {
  LRTFC_QUANT_PORTABLE = 0,    /* reference/portable_tensor_utils.cc:41-119 (default) */
  LRTFC_QUANT_NEON_V8 = 1,     /* optimized/neon_tensor_utils.cc:2412-2552, ARMv8 rounding */
  LRTFC_QUANT_NEON_LEGACY = 2, /* same file, RoundToNearest fallback :2351-2357 */
} LrtFcQuantVariant;

/* ---- library ------------------------------------------------------------ */

int lrtfc_abi_version(void);
/* Message for the last failing call on this thread ("" when none). */
const char* lrtfc_last_error(void);
/* Selects `device_ordinal` and checks that it is a gfx950 part. Must succeed
 * before any entry point that touches device memory is used. */
int lrtfc_init(int device_ordinal);

/* ---- Prepare-time math (host only, no device access) --------------------- */

/* Replaces tflite::QuantizeMultiplier,
 * tflite/kernels/internal/quantization_util.cc:53-104. */
int lrtfc_quantize_multiplier(double real_multiplier, int32_t* quantized_multiplier, int* shift);

/* Replaces the per-channel loop of fully_connected::PrepareImpl,
 * tflite/kernels/fully_connected.cc:552-564. Host arrays of `num_channels`. */
int lrtfc_prepare_per_channel(float input_scale, const float* filter_scales, int num_channels,
                              float output_scale, int32_t* multipliers, int32_t* shifts);

/* Replaces the per-tensor branch, tflite/kernels/fully_connected.cc:566-573 with
 * GetQuantizedConvolutionMultipler, tflite/kernels/kernel_util.cc:291-341
 * (bias-scale sanity check included: fails with LRTFC_INVALID_ARGUMENT as the
 * reference fails Prepare). */
int lrtfc_prepare_per_tensor(float input_scale, float filter_scale, int has_bias,
                             float bias_scale, float output_scale, int32_t* multiplier,
                             int32_t* shift);

/* Replaces CalculateActivationRangeQuantized for an int8 output,
 * tflite/kernels/kernel_util.cc:354-412. */
int lrtfc_activation_range_int8(int activation, float output_scale, int32_t output_zero_point,
                                int32_t* act_min, int32_t* act_max);

/* ---- weight preparation on the device (once per constant filter) --------- */

/* row_sums[n] = sum_k filter[n,k]. Replaces PortableReductionSumVector as used
 * for the hybrid path's compute_row_sums step
 * (tflite/kernels/internal/reference/portable_tensor_utils.cc:179-184); the
 * full-integer kernels use the same sums to fold input_offset. */
int lrtfc_row_sums_int8(const int8_t* filter, int out_depth, int depth, int32_t* row_sums,
                        void* stream);

/* Replaces tensor_utils::UnpackPackedIntToInt8 (bit_width 4, signed),
 * tflite/kernels/internal/portable_tensor_utils.cc:96-127: low nibble first. */
int lrtfc_unpack_int4(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                      void* stream);

/* The same routine with bit_width 2 (tflite/kernels/internal/portable_tensor_utils.cc:128-163):
 * four signed values per byte, the first in bits 0-1. What FULLY_CONNECTED does with an Int2
 * filter before its int8 kernels, hybrid (tflite/kernels/fully_connected.cc:812-818) and
 * full-integer (:1678-1685) alike. */
int lrtfc_unpack_int2(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                      void* stream);

/* dst[i] = src[i] ^ 0x80: a uint8 tensor as int8 (value - 128) and back; src == dst is allowed.
 * With it the legacy uint8 FULLY_CONNECTED (tflite/kernels/internal/reference/fully_connected.h
 * :118-166, reached from tflite/kernels/fully_connected.cc:1607-1626) runs on the int8 kernels:
 *   sum (w_u8 + fo)(x_u8 + io) = sum (w_i8 + fo + 128)(x_i8 + io + 128),
 *   y_u8 = clamp(M(acc) + oo, lo, hi)  <=>  y_i8 = clamp(M(acc) + oo - 128, lo - 128, hi - 128),
 * i.e. lrtfc_fc_int8 with every zero point lowered by 128 and the same multiplier and shift. */
int lrtfc_xor_sign_bit(const uint8_t* src, uint8_t* dst, size_t bytes, void* stream);

/* kfsum[n] = sum over blocks, in block order and float32, of
 * scale[n,b] * float(sum_k filter[n, b*blocksize + k]): the weight-only part of
 * EvalBlockwise4Bit's zero-point correction
 * (tflite/kernels/fully_connected.cc:1056-1077), hoisted out of the per-call loop. */
int lrtfc_blockwise_int4_kfsum(const uint8_t* packed_filter, const uint16_t* scales_f16,
                               int out_depth, int depth, int blocksize, float* kfsum,
                               void* stream);

/* Which filter layout the Eval entry points run fastest on for a shape: the row-major
 * tensor as the model stores it, or the re-tiled copy made by lrtfc_pack_int8_filter /
 * lrtfc_pack_int4_blockwise. The choice stands where the reference picks a kernel path
 * per shape (tflite/kernels/cpu_backend_gemm.h:116-160 routes matrix-vector products to
 * a custom GEMV and the rest to ruy). Pure host functions; no device needed.
 *   int8 / hybrid: packed, except for per-tensor filters with a non-zero zero point (and
 *   depths too large to stage a row in LDS), which need the row-major kernels. The answer
 *   does not depend on `batches` today; the parameter is kept so that it may. Hybrid callers
 *   pass filter_offset 0.
 *   blockwise int4: packed for block size 32 dividing the depth. */
enum { LRTFC_LAYOUT_ROW_MAJOR = 0, LRTFC_LAYOUT_PACKED = 1 };
int lrtfc_fc_int8_preferred_layout(int batches, int depth, int out_depth, int32_t filter_offset);
int lrtfc_fc_blockwise_int4_preferred_layout(int depth, int blocksize);

/* Up to how many batch rows lrtfc_fc_hybrid_packed should be handed float rows directly (one
 * launch: the row quantizer runs inside the product kernel, one wavefront per row) rather than
 * through lrtfc_fc_hybrid_packed_workspace (row quantizer launch, then the product). Both give
 * the same bits; this is the faster choice per shape, where the reference has a single code path
 * for every batch size (tflite/kernels/fully_connected.cc:847-851). Pure host function. */
int lrtfc_fc_hybrid_fused_max_batches(int depth, int out_depth);

/* Re-tiles a row-major int8 filter [out_depth, depth] for the matrix-core GEMV: tiles of
 * 16 output channels x 64 depth (1 KiB each, zero-padded at the edges), the 16 bytes of
 * lane L inside a tile being channel L % 16, depth 16 * (L / 16) .. +16; tiles of one
 * channel group are consecutive along the depth. This plays the part of the reference's
 * prepacked-LHS cache (tflite/kernels/cpu_backend_gemm_params.h:33-42: constant weights
 * are packed once and reused). `packed` must hold lrtfc_packed_int8_filter_bytes(). */
size_t lrtfc_packed_int8_filter_bytes(int out_depth, int depth);
int lrtfc_pack_int8_filter(const int8_t* filter, int out_depth, int depth, int8_t* packed,
                           void* stream);

/* ---- Eval --------------------------------------------------------------- */

/* Full-integer int8 FULLY_CONNECTED with MultiplyByQuantizedMultiplier
 * requantization (double rounding, tflite/kernels/internal/common.cc:80-90).
 * Replaces FullyConnectedPerChannelInt8 / FullyConnectedInt8
 * (tflite/kernels/fully_connected.cc:1383-1421, 1254-1284) and the kernels they
 * call (reference/integer_ops/fully_connected.h:35-77, 136-180).
 *   per_channel != 0: multipliers/shifts are arrays of out_depth, filter_offset
 *                     must be 0 (weights symmetric).
 *   per_channel == 0: multipliers/shifts point at one value each.
 *   bias may be NULL. filter_row_sums (from lrtfc_row_sums_int8) is required
 *   when input_offset != 0. Any batches >= 1: small batches run the bandwidth-
 *   bound GEMV kernel, large ones the int8 MFMA GEMM. */
int lrtfc_fc_int8(const int8_t* input, const int8_t* filter, const int32_t* bias,
                  const int32_t* multipliers, const int32_t* shifts, int per_channel,
                  const int32_t* filter_row_sums, int8_t* output, int batches, int depth,
                  int out_depth, int32_t input_offset, int32_t filter_offset,
                  int32_t output_offset, int32_t act_min, int32_t act_max, void* stream);

/* lrtfc_fc_int8 on a filter packed by lrtfc_pack_int8_filter, for every batch size: up to
 * 16 rows one matrix-core GEMV kernel whose cost barely grows with the batch; above that an
 * int8 MFMA GEMM that streams the filter once (any batch count and out_depth; depth a
 * multiple of 16, input and filter 16-byte aligned -- other shapes keep the GEMV, one pass
 * over the filter per 16 rows). Same arithmetic
 * contract as lrtfc_fc_int8 with filter_offset == 0; filter_row_sums (of the unpacked
 * filter) is required when input_offset != 0. */
int lrtfc_fc_int8_packed(const int8_t* input, const int8_t* packed_filter, const int32_t* bias,
                         const int32_t* multipliers, const int32_t* shifts, int per_channel,
                         const int32_t* filter_row_sums, int8_t* output, int batches, int depth,
                         int out_depth, int32_t input_offset, int32_t output_offset,
                         int32_t act_min, int32_t act_max, void* stream);

/* Per-row activation quantization. Replaces tensor_utils::BatchQuantizeFloats,
 * tflite/kernels/internal/portable_tensor_utils.h:158-176. zero_points may be
 * NULL when do_asymmetric == 0. */
int lrtfc_batch_quantize_floats(const float* values, int n_batch, int n_data, int8_t* quantized,
                                float* scaling_factors, int32_t* zero_points, int do_asymmetric,
                                int variant, void* stream);

/* Hybrid product on already-quantized activations. Replaces
 * MatrixBatchVectorMultiplyAccumulate (per-channel / offset form,
 * tflite/kernels/internal/reference/portable_tensor_utils.cc:165-206) together
 * with the bias initialisation and ApplyActivationToVector of EvalHybridDense
 * (tflite/kernels/fully_connected.cc:780-786, 854-856), but not its early exit for a whole-zero
 * input (:789-795), which belongs to the entry points that take the float rows.
 *   per_channel_scales NULL: per-tensor, filter_scale is folded into the batch
 *   scaling factor as the reference does (:838-843). bias may be NULL.
 *   zero_points NULL means symmetric activations (all zero). */
int lrtfc_fc_hybrid_int8(const int8_t* quantized_input, const float* scaling_factors,
                         const int32_t* zero_points, const int8_t* filter,
                         const float* per_channel_scales, float filter_scale,
                         const int32_t* filter_row_sums, const float* bias, float* output,
                         int batches, int depth, int out_depth, int activation, void* stream);

/* lrtfc_fc_hybrid_int8 on a packed filter (lrtfc_pack_int8_filter): the form for batches
 * whose rows were quantized by a separate lrtfc_batch_quantize_floats launch (GEMV up to 32
 * rows, MFMA GEMM with the same float epilogue above). Replaces the same reference
 * functions as lrtfc_fc_hybrid_int8. */
int lrtfc_fc_hybrid_int8_packed(const int8_t* quantized_input, const float* scaling_factors,
                                const int32_t* zero_points, const int8_t* packed_filter,
                                const float* per_channel_scales, float filter_scale,
                                const int32_t* filter_row_sums, const float* bias, float* output,
                                int batches, int depth, int out_depth, int activation,
                                void* stream);

/* Bytes of device scratch lrtfc_fc_hybrid / lrtfc_fc_blockwise_int4 need for
 * (batches, depth): quantized activations, scaling factors and zero points. */
size_t lrtfc_activation_workspace_bytes(int batches, int depth);

/* EvalHybridDense end to end (tflite/kernels/fully_connected.cc:763-858):
 * quantizes `input` per row into `workspace`, then runs lrtfc_fc_hybrid_int8.
 * The reference's all-zero-input early exit (:789-795: output = activation(bias), product
 * skipped) is reproduced, down to a bias element of -0.0f staying -0.0f. */
int lrtfc_fc_hybrid(const float* input, const int8_t* filter, const float* per_channel_scales,
                    float filter_scale, const int32_t* filter_row_sums, const float* bias,
                    float* output, int batches, int depth, int out_depth,
                    int asymmetric_quantize_inputs, int activation, int quant_variant,
                    void* workspace, size_t workspace_bytes, void* stream);

/* lrtfc_fc_hybrid without the workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc). It has
 * no counterpart in the reference. The activation scratch is a static device array of
 * LRTFC_STATIC_SCRATCH_BYTES that the library holds on every device it was initialised on
 * (lrtfc_init looks its address up); the call allocates and frees nothing and enqueues the same
 * two launches as lrtfc_fc_hybrid, with bit-identical results. Fails with
 * LRTFC_INVALID_ARGUMENT when lrtfc_activation_workspace_bytes(batches, depth) exceeds
 * LRTFC_STATIC_SCRATCH_BYTES (64 rows of depth 16384 fit). All calls on one device share the
 * one array: calls that overlap on a device (different streams or threads) race; calls ordered
 * on one stream do not. */
#define LRTFC_STATIC_SCRATCH_BYTES (1024 * 1024 + 64 * 1024)
size_t lrtfc_static_scratch_bytes(void);
int lrtfc_fc_hybrid_static_scratch(const float* input, const int8_t* filter,
                                   const float* per_channel_scales, float filter_scale,
                                   const int32_t* filter_row_sums, const float* bias,
                                   float* output, int batches, int depth, int out_depth,
                                   int asymmetric_quantize_inputs, int activation,
                                   int quant_variant, void* stream);

/* lrtfc_fc_hybrid on a packed filter (lrtfc_pack_int8_filter) with the row quantizer as a
 * launch of its own: the form for batch sizes where quantizing every row in every workgroup
 * (lrtfc_fc_hybrid_packed) costs more than a second launch. Replaces EvalHybridDense,
 * tflite/kernels/fully_connected.cc:763-858, all-zero-input early exit included; workspace as
 * for lrtfc_fc_hybrid. Bit-identical results. */
int lrtfc_fc_hybrid_packed_workspace(const float* input, const int8_t* packed_filter,
                                     const float* per_channel_scales, float filter_scale,
                                     const int32_t* filter_row_sums, const float* bias,
                                     float* output, int batches, int depth, int out_depth,
                                     int asymmetric_quantize_inputs, int activation,
                                     int quant_variant, void* workspace, size_t workspace_bytes,
                                     void* stream);

/* EvalHybridDense as ONE kernel on a packed filter: each workgroup quantizes the float
 * rows itself (BatchQuantizeFloats semantics, same three variants) while its weight loads
 * are in flight, so no workspace and no separate quantization launch are needed. Results
 * are bit-identical to lrtfc_fc_hybrid. */
int lrtfc_fc_hybrid_packed(const float* input, const int8_t* packed_filter,
                           const float* per_channel_scales, float filter_scale,
                           const int32_t* filter_row_sums, const float* bias, float* output,
                           int batches, int depth, int out_depth, int asymmetric_quantize_inputs,
                           int activation, int quant_variant, void* stream);

/* Blockwise-int4 hybrid FULLY_CONNECTED. Replaces EvalBlockwise4Bit,
 * tflite/kernels/fully_connected.cc:1014-1086: asymmetric per-row activation
 * quantization, per-block int32 sums, float32 accumulation over blocks in block
 * order, zero-point correction, input scale, bias; the fused activation is
 * ignored as in the reference. packed_filter: out_depth rows of depth/2 bytes,
 * low nibble = even k (depth even). scales_f16: [out_depth, depth/blocksize]
 * IEEE binary16. kfsum from lrtfc_blockwise_int4_kfsum. bias may be NULL. */
int lrtfc_fc_blockwise_int4(const float* input, const uint8_t* packed_filter,
                            const uint16_t* scales_f16, const float* kfsum, const float* bias,
                            float* output, int batches, int depth, int out_depth, int blocksize,
                            int quant_variant, void* workspace, size_t workspace_bytes,
                            void* stream);

/* Re-tiles a blockwise-int4 filter (block size 32) and its fp16 scales for the streaming
 * kernel: tiles of 8 output channels x 64 blocks, nine consecutive 1 KiB planes each (eight
 * of nibbles stored as w + 8, one of scales), tiles of a channel group consecutive along
 * the depth. `packed` must hold lrtfc_packed_int4_blockwise_bytes(). Like the int8
 * re-tiling this stands where the reference prepacks constant weights once
 * (tflite/kernels/fully_connected.cc:1130-1150 does so for its own 4-bit kernels). */
size_t lrtfc_packed_int4_blockwise_bytes(int out_depth, int depth);
int lrtfc_pack_int4_blockwise(const uint8_t* packed_filter, const uint16_t* scales_f16,
                              int out_depth, int depth, int blocksize, uint8_t* retiled,
                              void* stream);

/* lrtfc_fc_blockwise_int4 as ONE kernel on a re-tiled filter: the activation rows are
 * quantized in the kernel's prologue (no workspace). Bit-identical results. */
int lrtfc_fc_blockwise_int4_packed(const float* input, const uint8_t* retiled_filter,
                                   const float* kfsum, const float* bias, float* output,
                                   int batches, int depth, int out_depth, int quant_variant,
                                   void* stream);

/* The same on already-quantized activations. */
int lrtfc_fc_blockwise_int4_packed_quantized(const int8_t* quantized_input,
                                             const float* scaling_factors,
                                             const int32_t* zero_points,
                                             const uint8_t* retiled_filter, const float* kfsum,
                                             const float* bias, float* output, int batches,
                                             int depth, int out_depth, void* stream);

/* ---- BATCH_MATMUL, float x int8 (hybrid) -----------------------------------------------
 * Replaces batch_matmul::EvalHybrid, tflite/kernels/batch_matmul.cc:454-520, with the kernel it
 * runs (tflite/kernels/internal/reference/batch_matmul.h:111-210): every row of the float
 * operand is quantized as in the hybrid FULLY_CONNECTED, and output batch b is
 * rows(b) x weights(b)^T, where the zero-point correction goes through float as the reference
 * kernel's does (:199-200), so results match it bit for bit also beyond 2^24. No bias, no
 * activation (the op has neither).
 *   lhs: [lhs_batches, rows, depth] float32. packed_weights: weight_matrices matrices of
 *   [units, depth] int8 -- the op's RHS with its last two dimensions swapped unless adj_y --
 *   each re-tiled by lrtfc_pack_int8_filter and stored lrtfc_packed_int8_filter_bytes(units,
 *   depth) bytes apart; row_sums: [weight_matrices, units] from lrtfc_row_sums_int8 per matrix.
 *   Broadcasting: lhs_batches == weight_matrices, or either of them 1. output:
 *   [max(lhs_batches, weight_matrices), rows, units]. workspace:
 *   lrtfc_activation_workspace_bytes(lhs_batches * rows, depth), 256-byte aligned. */
int lrtfc_batch_matmul_hybrid_packed(const float* lhs, int lhs_batches, int rows, int depth,
                                     const int8_t* packed_weights, int weight_matrices, int units,
                                     const float* per_channel_scales, float filter_scale,
                                     const int32_t* row_sums, float* output,
                                     int asymmetric_quantize_inputs, int quant_variant,
                                     void* workspace, size_t workspace_bytes, void* stream);

/* The same op with everything its shapes allow (tflite/kernels/batch_matmul.cc:745-813 in front
 * of EvalHybrid): up to three batch dimensions per side (the op extends both shapes to rank 5,
 * reference/batch_matmul.h:120-146), each pair equal or 1 on either side -- also 1 on different
 * sides in different dimensions --, and adj_x. lhs_batch_dims / weight_batch_dims: three ints
 * each, leading 1s for shapes of lower rank. adj_x: lhs is [.., depth, rows] and is transposed
 * into the workspace first, as the op transposes it into a temporary (:811-813). Output:
 * [d0, d1, d2, rows, units] with d_i the broadcast of the two sides' dimension i. workspace:
 * lrtfc_batch_matmul_workspace_bytes(product of lhs_batch_dims, rows, depth, adj_x) bytes,
 * 256-byte aligned. Everything else as above. */
size_t lrtfc_batch_matmul_workspace_bytes(int lhs_matrices, int rows, int depth, int adj_x);
int lrtfc_batch_matmul_hybrid_packed_nd(const float* lhs, const int* lhs_batch_dims, int rows,
                                        int depth, int adj_x, const int8_t* packed_weights,
                                        const int* weight_batch_dims, int units,
                                        const float* per_channel_scales, float filter_scale,
                                        const int32_t* row_sums, float* output,
                                        int asymmetric_quantize_inputs, int quant_variant,
                                        void* workspace, size_t workspace_bytes, void* stream);

/* ---- Per-channel int4 hybrid FULLY_CONNECTED ------------------------------------------
 * Replaces EvalHybridDense4Bit (tflite/kernels/fully_connected.cc:1088-1178) in the
 * arithmetic of its reference kernels
 * (tflite/kernels/internal/optimized/4bit/fully_connected_reference.cc): symmetric per-row
 * quantization with scale max|x| / 127 (ReferenceBatchQuantizeFloats4Bit :121-180), input
 * offsets -7 * sum(q), out = (offset * sf) * fs + bias, then += (float(sum((w + 7) q)) * sf)
 * * fs (:182-272), then the fused activation. Weights are expected in [-7, 7] as the
 * reference's prepacking assumes.
 *   The filter is handed over as int8: unpack the model's nibbles with lrtfc_unpack_int4 and
 *   re-tile with lrtfc_pack_int8_filter (the reference prepacks its own layout once,
 *   fully_connected.cc:1109-1120). per_channel_scales NULL: filter_scale for every channel.
 *   workspace: lrtfc_activation_workspace_bytes(batches, depth), 256-byte aligned. */
int lrtfc_batch_quantize_floats_4bit(const float* values, int n_batch, int n_data,
                                     int8_t* quantized, float* scaling_factors,
                                     int32_t* input_offsets, void* stream);
int lrtfc_fc_hybrid_int4_per_channel_packed(const float* input, const int8_t* packed_filter,
                                            const float* per_channel_scales, float filter_scale,
                                            const float* bias, float* output, int batches,
                                            int depth, int out_depth, int activation,
                                            void* workspace, size_t workspace_bytes,
                                            void* stream);

/* The same op on a filter that stays 4 bits per weight in device memory (half the bytes to
 * stream per decode step): lrtfc_pack_int4_per_channel re-tiles the model's nibble-packed rows
 * ([out_depth, depth / 2] bytes, low nibble first; even depth) into
 * lrtfc_packed_int4_per_channel_bytes(out_depth, depth) bytes, 16-byte aligned. Meant for
 * decode batches (it makes one pass over the filter per 16 rows); prefill batches are faster on
 * the int8 copy above. Results are identical bit for bit. */
size_t lrtfc_packed_int4_per_channel_bytes(int out_depth, int depth);
int lrtfc_pack_int4_per_channel(const uint8_t* packed_filter, int out_depth, int depth,
                                uint8_t* retiled_filter, void* stream);
int lrtfc_fc_hybrid_int4_per_channel_nibbles(const float* input, const uint8_t* retiled_filter,
                                             const float* per_channel_scales, float filter_scale,
                                             const float* bias, float* output, int batches,
                                             int depth, int out_depth, int activation,
                                             void* workspace, size_t workspace_bytes,
                                             void* stream);

/* ---- Several blockwise-int4 nodes in one launch ----------------------------------------
 * Nodes of a graph that do not depend on each other (the q/k/v or the gate/up projections of
 * a decoder layer) and share depth and batch count can run as ONE kernel: the gaps between
 * launches disappear and small filters overlap large ones. The reference has no counterpart
 * (its interpreter runs nodes one after another, tflite/core/subgraph.cc:1687-1693); every
 * node computes exactly what lrtfc_fc_blockwise_int4_packed computes for it.
 *   lrtfc_int4_group_prepare: once per group (and again when a pointer or shape changes);
 *     writes a table of lrtfc_int4_group_table_bytes() into `device_table` (synchronously)
 *     and fills `launch`. count at most LRTFC_INT4_GROUP_MAX; all pointers are device
 *     pointers; bias may be NULL per node.
 *   lrtfc_fc_blockwise_int4_packed_grouped: the launch (one kernel per 4 batch rows; above
 *     depth 4096 per 2 rows, or -- when every node brought a `workspace` and there are more
 *     than 2 rows -- one launch that quantizes all rows of all nodes into the workspaces and
 *     one kernel per 4 rows on them, so that every filter is streamed once); allocates and
 *     copies nothing. */
#define LRTFC_INT4_GROUP_MAX 128
enum { LRTFC_INT4_FORM_DECODE = 0, LRTFC_INT4_FORM_GEMM_NIBBLES = 1, LRTFC_INT4_FORM_GEMM_INT8 = 2 };
typedef struct lrtfc_int4_group_node {
  const float* input;            /* [batches, depth] */
  const uint8_t* retiled_filter; /* from lrtfc_pack_int4_blockwise */
  const float* kfsum;            /* [out_depth] */
  const float* bias;             /* [out_depth] or NULL */
  float* output;                 /* [batches, out_depth] */
  int out_depth;
  void* workspace;               /* NULL, or lrtfc_activation_workspace_bytes(batches, depth)
                                    bytes of this node's own, 256-byte aligned */
  const uint8_t* nibble_filter;  /* NULL, or from lrtfc_pack_int4_blockwise_gemm_nibbles. When
                                    every node of a group brings one (and a workspace) and the
                                    group's shape is one the 4-bit-resident form is faster on
                                    (three or four rows deeper than 8192), the group runs on it;
                                    retiled_filter may then be NULL. Otherwise it is ignored and
                                    retiled_filter is required. */
} lrtfc_int4_group_node;
typedef struct lrtfc_int4_group_launch {
  int count, grid_blocks, ksplit, groups_per_wave, batches, depth;
  int split_quantize;            /* 0: rows quantized in the kernel's prologue; 1: by a launch of
                                    their own; 2: in the prologue, three or four rows of a small
                                    group as two pairs side by side in one launch */
  int form;                      /* LRTFC_INT4_FORM_DECODE or LRTFC_INT4_FORM_GEMM_NIBBLES */
} lrtfc_int4_group_launch;
size_t lrtfc_int4_group_table_bytes(void);
/* Which filter form a group of `count` nodes with these output depths runs fastest on at this
 * batch count and depth: LRTFC_INT4_FORM_DECODE (retiled_filter), or
 * LRTFC_INT4_FORM_GEMM_NIBBLES (nibble_filter and a workspace per node: three or four rows of
 * filters deeper than 8192 with at least a wavefront's worth of channels per SIMD in all).
 * lrtfc_int4_group_prepare applies the same rule to what the nodes bring. */
int lrtfc_int4_group_preferred_form(const int* out_depths, int count, int batches, int depth);
int lrtfc_int4_group_prepare(const lrtfc_int4_group_node* nodes, int count, int batches,
                             int depth, void* device_table, lrtfc_int4_group_launch* launch,
                             void* stream);
int lrtfc_fc_blockwise_int4_packed_grouped(const void* device_table,
                                           const lrtfc_int4_group_launch* launch,
                                           int quant_variant, void* stream);


/* Same product on already-quantized activations (workspace layout not needed). */
int lrtfc_fc_blockwise_int4_quantized(const int8_t* quantized_input,
                                      const float* scaling_factors, const int32_t* zero_points,
                                      const uint8_t* packed_filter, const uint16_t* scales_f16,
                                      const float* kfsum, const float* bias, float* output,
                                      int batches, int depth, int out_depth, int blocksize,
                                      void* stream);

/* ---- Blockwise-int4 FULLY_CONNECTED for prefill batches ---------------------------------
 * EvalBlockwise4Bit (tflite/kernels/fully_connected.cc:1014-1086) as a matrix-core GEMM: the
 * filter streams once for the whole batch instead of once per four rows. Same results, bit for
 * bit, as lrtfc_fc_blockwise_int4 (every output adds its blocks' `float(int32 sum) * scale` in
 * block order). Block size 32.
 *   lrtfc_gemm_int4_blockwise_bytes / lrtfc_pack_int4_blockwise_gemm: the filter re-tiled for
 *     this kernel (16 channels x one block per 512-byte tile, sign-extended to int8, then the
 *     scales as float32); made once, like the other re-tilings.
 *   lrtfc_fc_blockwise_int4_gemm_workspace_bytes: device scratch for the quantized rows in
 *     the kernel's tile order, their scaling factors and zero points (256-byte aligned).
 *   lrtfc_fc_blockwise_int4_gemm: row quantizer launch (it writes the tile order itself),
 *     GEMM launch. */
size_t lrtfc_gemm_int4_blockwise_bytes(int out_depth, int depth);
int lrtfc_pack_int4_blockwise_gemm(const uint8_t* packed_filter, const uint16_t* scales_f16,
                                   int out_depth, int depth, int blocksize, uint8_t* gemm_filter,
                                   void* stream);
size_t lrtfc_fc_blockwise_int4_gemm_workspace_bytes(int batches, int depth);
int lrtfc_fc_blockwise_int4_gemm(const float* input, const uint8_t* gemm_filter,
                                 const float* kfsum, const float* bias, float* output,
                                 int batches, int depth, int out_depth, int quant_variant,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* The same GEMM on a filter that stays 4 bits per weight in device memory, for batches between
 * decode and prefill (5 to a few dozen rows), where the filter stream bounds the kernel and the
 * int8 form above would double it: lrtfc_pack_int4_blockwise_gemm_nibbles re-tiles the model's
 * nibbles and fp16 scales into lrtfc_gemm_int4_blockwise_nibble_bytes(out_depth, depth) bytes
 * (16-byte aligned), and lrtfc_fc_blockwise_int4_gemm_nibbles takes that filter with the
 * arguments, the workspace and the results -- bit for bit -- of lrtfc_fc_blockwise_int4_gemm.
 * A wavefront expands each block's nibbles to the matrix cores' int8 operand itself. */
/* (the LRTFC_INT4_FORM_* values are declared with the grouped launch above) */
/* Which of the three forms of the blockwise-int4 op runs a shape fastest (block size 32): the
 * streaming kernel of lrtfc_fc_blockwise_int4_packed (up to four rows per pass over the filter),
 * this nibble-resident GEMM, or the int8-expanded GEMM. All three give the same bits; a caller
 * keeps the filter in the one layout its batch size asks for. Pure host function. */
int lrtfc_fc_blockwise_int4_preferred_form(int batches, int depth, int out_depth);
size_t lrtfc_gemm_int4_blockwise_nibble_bytes(int out_depth, int depth);
int lrtfc_pack_int4_blockwise_gemm_nibbles(const uint8_t* packed_filter,
                                           const uint16_t* scales_f16, int out_depth, int depth,
                                           int blocksize, uint8_t* nibble_filter, void* stream);
int lrtfc_fc_blockwise_int4_gemm_nibbles(const float* input, const uint8_t* nibble_filter,
                                         const float* kfsum, const float* bias, float* output,
                                         int batches, int depth, int out_depth,
                                         int quant_variant, void* workspace,
                                         size_t workspace_bytes, void* stream);

/* ---- EMBEDDING_LOOKUP from quantized tables (the op that feeds a decoder's first
 * FULLY_CONNECTED nodes) ------------------------------------------------------------------ */

/* Output element types of the lookups below. */
#define LRTFC_OUT_FLOAT32 0
#define LRTFC_OUT_FLOAT16 1

/* Blockwise Int4 table -> float rows. Replaces EvalBlockwise,
 * tflite/kernels/embedding_lookup.cc:194-307 with Unpack4Bit :140-159: output[i, c] =
 * float((int8)(nibble << 4)) * (scale[lookup[i], c / blocksize] / 16), converted to binary16 for
 * LRTFC_OUT_FLOAT16. table: rows x cols/2 bytes, low nibble = even column; scales_f16:
 * [rows, cols / blocksize] IEEE binary16; lookup: [count] int32; output: [count, cols].
 * cols must be a multiple of blocksize (:269-275) and both even (the reference reads rows from
 * byte boundaries). status: device int32[3] or NULL; every call rewrites it as {0, -1, 0}, or
 * {1, p, lookup[p]} when lookup[p] is the first index outside [0, rows) -- where the reference
 * fails the invoke and reports that index (:280-286); rows with such an index are left
 * unwritten. All pointers are device
 * pointers; the call only enqueues work on `stream`. */
int lrtfc_embedding_lookup_blockwise_int4(const int32_t* lookup, int count, const uint8_t* table,
                                          int rows, int cols, const uint16_t* scales_f16,
                                          int blocksize, int out_type, void* output,
                                          int32_t* status, void* stream);

/* Int8 (value_bits 8) or Int4 (4) table with one scale, or one per row when row_scales is not
 * NULL -> float rows. Replaces EvalHybrid, tflite/kernels/embedding_lookup.cc:309-395:
 * output[i, c] = float(value) * scale for Int8 and Unpack4Bit's arithmetic for Int4 (cols even).
 * status as above (:365-371). */
int lrtfc_embedding_lookup_hybrid(const int32_t* lookup, int count, const void* table,
                                  int value_bits, int rows, int cols, float scale,
                                  const float* row_scales, int out_type, void* output,
                                  int32_t* status, void* stream);

/* ---- completion mark ------------------------------------------------------------------------
 * No counterpart in the reference, whose kernels return when their work is done. Enqueues on
 * `stream` a one-wavefront kernel that stores `value` to *flag once everything enqueued on the
 * stream before it has finished and its results are visible to the host. `flag` is the device
 * address of 4 bytes of page-locked host memory (hipHostMalloc + hipHostGetDevicePointer). For
 * callers that wait for a short chain of kernels by polling that word from the CPU: on an idle
 * stream the store is seen about 3.5 us earlier than hipStreamSynchronize returns. The caller
 * bounds its polling and falls back to hipStreamSynchronize, which also reports a failed
 * kernel. */
int lrtfc_mark_completion(uint32_t* flag, uint32_t value, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LITERT_AMD_FC_H_ */

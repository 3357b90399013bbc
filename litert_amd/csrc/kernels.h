// Internal launcher interface between the C-ABI layer (capi.hip) and the kernel
// translation units. All pointers are device pointers.
#ifndef LITERT_AMD_CSRC_KERNELS_H_
#define LITERT_AMD_CSRC_KERNELS_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/litert_amd_fc.h"
#include "device_utils.h"

namespace lrtfc {

// Raises a kernel's dynamic-LDS limit when a launch needs more than the default 48 KiB. The
// attribute belongs to the (kernel, device) pair, so what has been granted is remembered per
// pair (defined in capi.hip; safe to call from several threads).
hipError_t EnsureDynamicLds(const void* kernel, size_t bytes);


// Layout of the activation workspace of lrtfc_activation_workspace_bytes(batches, depth):
// quantized rows, then scaling factors, then zero points, each region on a 256-byte boundary.
struct ActivationWorkspace {
  int8_t* q;
  float* sf;
  int32_t* zp;
};
inline size_t AlignUp256(size_t v) { return (v + 255) / 256 * 256; }
inline size_t ActivationWorkspaceBytes(int batches, int depth) {
  return AlignUp256(static_cast<size_t>(batches) * depth) +
         2 * AlignUp256(static_cast<size_t>(batches) * 4);
}
inline ActivationWorkspace SplitActivationWorkspace(void* base, int batches, int depth) {
  char* p = static_cast<char*>(base);
  ActivationWorkspace w;
  w.q = reinterpret_cast<int8_t*>(p);
  p += AlignUp256(static_cast<size_t>(batches) * depth);
  w.sf = reinterpret_cast<float*>(p);
  p += AlignUp256(static_cast<size_t>(batches) * 4);
  w.zp = reinterpret_cast<int32_t*>(p);
  return w;
}

// Arguments of the int8-weight kernels (full-integer and hybrid epilogues).
struct FcInt8Args {
  const int8_t* input;   // [batches, depth] int8 (quantized activations)
  const int8_t* filter;  // [out_depth, depth]
  int batches, depth, out_depth;
  const int32_t* filter_row_sums;  // [out_depth] or nullptr
  // full-integer epilogue
  const int32_t* bias_i32;
  const int32_t* multipliers;
  const int32_t* shifts;
  int per_channel;
  int32_t input_offset, filter_offset, output_offset, act_min, act_max;
  int8_t* output_i8;
  // hybrid epilogue
  const float* scaling_factors;     // [batches]
  const int32_t* zero_points;       // [batches] or nullptr
  const float* per_channel_scales;  // [out_depth] or nullptr
  float filter_scale;
  const float* bias_f32;
  int activation;
  float* output_f32;
  // Non-zero: EvalHybridDense semantics for a whole-zero input (output = activation(bias), no
  // product added; fully_connected.cc:789-795). Zero: MatrixBatchVectorMultiplyAccumulate as is.
  int zero_input_exit;
  // Non-zero: the arithmetic of the hybrid BATCH_MATMUL kernel (reference/batch_matmul.h:
  // 190-206) instead of MatrixBatchVectorMultiplyAccumulate's; no bias, no activation.
  int batch_matmul;
};

// kHybrid4Bit: the float epilogue of the per-channel int4 hybrid path; a.zero_points then
// holds the rows' input offsets (-7 * sum(q)) and a.filter_row_sums is unused.
enum class Int8Epilogue { kRequantize, kHybrid, kHybrid4Bit };

hipError_t LaunchBatchQuantize(const float* values, int n_batch, int n_data, int8_t* quantized,
                               float* scaling_factors, int32_t* zero_points, int do_asymmetric,
                               int variant, hipStream_t stream);

hipError_t LaunchBatchQuantize4Bit(const float* values, int n_batch, int n_data, int8_t* quantized,
                                   float* scaling_factors, int32_t* input_offsets,
                                   hipStream_t stream);
// `matrices` row-major [in_rows, in_cols] float32 matrices -> [in_cols, in_rows] each.
hipError_t LaunchTransposeLastTwoF32(const float* src, int matrices, int in_rows, int in_cols,
                                     float* dst, hipStream_t stream);
hipError_t LaunchZeroFill(void* dst, size_t bytes, hipStream_t stream);
hipError_t LaunchRowSumsInt8(const int8_t* filter, int out_depth, int depth, int32_t* row_sums,
                             hipStream_t stream);
hipError_t LaunchUnpackInt4(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                            hipStream_t stream);
hipError_t LaunchUnpackInt2(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                            hipStream_t stream);
// dst[i] = src[i] ^ 0x80 (uint8 value - 128 as int8, and back); src == dst allowed.
hipError_t LaunchXorSignBit(const uint8_t* src, uint8_t* dst, size_t bytes, hipStream_t stream);

// Small-batch path: bandwidth-bound GEMV (any shape; fast path needs depth % 16 == 0).
hipError_t LaunchFcInt8Gemv(const FcInt8Args& a, Int8Epilogue epilogue, hipStream_t stream);
// Large-batch full-integer path: int8 MFMA GEMM. Returns hipErrorNotSupported when
// the shape does not meet its tiling constraints (caller falls back to the GEMV).
hipError_t LaunchFcInt8GemmMfma(const FcInt8Args& a, hipStream_t stream);
bool FcInt8GemmMfmaSupports(const FcInt8Args& a);

// Matrix-core GEMV on a filter re-tiled by LaunchPackInt8Filter (a.filter = packed).
// input_f32 != nullptr selects the fused form that quantizes the float rows in-kernel.
size_t PackedInt8FilterBytes(int out_depth, int depth);
hipError_t LaunchPackInt8Filter(const int8_t* filter, int out_depth, int depth, int8_t* packed,
                                hipStream_t stream);
bool FcInt8PackedGemvSupports(const FcInt8Args& a);
// Rows up to which the fused (quantize-in-kernel) form beats quantizer launch + product.
int FcInt8PackedGemvFusedMaxRows(int depth);
hipError_t LaunchFcInt8PackedGemv(const FcInt8Args& a, Int8Epilogue epilogue,
                                  const float* input_f32, int asymmetric, int variant,
                                  hipStream_t stream);

// Per-channel int4 hybrid GEMV on the filter kept at 4 bits per weight (tile16x128n, made by
// LaunchPackInt4PerChannel from the model's nibble-packed rows); rows quantized by
// LaunchBatchQuantize4Bit. Any batch count (tiles of 16 rows), any out_depth, even depth.
size_t PackedInt4PerChannelBytes(int out_depth, int depth);
hipError_t LaunchPackInt4PerChannel(const uint8_t* filter, int out_depth, int depth,
                                    uint8_t* packed, hipStream_t stream);
bool FcInt4PerChannelGemvSupports(int depth);
// input_f32 != nullptr: the fused form (row quantizer in the prologue; only where
// FcInt4PerChannelGemvFuses says so), quantized_input / scaling_factors / input_offsets unused.
bool FcInt4PerChannelGemvFuses(const float* input_f32, int batches, int depth);
hipError_t LaunchFcInt4PerChannelGemv(const uint8_t* packed, const float* input_f32,
                                      const int8_t* quantized_input,
                                      const float* scaling_factors, const int32_t* input_offsets,
                                      const float* per_channel_scales, float filter_scale,
                                      const float* bias, float* output, int batches, int depth,
                                      int out_depth, int activation, hipStream_t stream);

// Prefill batches on the same re-tiled filter: int8 MFMA GEMM (a.filter = packed, a.input =
// int8 rows; the hybrid epilogue reads a.scaling_factors / a.zero_points). Any batch count,
// any out_depth; depth a multiple of 16.
// Whether the GEMV streams the filter once for all of a.batches rows (up to 16 always; 17 to 32
// rows that arrive quantized when their LDS image fits a compute unit).
bool FcInt8PackedGemvTakesRowsInOnePass(const FcInt8Args& a);
// 33 to 128 quantized rows on wide re-tiled filters: the filter streamed once, the rows through
// LDS in depth chunks (fc_int8_rows_gemv.hip). FcInt8RowsGemvTakes: the shapes it is meant for.
bool FcInt8RowsGemvTakes(const FcInt8Args& a);
hipError_t LaunchFcInt8RowsGemv(const FcInt8Args& a, Int8Epilogue epilogue, hipStream_t stream);
bool FcInt8PackedGemmSupports(const FcInt8Args& a);
hipError_t LaunchFcInt8PackedGemm(const FcInt8Args& a, Int8Epilogue epilogue, hipStream_t stream);

struct FcInt4Args {
  const int8_t* input;           // [batches, depth] quantized activations
  const float* scaling_factors;  // [batches]
  const int32_t* zero_points;    // [batches]
  const uint8_t* packed_filter;  // [out_depth, depth / 2]
  const uint16_t* scales_f16;    // [out_depth, depth / blocksize]
  const float* kfsum;            // [out_depth]
  const float* bias;
  float* output;
  int batches, depth, out_depth, blocksize;
};

hipError_t LaunchBlockwiseInt4Kfsum(const uint8_t* packed_filter, const uint16_t* scales_f16,
                                    int out_depth, int depth, int blocksize, float* kfsum,
                                    hipStream_t stream);
hipError_t LaunchFcBlockwiseInt4(const FcInt4Args& a, hipStream_t stream);

// Streaming kernel on a filter re-tiled by LaunchPackInt4Blockwise (block size 32).
// input_f32 != nullptr quantizes the rows in-kernel; otherwise q.input/scaling_factors/
// zero_points are used.
size_t PackedInt4BlockwiseBytes(int out_depth, int depth);
hipError_t LaunchPackInt4Blockwise(const uint8_t* filter, const uint16_t* scales, int out_depth,
                                   int depth, uint8_t* packed, hipStream_t stream);
bool FcInt4PackedSupports(int depth, int blocksize);
// Grouped launch: several filters of one depth, one kernel (see lrtfc_int4_group_prepare).
size_t Int4GroupTableBytes();
hipError_t PrepareInt4Group(const lrtfc_int4_group_node* nodes, int count, int batches, int depth,
                            void* device_table, lrtfc_int4_group_launch* launch,
                            hipStream_t stream);
hipError_t LaunchFcInt4PackedGrouped(const void* table, const lrtfc_int4_group_launch& launch,
                                     int variant, hipStream_t stream);
// The grouped launch on the 4-bit-resident filters (one to four rows; every node brings its
// nibble filter and a workspace). Int4NibbleGroupWins: the shapes for which PrepareInt4Group
// chooses it when it can.
size_t Int4NibbleGroupTableBytes();
bool Int4NibbleGroupWins(int batches, int depth, int total_channel_tiles);
hipError_t PrepareInt4NibbleGroup(const lrtfc_int4_group_node* nodes, int count, int batches,
                                  int depth, void* device_table, lrtfc_int4_group_launch* launch,
                                  hipStream_t stream);
hipError_t LaunchFcInt4NibbleGrouped(const void* table, const lrtfc_int4_group_launch& launch,
                                     int variant, hipStream_t stream);
hipError_t LaunchFcInt4Packed(const FcInt4Args& q, const uint8_t* packed, const float* input_f32,
                              int variant, hipStream_t stream);

// Blockwise-int4 FULLY_CONNECTED for prefill batches: matrix-core GEMM with one float32
// accumulator per output walking the blocks in order (block size 32). The filter is re-tiled by
// LaunchPackInt4BlockwiseGemm (GemmInt4BlockwiseBytes bytes: int8 tiles, then float32 scales);
// the float rows are quantized (BatchQuantizeFloats, asymmetric, `variant`) straight into
// `tiled_rows` (TiledRowsBytes bytes), their scaling factors and zero points into the two
// arrays of `batches` entries, by a launch ahead of the GEMM's.
size_t GemmInt4BlockwiseBytes(int out_depth, int depth);
bool FcInt4BlockwiseGemmSupports(int depth, int blocksize);
hipError_t LaunchPackInt4BlockwiseGemm(const uint8_t* filter, const uint16_t* scales_f16,
                                       int out_depth, int depth, uint8_t* packed,
                                       hipStream_t stream);
size_t TiledRowsBytes(int batches, int depth);
hipError_t LaunchFcInt4BlockwiseGemm(const float* input, int variant, float* scaling_factors,
                                     int32_t* zero_points, const uint8_t* gemm_filter,
                                     const float* kfsum, const float* bias, float* output,
                                     int batches, int depth, int out_depth, void* tiled_rows,
                                     hipStream_t stream);

// The same product on a filter kept at 4 bits per weight (`tile16x128n` + fp16 scales), for
// batches between decode and prefill.
size_t GemmInt4BlockwiseNibbleBytes(int out_depth, int depth);
hipError_t LaunchPackInt4BlockwiseNibbles(const uint8_t* filter, const uint16_t* scales_f16,
                                          int out_depth, int depth, uint8_t* packed,
                                          hipStream_t stream);
hipError_t LaunchFcInt4BlockwiseNibbleGemm(const float* input, int variant,
                                           float* scaling_factors, int32_t* zero_points,
                                           const uint8_t* nibble_filter, const float* kfsum,
                                           const float* bias, float* output, int batches,
                                           int depth, int out_depth, void* tiled_rows,
                                           hipStream_t stream);

// EMBEDDING_LOOKUP from an Int4 (value_bits 4) or Int8 (8) table to float32 / binary16 rows.
// block_scales != nullptr: blockwise fp16 scales [rows, cols / blocksize]; otherwise row_scales
// [rows] or `scale`. status: three device int32 {0 or 1, first offending position or -1, the
// index there or 0}, rewritten by every launch; may be nullptr. Int4 tables need even cols and blocksize.
hipError_t LaunchEmbeddingLookup(const int32_t* lookup, int count, const void* table,
                                 int value_bits, int rows, int cols, const uint16_t* block_scales,
                                 int blocksize, const float* row_scales, float scale, int out_f16,
                                 void* output, int32_t* status, hipStream_t stream);

}  // namespace lrtfc

#endif  // LITERT_AMD_CSRC_KERNELS_H_

// extern "C" doorway to the few reference translation units that compile from
// their own sources with g++ alone. TEST INFRASTRUCTURE ONLY. Built only when
// the reference tree is present; see oracle/Makefile (target `ref`). The
// reference sources are compiled where they lie; nothing is copied.
//
// Covered: tflite/kernels/internal/quantization_util.cc (QuantizeMultiplier),
// tflite/kernels/internal/portable_tensor_utils.cc (UnpackPackedIntToInt8,
// ApplyRelu*ToVector), tflite/kernels/internal/optimized/4bit/fully_connected_reference.cc
// (the reference kernels of the per-channel int4 hybrid path). Every other file on the path
// needs gemmlowp, ruy, Eigen or generated flatbuffer headers and is treated as unbuildable.
#include <cstdint>
#include <vector>

#include "tflite/kernels/internal/optimized/4bit/fully_connected_reference.h"
#include "tflite/kernels/internal/portable_tensor_utils.h"
#include "tflite/kernels/internal/quantization_util.h"

extern "C" {

void ref_quantize_multiplier(double m, int32_t* quantized_multiplier, int* shift) {
  tflite::QuantizeMultiplier(m, quantized_multiplier, shift);
}

void ref_unpack_int4(const int8_t* src, int num_elements, int8_t* dst) {
  tflite::tensor_utils::UnpackPackedIntToInt8(src, num_elements, /*bit_width=*/4, dst,
                                              /*unpack_unsigned=*/false);
}

void ref_unpack_int2(const int8_t* src, int num_elements, int8_t* dst) {
  tflite::tensor_utils::UnpackPackedIntToInt8(src, num_elements, /*bit_width=*/2, dst,
                                              /*unpack_unsigned=*/false);
}

void ref_apply_relu(const float* in, int n, float* out) {
  tflite::tensor_utils::ApplyReluToVector(in, n, out);
}
void ref_apply_relu1(const float* in, int n, float* out) {
  tflite::tensor_utils::ApplyRelu1ToVector(in, n, out);
}
void ref_apply_relu6(const float* in, int n, float* out) {
  tflite::tensor_utils::ApplyRelu6ToVector(in, n, out);
}

// The call sequence of EvalHybridDense4Bit (tflite/kernels/fully_connected.cc:1088-1178) on the
// reference kernels, without the fused activation: prepack, quantize the rows, assign bias and
// offsets, run the kernel and unpack. rhs width is 1 (GetMaxSupportedRows() of the reference).
void ref_fc_hybrid_int4(const float* input, int batch_size, int cols, const int8_t* packed_filter,
                        int output_depth, const float* filter_scales_in, const float* bias,
                        float* output) {
  namespace o4 = tflite::optimized_4bit;
  const int lhs_width = 4, depth = 32, rhs_width = 1;
  const int lhs_layout_rows = (output_depth + (lhs_width - 1)) & ~(lhs_width - 1);
  const int lhs_layout_cols = (cols + (depth - 1)) & ~(depth - 1);
  const int rhs_layout_rows = (batch_size + (rhs_width - 1)) & ~(rhs_width - 1);
  const int rhs_layout_cols = lhs_layout_cols;
  const int dst_layout_rows = rhs_layout_rows;
  const int dst_layout_cols = lhs_layout_rows;
  std::vector<uint8_t> prepacked(static_cast<size_t>(lhs_layout_rows) * lhs_layout_cols / 2);
  o4::Prepack(prepacked.data(), packed_filter, lhs_layout_rows, lhs_layout_cols, output_depth,
              cols, lhs_width, depth);
  std::vector<float> filter_scales(lhs_layout_rows, 0.0f);
  for (int i = 0; i < output_depth; ++i) filter_scales[i] = filter_scales_in[i];
  std::vector<int8_t> quant(static_cast<size_t>(rhs_layout_rows) * rhs_layout_cols);
  std::vector<float> scaling_factors(rhs_layout_rows, 0.0f);
  std::vector<int32_t> input_offsets(rhs_layout_rows, 0);
  o4::BatchQuantizeFloats4Bit(input, batch_size, cols, quant.data(), scaling_factors.data(),
                              rhs_width, depth, input_offsets.data());
  o4::AssignBiasAndComputeOffsets(input_offsets.data(), scaling_factors.data(),
                                  filter_scales.data(), bias, output, output_depth, batch_size);
  std::vector<int32_t> dst(static_cast<size_t>(dst_layout_rows) * dst_layout_cols);
  o4::RunAndUnpack(rhs_width, prepacked.data(), quant.data(), dst.data(), output_depth,
                   batch_size, lhs_layout_rows, lhs_layout_cols, rhs_layout_rows,
                   rhs_layout_cols, dst_layout_rows, dst_layout_cols, output,
                   scaling_factors.data(), filter_scales.data());
}

}  // extern "C"

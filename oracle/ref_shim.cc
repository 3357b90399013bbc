// extern "C" doorway to the few reference translation units that compile from
// their own sources with g++ alone. TEST INFRASTRUCTURE ONLY. Built only when
// the reference tree is present; see oracle/Makefile (target `ref`). The
// reference sources are compiled where they lie; nothing is copied.
//
// Covered: tflite/kernels/internal/quantization_util.cc (QuantizeMultiplier),
// tflite/kernels/internal/portable_tensor_utils.cc (UnpackPackedIntToInt8,
// ApplyRelu*ToVector). Every other file on the path needs gemmlowp, ruy, Eigen
// or generated flatbuffer headers and is treated as unbuildable.
#include <cstdint>

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

void ref_apply_relu(const float* in, int n, float* out) {
  tflite::tensor_utils::ApplyReluToVector(in, n, out);
}
void ref_apply_relu1(const float* in, int n, float* out) {
  tflite::tensor_utils::ApplyRelu1ToVector(in, n, out);
}
void ref_apply_relu6(const float* in, int n, float* out) {
  tflite::tensor_utils::ApplyRelu6ToVector(in, n, out);
}

}  // extern "C"

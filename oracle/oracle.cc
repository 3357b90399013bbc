// CPU oracle for the quantized FULLY_CONNECTED path. TEST INFRASTRUCTURE ONLY:
// see oracle.h. Compile with -ffp-contract=off and without fast-math.
#include "oracle.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <vector>

namespace {

// ---- fixed-point helpers --------------------------------------------------

// gemmlowp SaturatingRoundingDoublingHighMul (fixedpoint.h @16e8662c): the
// high 32 bits of 2*a*b, rounded to nearest through a sign-dependent nudge and a
// truncating 64-bit division (exact halves end up rounded toward +infinity).
inline int32_t Srdhm(int32_t a, int32_t b) {
  if (a == b && a == std::numeric_limits<int32_t>::min()) {
    return std::numeric_limits<int32_t>::max();
  }
  const int64_t ab = static_cast<int64_t>(a) * static_cast<int64_t>(b);
  const int64_t nudge = ab >= 0 ? (1ll << 30) : (1 - (1ll << 30));
  return static_cast<int32_t>((ab + nudge) / (1ll << 31));
}

// gemmlowp RoundingDivideByPOT: arithmetic shift right with round-to-nearest,
// ties away from zero.
inline int32_t RoundingDivideByPot(int32_t x, int exponent) {
  const int32_t mask = static_cast<int32_t>((1ll << exponent) - 1);
  const int32_t remainder = x & mask;
  const int32_t threshold = (mask >> 1) + (x < 0 ? 1 : 0);
  return (x >> exponent) + (remainder > threshold ? 1 : 0);
}

// common.cc:80-90. `x * (1 << left_shift)` wraps in the reference build (the
// function is marked no-sanitize-integer-overflow); reproduce with unsigned.
inline int32_t Mbqm(int32_t x, int32_t quantized_multiplier, int shift) {
  const int left_shift = shift > 0 ? shift : 0;
  const int right_shift = shift > 0 ? 0 : -shift;
  const int32_t shifted = static_cast<int32_t>(static_cast<uint32_t>(x) << left_shift);
  return RoundingDivideByPot(Srdhm(shifted, quantized_multiplier), right_shift);
}

// common.cc:33-47.
inline int32_t MbqmSingleRounding(int32_t x, int32_t quantized_multiplier, int shift) {
  const int64_t total_shift = 31 - shift;
  const int64_t round = static_cast<int64_t>(1) << (total_shift - 1);
  int64_t result = x * static_cast<int64_t>(quantized_multiplier) + round;
  result = result >> total_shift;
  return static_cast<int32_t>(result);
}

inline int32_t ClampI32(int32_t v, int32_t lo, int32_t hi) {
  v = std::max(v, lo);
  v = std::min(v, hi);
  return v;
}

// kernel_util.cc:343-352: float division, round half away, then add.
inline bool QuantizeForRange(float scale, int32_t zero_point, float f, int32_t* q) {
  const float tmp = std::round(f / scale);
  const bool fits = tmp >= static_cast<float>(std::numeric_limits<int32_t>::min()) &&
                    tmp <= static_cast<float>(std::numeric_limits<int32_t>::max());
  if (!fits) return false;
  *q = zero_point + static_cast<int32_t>(tmp);
  return true;
}

// ---- activation quantization ---------------------------------------------

// neon_tensor_utils.cc:2347-2359.
inline int32_t RoundToNearestVariant(float x, int variant) {
  if (variant == ORC_QUANT_NEON_LEGACY) {
    const float nudge = (x < 0.0f ? -1.0f : 0.0f) + 0.5f;
    return static_cast<int32_t>(x + nudge);  // float add, then truncation
  }
  return static_cast<int32_t>(std::round(x));  // vcvta: nearest, ties away
}

// neon_tensor_utils.cc:2363-2399: min/max capped at zero; NaN handling aside,
// the value equals min(0, min v) / max(0, max v).
inline void MinMaxCappedAtZero(const float* values, int size, float* mn, float* mx) {
  float rmin = 0.0f, rmax = 0.0f;
  for (int i = 0; i < size; ++i) {
    rmin = std::min(rmin, values[i]);
    rmax = std::max(rmax, values[i]);
  }
  *mn = rmin;
  *mx = rmax;
}

void AsymmetricQuantize(const float* values, int size, int8_t* quantized, float* scaling_factor,
                        int32_t* offset, int variant) {
  const double qmin = -128.0, qmax = 127.0;
  double rmin, rmax, scale;
  if (variant == ORC_QUANT_PORTABLE) {
    // reference/portable_tensor_utils.cc:74-84: the range is widened to
    // double before the subtraction.
    const auto mm = std::minmax_element(values, values + size);
    rmin = static_cast<double>(std::min(0.0f, *mm.first));
    rmax = static_cast<double>(std::max(0.0f, *mm.second));
    if (rmin == rmax) {
      std::memset(quantized, 0, size);
      *scaling_factor = 1;
      *offset = 0;
      return;
    }
    scale = (rmax - rmin) / (qmax - qmin);
  } else {
    // neon_tensor_utils.cc:2470-2486: rmin/rmax stay float, so the range
    // subtraction is a float operation.
    float fmin, fmax;
    MinMaxCappedAtZero(values, size, &fmin, &fmax);
    if (fmin == fmax) {
      std::memset(quantized, 0, size);
      *scaling_factor = 1;
      *offset = 0;
      return;
    }
    scale = (fmax - fmin) / (qmax - qmin);
    rmin = fmin;
    rmax = fmax;
  }
  const double zp_from_min = qmin - rmin / scale;
  const double zp_from_max = qmax - rmax / scale;
  const double err_from_min = std::abs(qmin) + std::abs(rmin / scale);
  const double err_from_max = std::abs(qmax) + std::abs(rmax / scale);
  const double zp_double = err_from_min < err_from_max ? zp_from_min : zp_from_max;
  int8_t nudged;
  if (zp_double <= qmin) {
    nudged = -128;
  } else if (zp_double >= qmax) {
    nudged = 127;
  } else {
    nudged = static_cast<int8_t>(std::round(zp_double));
  }
  *scaling_factor = static_cast<float>(scale);
  *offset = nudged;

  if (variant == ORC_QUANT_PORTABLE) {
    // reference/portable_tensor_utils.cc:112-118.
    const float inv = 1.0f / *scaling_factor;
    for (int i = 0; i < size; ++i) {
      const float scaled = values[i] * inv;
      const float shifted = static_cast<float>(*offset) + scaled;
      const int32_t q = static_cast<int32_t>(std::round(shifted));
      quantized[i] = static_cast<int8_t>(std::min(127, std::max(-128, q)));
    }
    return;
  }
  // neon_tensor_utils.cc:2509-2551: inverse through double, round first, add
  // the zero point as an integer. The scalar tail (size % 8 elements) rounds
  // with std::round whichever build it is.
  const float inv = *scaling_factor == 0 ? 0.0f
                                         : static_cast<float>(1.0 / static_cast<double>(*scaling_factor));
  const int vector_end = size - (size % 8);
  for (int i = 0; i < size; ++i) {
    const float scaled = values[i] * inv;
    int32_t q;
    if (i < vector_end) {
      q = RoundToNearestVariant(scaled, variant) + *offset;
    } else {
      q = static_cast<int32_t>(static_cast<float>(*offset) + std::round(inv * values[i]));
    }
    quantized[i] = static_cast<int8_t>(std::min(127, std::max(-128, q)));
  }
}

void SymmetricQuantize(const float* values, int size, int8_t* quantized, float* scaling_factor,
                       int variant) {
  // reference/portable_tensor_utils.cc:41-71; neon_tensor_utils.cc:2401-2468.
  const auto mm = std::minmax_element(values, values + size);
  const float range = std::max(std::abs(*mm.first), std::abs(*mm.second));
  if (range == 0) {
    std::memset(quantized, 0, size);
    *scaling_factor = 1;
    return;
  }
  *scaling_factor = range / 127;
  const float inv = 127 / range;
  const int vector_end = (variant == ORC_QUANT_PORTABLE) ? 0 : size - (size % 8);
  for (int i = 0; i < size; ++i) {
    int32_t q;
    if (i < vector_end) {
      q = RoundToNearestVariant(values[i] * inv, variant);
    } else {
      q = static_cast<int32_t>(std::round(values[i] * inv));
    }
    quantized[i] = static_cast<int8_t>(std::min(127, std::max(-127, q)));
  }
}

}  // namespace

extern "C" {

void orc_quantize_multiplier(double real_multiplier, int32_t* quantized_multiplier, int* shift) {
  if (real_multiplier == 0.) {
    *quantized_multiplier = 0;
    *shift = 0;
    return;
  }
  const double q = std::frexp(real_multiplier, shift);
  int64_t q_fixed = static_cast<int64_t>(std::round(q * static_cast<double>(1ll << 31)));
  if (q_fixed == (1ll << 31)) {
    q_fixed /= 2;
    ++*shift;
  }
  if (*shift < -31) {
    *shift = 0;
    q_fixed = 0;
  }
  *quantized_multiplier = static_cast<int32_t>(q_fixed);
}

int32_t orc_srdhm(int32_t a, int32_t b) { return Srdhm(a, b); }
int32_t orc_rounding_divide_by_pot(int32_t x, int exponent) { return RoundingDivideByPot(x, exponent); }
int32_t orc_mbqm(int32_t x, int32_t m, int shift) { return Mbqm(x, m, shift); }
int32_t orc_mbqm_single_rounding(int32_t x, int32_t m, int shift) {
  return MbqmSingleRounding(x, m, shift);
}

int orc_activation_range_int8(int activation, float out_scale, int32_t out_zero_point,
                              int32_t* act_min, int32_t* act_max) {
  const int32_t qmin = -128, qmax = 127;
  int32_t q;
  if (activation == ORC_ACT_RELU) {
    if (!QuantizeForRange(out_scale, out_zero_point, 0.0f, &q)) return 1;
    *act_min = std::max(qmin, q);
    *act_max = qmax;
  } else if (activation == ORC_ACT_RELU6) {
    if (!QuantizeForRange(out_scale, out_zero_point, 0.0f, &q)) return 1;
    *act_min = std::max(qmin, q);
    if (!QuantizeForRange(out_scale, out_zero_point, 6.0f, &q)) return 1;
    *act_max = std::min(qmax, q);
  } else if (activation == ORC_ACT_RELU_N1_TO_1) {
    if (!QuantizeForRange(out_scale, out_zero_point, -1.0f, &q)) return 1;
    *act_min = std::max(qmin, q);
    if (!QuantizeForRange(out_scale, out_zero_point, 1.0f, &q)) return 1;
    *act_max = std::min(qmax, q);
  } else {
    *act_min = qmin;
    *act_max = qmax;
  }
  return 0;
}

float orc_half_to_float(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      // subnormal half: normalise into a float exponent
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      bits = sign | static_cast<uint32_t>(127 - 15 - e) << 23 | (man & 0x3FFu) << 13;
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | man << 13;
  } else {
    bits = sign | (exp + (127 - 15)) << 23 | man << 13;
  }
  float f;
  std::memcpy(&f, &bits, sizeof f);
  return f;
}

void orc_unpack_int4(const int8_t* src, int num_elements, int8_t* dst) {
  // The reference shifts the signed byte left (`byte << 4`, undefined for negative values before
  // C++20, though every compiler it is built with gives the two's-complement result); the same
  // value is formed here from the unsigned byte.
  auto low = [](int8_t byte) {
    return static_cast<int8_t>(static_cast<int8_t>(static_cast<uint8_t>(byte) << 4) >> 4);
  };
  for (int i = 0; i < num_elements / 2; ++i) {
    const int8_t byte = src[i];
    dst[2 * i] = low(byte);
    dst[2 * i + 1] = static_cast<int8_t>(byte >> 4);
  }
  if (num_elements % 2 != 0) dst[num_elements - 1] = low(src[num_elements / 2]);
}

void orc_unpack_int2(const int8_t* src, int num_elements, int8_t* dst) {
  // Field k of a byte (bits 2k, 2k + 1) is moved to the top of the byte and shifted back down
  // arithmetically, as the reference does; formed from the unsigned byte for the reason given
  // in orc_unpack_int4.
  auto field = [](int8_t byte, int k) {
    return static_cast<int8_t>(
        static_cast<int8_t>((static_cast<uint8_t>(byte) << (6 - 2 * k)) & 0xFF) >> 6);
  };
  for (int i = 0; i < num_elements / 4; ++i) {
    for (int k = 0; k < 4; ++k) dst[4 * i + k] = field(src[i], k);
  }
  const int remaining = num_elements % 4;
  for (int k = 0; k < remaining; ++k) {
    dst[num_elements - remaining + k] = field(src[num_elements / 4], k);
  }
}

int orc_fc_prepare_per_channel(float input_scale, const float* filter_scales, int num_channels,
                               float output_scale, int32_t* multipliers, int32_t* shifts) {
  for (int i = 0; i < num_channels; ++i) {
    const double filter_scale = static_cast<double>(filter_scales[i]);
    const double effective = static_cast<double>(input_scale) * filter_scale /
                             static_cast<double>(output_scale);
    int shift;
    orc_quantize_multiplier(effective, &multipliers[i], &shift);
    shifts[i] = shift;
  }
  return 0;
}

int orc_fc_prepare_per_tensor(float input_scale, float filter_scale, int has_bias,
                              float bias_scale, float output_scale, int32_t* multiplier,
                              int32_t* shift) {
  if (has_bias) {
    // kernel_util.cc:296-322: product formed in double for the check.
    const double product = static_cast<double>(input_scale) * static_cast<double>(filter_scale);
    const double diff = std::abs(product - static_cast<double>(bias_scale));
    if (!(diff / static_cast<double>(output_scale) <= 0.02)) return 1;
  }
  // kernel_util.cc:333-338: product formed in float, then widened.
  const double product = static_cast<double>(input_scale * filter_scale);
  if (!(product >= 0)) return 1;
  const double real_multiplier = product / static_cast<double>(output_scale);
  int s;
  orc_quantize_multiplier(real_multiplier, multiplier, &s);
  *shift = s;
  return 0;
}

void orc_fc_int8_per_channel(const int8_t* input, const int8_t* filter, const int32_t* bias,
                             const int32_t* multipliers, const int32_t* shifts, int8_t* output,
                             int batches, int depth, int out_depth, int32_t input_offset,
                             int32_t output_offset, int32_t act_min, int32_t act_max) {
  for (int b = 0; b < batches; ++b) {
    for (int c = 0; c < out_depth; ++c) {
      int32_t acc = 0;
      for (int d = 0; d < depth; ++d) {
        acc += static_cast<int32_t>(filter[c * depth + d]) *
               (static_cast<int32_t>(input[b * depth + d]) + input_offset);
      }
      if (bias) acc += bias[c];
      int32_t v = Mbqm(acc, multipliers[c], shifts[c]) + output_offset;
      output[c + out_depth * b] = static_cast<int8_t>(ClampI32(v, act_min, act_max));
    }
  }
}

void orc_fc_int8_per_channel_single_rounding(const int8_t* input, const int8_t* filter,
                                             const int32_t* bias, const int32_t* multipliers,
                                             const int32_t* shifts, int8_t* output, int batches,
                                             int depth, int out_depth, int32_t input_offset,
                                             int32_t output_offset, int32_t act_min,
                                             int32_t act_max) {
  for (int b = 0; b < batches; ++b) {
    for (int c = 0; c < out_depth; ++c) {
      int32_t acc = 0;
      for (int d = 0; d < depth; ++d) {
        acc += static_cast<int32_t>(filter[c * depth + d]) *
               (static_cast<int32_t>(input[b * depth + d]) + input_offset);
      }
      if (bias) acc += bias[c];
      int32_t v = MbqmSingleRounding(acc, multipliers[c], shifts[c]) + output_offset;
      output[c + out_depth * b] = static_cast<int8_t>(ClampI32(v, act_min, act_max));
    }
  }
}

void orc_fc_int8_per_channel_float_scale(const int8_t* input, const int8_t* filter,
                                         const int32_t* bias, const float* filter_scales,
                                         float input_scale, float output_scale, int8_t* output,
                                         int batches, int depth, int out_depth,
                                         int32_t input_offset, int32_t output_offset,
                                         int32_t act_min, int32_t act_max) {
  for (int b = 0; b < batches; ++b) {
    for (int c = 0; c < out_depth; ++c) {
      int32_t acc = 0;
      for (int d = 0; d < depth; ++d) {
        acc += static_cast<int32_t>(filter[c * depth + d]) *
               (static_cast<int32_t>(input[b * depth + d]) + input_offset);
      }
      if (bias) acc += bias[c];
      const double effective = static_cast<double>(input_scale) *
                               static_cast<double>(filter_scales[c]) /
                               static_cast<double>(output_scale);
      int32_t v = static_cast<int32_t>(std::round(static_cast<double>(acc) * effective));
      v += output_offset;
      output[c + out_depth * b] = static_cast<int8_t>(ClampI32(v, act_min, act_max));
    }
  }
}

void orc_fc_int8_per_tensor(const int8_t* input, const int8_t* filter, const int32_t* bias,
                            int32_t multiplier, int shift, int8_t* output, int batches, int depth,
                            int out_depth, int32_t input_offset, int32_t filter_offset,
                            int32_t output_offset, int32_t act_min, int32_t act_max) {
  for (int b = 0; b < batches; ++b) {
    for (int c = 0; c < out_depth; ++c) {
      int32_t acc = 0;
      for (int d = 0; d < depth; ++d) {
        acc += (static_cast<int32_t>(filter[c * depth + d]) + filter_offset) *
               (static_cast<int32_t>(input[b * depth + d]) + input_offset);
      }
      if (bias) acc += bias[c];
      int32_t v = Mbqm(acc, multiplier, shift) + output_offset;
      output[c + out_depth * b] = static_cast<int8_t>(ClampI32(v, act_min, act_max));
    }
  }
}

void orc_fc_uint8_per_tensor(const uint8_t* input, const uint8_t* filter, const int32_t* bias,
                             int32_t multiplier, int shift, uint8_t* output, int batches, int depth,
                             int out_depth, int32_t input_offset, int32_t filter_offset,
                             int32_t output_offset, int32_t act_min, int32_t act_max) {
  for (int b = 0; b < batches; ++b) {
    for (int c = 0; c < out_depth; ++c) {
      int32_t acc = 0;
      for (int d = 0; d < depth; ++d) {
        const int32_t input_val = input[b * depth + d];
        const int32_t filter_val = filter[c * depth + d];
        acc += (filter_val + filter_offset) * (input_val + input_offset);
      }
      if (bias) acc += bias[c];
      acc = Mbqm(acc, multiplier, shift);
      acc += output_offset;
      acc = std::max(acc, act_min);
      acc = std::min(acc, act_max);
      output[c + out_depth * b] = static_cast<uint8_t>(acc);
    }
  }
}

int orc_activation_range_uint8(int activation, float out_scale, int32_t out_zero_point,
                               int32_t* act_min, int32_t* act_max) {
  const int32_t qmin = 0, qmax = 255;
  int32_t q;
  if (activation == ORC_ACT_RELU) {
    if (!QuantizeForRange(out_scale, out_zero_point, 0.0f, &q)) return 1;
    *act_min = std::max(qmin, q);
    *act_max = qmax;
  } else if (activation == ORC_ACT_RELU6) {
    if (!QuantizeForRange(out_scale, out_zero_point, 0.0f, &q)) return 1;
    *act_min = std::max(qmin, q);
    if (!QuantizeForRange(out_scale, out_zero_point, 6.0f, &q)) return 1;
    *act_max = std::min(qmax, q);
  } else if (activation == ORC_ACT_RELU_N1_TO_1) {
    if (!QuantizeForRange(out_scale, out_zero_point, -1.0f, &q)) return 1;
    *act_min = std::max(qmin, q);
    if (!QuantizeForRange(out_scale, out_zero_point, 1.0f, &q)) return 1;
    *act_max = std::min(qmax, q);
  } else {
    *act_min = qmin;
    *act_max = qmax;
  }
  return 0;
}

void orc_fc_int8_per_tensor_float_scale(const int8_t* input, const int8_t* filter,
                                        const int32_t* bias, float input_scale,
                                        float filter_scale, float output_scale, int8_t* output,
                                        int batches, int depth, int out_depth,
                                        int32_t input_offset, int32_t filter_offset,
                                        int32_t output_offset, int32_t act_min, int32_t act_max) {
  const double effective = static_cast<double>(input_scale) * static_cast<double>(filter_scale) /
                           static_cast<double>(output_scale);
  for (int b = 0; b < batches; ++b) {
    for (int c = 0; c < out_depth; ++c) {
      int32_t acc = 0;
      for (int d = 0; d < depth; ++d) {
        acc += (static_cast<int32_t>(filter[c * depth + d]) + filter_offset) *
               (static_cast<int32_t>(input[b * depth + d]) + input_offset);
      }
      if (bias) acc += bias[c];
      int32_t v = static_cast<int32_t>(std::round(static_cast<double>(acc) * effective));
      v += output_offset;
      output[c + out_depth * b] = static_cast<int8_t>(ClampI32(v, act_min, act_max));
    }
  }
}

void orc_asymmetric_quantize_floats(const float* values, int size, int8_t* quantized,
                                    float* scaling_factor, int32_t* offset, int variant) {
  AsymmetricQuantize(values, size, quantized, scaling_factor, offset, variant);
}

void orc_symmetric_quantize_floats(const float* values, int size, int8_t* quantized,
                                   float* scaling_factor, int variant) {
  SymmetricQuantize(values, size, quantized, scaling_factor, variant);
}

void orc_batch_quantize_floats(const float* values, int n_batch, int n_data, int8_t* quantized,
                               float* scaling_factors, int32_t* zero_points, int do_asymmetric,
                               int variant) {
  for (int b = 0; b < n_batch; ++b) {
    const size_t off = static_cast<size_t>(b) * n_data;
    if (do_asymmetric) {
      AsymmetricQuantize(values + off, n_data, quantized + off, &scaling_factors[b],
                         &zero_points[b], variant);
    } else {
      SymmetricQuantize(values + off, n_data, quantized + off, &scaling_factors[b], variant);
      if (zero_points) zero_points[b] = 0;
    }
  }
}

void orc_matrix_batch_vector_multiply_accumulate(const int8_t* matrix, int m_rows, int m_cols,
                                                 const int8_t* vectors,
                                                 const float* scaling_factors, int n_batch,
                                                 float* result, const float* per_channel_scale,
                                                 const int32_t* input_offset, int32_t* row_sums,
                                                 int compute_row_sums) {
  if (input_offset == nullptr) {
    // reference/portable_tensor_utils.cc:140-163.
    for (int b = 0; b < n_batch; ++b) {
      const int8_t* vec = vectors + static_cast<size_t>(b) * m_cols;
      for (int r = 0; r < m_rows; ++r) {
        const int8_t* row = matrix + static_cast<size_t>(r) * m_cols;
        int32_t dot = 0;
        for (int c = 0; c < m_cols; ++c) dot += row[c] * vec[c];
        const float term = static_cast<float>(dot) * scaling_factors[b];
        result[static_cast<size_t>(b) * m_rows + r] += term;
      }
    }
    return;
  }
  if (compute_row_sums) {
    for (int r = 0; r < m_rows; ++r) {
      int32_t s = 0;
      for (int c = 0; c < m_cols; ++c) s += matrix[static_cast<size_t>(r) * m_cols + c];
      row_sums[r] = s;
    }
  }
  for (int b = 0; b < n_batch; ++b) {
    const int8_t* vec = vectors + static_cast<size_t>(b) * m_cols;
    const float batch_scale = scaling_factors[b];
    const int32_t batch_offset = input_offset[b];
    for (int r = 0; r < m_rows; ++r) {
      const int8_t* row = matrix + static_cast<size_t>(r) * m_cols;
      float scale = batch_scale;
      if (per_channel_scale) scale *= per_channel_scale[r];
      int32_t dot = 0;
      for (int c = 0; c < m_cols; ++c) dot += row[c] * vec[c];
      dot -= row_sums[r] * batch_offset;
      const float term = static_cast<float>(dot) * scale;
      result[static_cast<size_t>(b) * m_rows + r] += term;
    }
  }
}

int orc_apply_activation(float* data, int size, int activation) {
  switch (activation) {
    case ORC_ACT_NONE:
      return 0;
    case ORC_ACT_RELU:
      for (int i = 0; i < size; ++i) data[i] = std::max(0.0f, data[i]);
      return 0;
    case ORC_ACT_RELU_N1_TO_1:
      for (int i = 0; i < size; ++i) data[i] = std::max(-1.0f, std::min(data[i], 1.0f));
      return 0;
    case ORC_ACT_RELU6:
      for (int i = 0; i < size; ++i) data[i] = std::max(0.0f, std::min(data[i], 6.0f));
      return 0;
    case ORC_ACT_SIGN_BIT:
      for (int i = 0; i < size; ++i) data[i] = std::signbit(data[i]) ? 1.0f : 0.0f;
      return 0;
    default:
      return 1;
  }
}

int orc_fc_hybrid_cached(const float* input, int batches, int depth, const int8_t* filter,
                         int out_depth, const float* per_channel_scales, float filter_scale,
                         const float* bias, int asymmetric_quantize_inputs, int activation,
                         int quant_variant, float* output, int8_t* q_out, float* sf_out,
                         int32_t* zp_out, int32_t* row_sums, int compute_row_sums) {
  const size_t total_in = static_cast<size_t>(batches) * depth;
  // fully_connected.cc:780-786.
  for (int b = 0; b < batches; ++b) {
    for (int n = 0; n < out_depth; ++n) {
      output[static_cast<size_t>(b) * out_depth + n] = bias ? bias[n] : 0.0f;
    }
  }
  // fully_connected.cc:789-795: all-zero input skips the product.
  bool all_zero = true;
  for (size_t i = 0; i < total_in; ++i) {
    if (input[i] != 0.0f) {
      all_zero = false;
      break;
    }
  }
  std::vector<int8_t> q(total_in);
  std::vector<float> sf(batches);
  std::vector<int32_t> zp(batches);
  if (all_zero) {
    if (q_out) std::memset(q_out, 0, total_in);
    for (int b = 0; b < batches; ++b) {
      if (sf_out) sf_out[b] = 1.0f;
      if (zp_out) zp_out[b] = 0;
    }
    return orc_apply_activation(output, batches * out_depth, activation);
  }
  orc_batch_quantize_floats(input, batches, depth, q.data(), sf.data(), zp.data(),
                            asymmetric_quantize_inputs, quant_variant);
  if (q_out) std::memcpy(q_out, q.data(), total_in);
  if (sf_out) std::memcpy(sf_out, sf.data(), batches * sizeof(float));
  if (zp_out) std::memcpy(zp_out, zp.data(), batches * sizeof(int32_t));
  if (!per_channel_scales) {
    // fully_connected.cc:838-843.
    for (int b = 0; b < batches; ++b) sf[b] *= filter_scale;
  }
  orc_matrix_batch_vector_multiply_accumulate(filter, out_depth, depth, q.data(), sf.data(),
                                              batches, output, per_channel_scales, zp.data(),
                                              row_sums, compute_row_sums);
  return orc_apply_activation(output, batches * out_depth, activation);
}

int orc_fc_hybrid(const float* input, int batches, int depth, const int8_t* filter, int out_depth,
                  const float* per_channel_scales, float filter_scale, const float* bias,
                  int asymmetric_quantize_inputs, int activation, int quant_variant,
                  float* output, int8_t* q_out, float* sf_out, int32_t* zp_out) {
  std::vector<int32_t> row_sums(out_depth);
  return orc_fc_hybrid_cached(input, batches, depth, filter, out_depth, per_channel_scales,
                              filter_scale, bias, asymmetric_quantize_inputs, activation,
                              quant_variant, output, q_out, sf_out, zp_out, row_sums.data(), 1);
}

// tflite/kernels/batch_matmul.cc:454-520 (EvalHybrid) over
// tflite/kernels/internal/reference/batch_matmul.h:111-210 (the hybrid BatchMatMul kernel, which
// both registrations run). The op has already put the int8 operand into [matrix][unit][depth]
// order (its RHS transposed unless adj_y) and flattened the float operand to rows of `depth`
// values; broadcasting arrives here resolved: output batch b multiplies the `rows` rows of float
// batch lhs_batch_index[b] with weight matrix rhs_batch_index[b].
// Note the zero-point correction: `total -= row_sum * batch_offset` with a FLOAT batch_offset
// (batch_matmul.h:199-200), i.e. int32 total -> float, float product, float subtraction, and
// truncation back to int32; and the final `out += scale * total` onto a zero-filled output.
void orc_batch_matmul_hybrid(const float* lhs, int lhs_batches, int rows, int depth,
                             const int8_t* weights, int weight_matrices, int units,
                             const float* per_channel_scales, float filter_scale,
                             int asymmetric_quantize_inputs, int quant_variant,
                             const int* lhs_batch_index, const int* rhs_batch_index,
                             int out_batches, float* output) {
  const int quant_rows = lhs_batches * rows;  // num_batches_to_quantize, batch_matmul.cc:472-475
  std::vector<int8_t> q(static_cast<size_t>(quant_rows) * depth);
  std::vector<float> sf(quant_rows);
  std::vector<int32_t> offsets(quant_rows, 0);  // memset to 0 when symmetric, :487-489
  orc_batch_quantize_floats(lhs, quant_rows, depth, q.data(), sf.data(), offsets.data(),
                            asymmetric_quantize_inputs, quant_variant);
  if (!asymmetric_quantize_inputs) std::fill(offsets.begin(), offsets.end(), 0);
  if (!per_channel_scales) {
    for (int b = 0; b < quant_rows; ++b) sf[b] *= filter_scale;  // :508-513
  }
  // ReductionSumVector over every weight matrix, batch_matmul.h:148-163.
  std::vector<int32_t> row_sums(static_cast<size_t>(weight_matrices) * units);
  for (size_t r = 0; r < row_sums.size(); ++r) {
    int32_t sum = 0;
    for (int k = 0; k < depth; ++k) sum += weights[r * depth + k];
    row_sums[r] = sum;
  }
  std::fill_n(output, static_cast<size_t>(out_batches) * rows * units, 0.0f);  // :520
  for (int b = 0; b < out_batches; ++b) {
    const int8_t* w = weights + static_cast<size_t>(rhs_batch_index[b]) * units * depth;
    const int32_t* wsum = row_sums.data() + static_cast<size_t>(rhs_batch_index[b]) * units;
    const size_t row0 = static_cast<size_t>(lhs_batch_index[b]) * rows;
    float* out = output + static_cast<size_t>(b) * rows * units;
    for (int j = 0; j < rows; ++j) {
      const float batch_scaling_factor = sf[row0 + j];
      const float batch_offset = static_cast<float>(offsets[row0 + j]);
      const int8_t* x = q.data() + (row0 + j) * depth;
      for (int i = 0; i < units; ++i) {
        int32_t total = 0;
        for (int k = 0; k < depth; ++k) total += w[static_cast<size_t>(i) * depth + k] * x[k];
        const int32_t row_sum = wsum[i];
        total -= row_sum * batch_offset;  // the reference's mixed int/float compound assignment
        float scale = batch_scaling_factor;
        if (per_channel_scales) scale *= per_channel_scales[i];
        out[static_cast<size_t>(units) * j + i] += scale * total;
      }
    }
  }
}

void orc_fc_blockwise_int4(const float* input, int batches, int depth,
                           const uint8_t* packed_filter, int out_depth,
                           const uint16_t* scales_f16, int blocksize, const float* bias,
                           int quant_variant, float* output) {
  const size_t num_blocks = static_cast<size_t>(depth) / blocksize;
  const size_t k2 = (static_cast<size_t>(depth) + 1) & ~static_cast<size_t>(1);
  std::vector<float> scales(static_cast<size_t>(out_depth) * num_blocks);
  for (size_t i = 0; i < scales.size(); ++i) scales[i] = orc_half_to_float(scales_f16[i]);
  std::vector<int8_t> q(static_cast<size_t>(batches) * depth);
  std::vector<float> in_scales(batches);
  std::vector<int32_t> in_zps(batches);
  orc_batch_quantize_floats(input, batches, depth, q.data(), in_scales.data(), in_zps.data(),
                            /*do_asymmetric=*/1, quant_variant);
  for (int m = 0; m < batches; ++m) {
    for (int n = 0; n < out_depth; ++n) {
      float out = 0.0f;
      float kfsum = 0.0f;
      for (size_t bi = 0; bi < num_blocks; ++bi) {
        int32_t ksum = 0;
        int32_t acc = 0;
        for (int ki = 0; ki < blocksize; ++ki) {
          const size_t k = bi * blocksize + ki;
          const size_t byte_index = (static_cast<size_t>(n) * k2 + k) / 2;
          const uint8_t byte = packed_filter[byte_index];
          const int nibble = (k % 2 == 0) ? (byte & 0xF) : (byte >> 4);
          const int32_t w = (nibble ^ 0x8) - 8;
          ksum += w;
          acc += static_cast<int32_t>(q[static_cast<size_t>(m) * depth + k]) * w;
        }
        const float scale = scales[static_cast<size_t>(n) * num_blocks + bi];
        const float term = static_cast<float>(acc) * scale;
        out = out + term;
        const float kterm = scale * static_cast<float>(ksum);
        kfsum = kfsum + kterm;
      }
      const float zp_term = static_cast<float>(in_zps[m]) * kfsum;
      out = out - zp_term;
      out = out * in_scales[m];
      if (bias) out = out + bias[n];
      output[static_cast<size_t>(m) * out_depth + n] = out;
    }
  }
}

// Per-channel int4 hybrid FULLY_CONNECTED: EvalHybridDense4Bit, tflite/kernels/fully_connected.cc
// :1088-1178, in the arithmetic of its reference kernels
// (tflite/kernels/internal/optimized/4bit/fully_connected_reference.cc):
//   ReferenceBatchQuantizeFloats4Bit :121-180  symmetric per-row quantization, scale 127 / max|x|
//     computed in double and stored as float, q = (int8)round(x * scale), and
//     input_offset = sum(q) * zero_point_4bit (-7, fully_connected_common.h:27);
//   ReferenceAssignBiasAndComputeOffsets :182-206  out = (offset * sf) * fs + bias;
//   ReferenceRunKernel :290-329 with ReferenceUnpack :215-272
//     out += (float(sum((w + 7) * q)) * sf) * fs, the weights being stored as w + 7;
//   then ApplyActivationToVector. The tile layouts of the reference (4 x 32 boxes) only
//   permute exact integer sums and are not restated. Weights are expected in [-7, 7], as the
//   reference's prepacking assumes (merge(), fully_connected_common.h:36-42).
void orc_fc_hybrid_int4_per_channel(const float* input, int batches, int depth,
                                    const uint8_t* packed_filter, int out_depth,
                                    const float* filter_scales, const float* bias,
                                    int activation, float* output) {
  const size_t k2 = (static_cast<size_t>(depth) + 1) & ~static_cast<size_t>(1);
  std::vector<int8_t> q(depth);
  for (int m = 0; m < batches; ++m) {
    const float* x = input + static_cast<size_t>(m) * depth;
    float scale_denom = 0;
    for (int c = 0; c < depth; ++c) scale_denom = std::max(scale_denom, std::abs(x[c]));
    if (scale_denom == 0) scale_denom = 127.0;
    const float scale = 127.0 / scale_denom;           // double division, float store
    const float batch_scale = scale_denom / 127.0;     // likewise
    int32_t offset = 0;
    for (int d = 0; d < depth; ++d) {
      const float prod = x[d] * scale;
      q[d] = static_cast<int8_t>(std::round(prod));
      offset += q[d];
    }
    offset = offset * -7;
    const float val = offset * batch_scale;
    for (int n = 0; n < out_depth; ++n) {
      int32_t acc = 0;
      for (int k = 0; k < depth; ++k) {
        const uint8_t byte = packed_filter[(static_cast<size_t>(n) * k2 + k) / 2];
        const int nibble = (k % 2 == 0) ? (byte & 0xF) : (byte >> 4);
        const int32_t w = (nibble ^ 0x8) - 8;
        acc += (w + 7) * static_cast<int32_t>(q[k]);
      }
      float out = val * filter_scales[n];
      if (bias) out = out + bias[n];
      const float term = acc * batch_scale;
      out = out + term * filter_scales[n];
      output[static_cast<size_t>(m) * out_depth + n] = out;
    }
  }
  orc_apply_activation(output, static_cast<int64_t>(batches) * out_depth, activation);
}

// IEEE binary32 -> binary16, round to nearest even, subnormals kept, overflow to infinity: what
// `tflite::half(float)` does in either of its builds (tflite/types/half.h:69 through _Float16,
// :129 through fp16_ieee_from_fp32_value).
uint16_t orc_float_to_half(float f) {
  uint32_t bits;
  std::memcpy(&bits, &f, sizeof bits);
  const uint16_t sign = static_cast<uint16_t>((bits >> 16) & 0x8000u);
  const uint32_t abs = bits & 0x7FFFFFFFu;
  if (abs >= 0x7F800000u) {  // inf / NaN (quiet, payload top bits kept)
    return static_cast<uint16_t>(sign | 0x7C00u | (abs > 0x7F800000u ? 0x200u | ((abs >> 13) & 0x3FFu) : 0));
  }
  if (abs >= 0x477FF000u) return static_cast<uint16_t>(sign | 0x7C00u);  // rounds to >= 65520
  const int exp = static_cast<int>(abs >> 23) - 127;
  if (exp >= -14) {  // normal half
    const uint32_t man = abs & 0x7FFFFFu;
    uint32_t h = (static_cast<uint32_t>(exp + 15) << 10) | (man >> 13);
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;  // carry may bump the exponent
    return static_cast<uint16_t>(sign | h);
  }
  if (exp < -25) return sign;  // below half of the smallest subnormal
  // subnormal half: value = man24 * 2^(exp-23), unit 2^-24
  const uint32_t man24 = (abs & 0x7FFFFFu) | 0x800000u;
  const int shift = -exp - 1;  // 14..24
  uint32_t h = man24 >> shift;
  const uint32_t rem = man24 & ((1u << shift) - 1u);
  const uint32_t half_way = 1u << (shift - 1);
  if (rem > half_way || (rem == half_way && (h & 1u))) ++h;
  return static_cast<uint16_t>(sign | h);
}

namespace {

// Unpack4Bit, tflite/kernels/embedding_lookup.cc:140-159: the nibble is moved to the top of an
// int8 (16 x its signed value) and multiplied by scale / 16.
inline void EmbeddingStore(float v, int out_f16, void* output, size_t index) {
  if (out_f16) {
    static_cast<uint16_t*>(output)[index] = orc_float_to_half(v);
  } else {
    static_cast<float*>(output)[index] = v;
  }
}

void EmbeddingUnpack4Bit(float scaling_factor, size_t col_size, const int8_t* value_ptr,
                         int out_f16, void* output, size_t out_off) {
  const float scaling_factor0 = scaling_factor / 16;
  size_t j = 0, i4 = 0;
  for (; j + 1 < col_size; j += 2, ++i4) {
    const int8_t v = value_ptr[i4];
    const int8_t lo = static_cast<int8_t>(v << 4);
    const int8_t hi = static_cast<int8_t>(v & 0xF0);
    EmbeddingStore(lo * scaling_factor0, out_f16, output, out_off + j);
    EmbeddingStore(hi * scaling_factor0, out_f16, output, out_off + j + 1);
  }
  if (col_size & 1) {
    const int8_t lo = static_cast<int8_t>(value_ptr[i4] << 4);
    EmbeddingStore(lo * scaling_factor0, out_f16, output, out_off + j);
  }
}

}  // namespace

// EMBEDDING_LOOKUP on an Int4 table with blockwise quantization: EvalBlockwise,
// tflite/kernels/embedding_lookup.cc:194-307. Rows are written in lookup order until an index
// falls outside [0, rows): then -(position + 1) is returned, as the kernel fails there (:280-286).
// A column count that the block size does not divide returns 1 (:269-275).
int orc_embedding_lookup_blockwise_int4(const int32_t* lookup, int count, const uint8_t* table,
                                        int rows, int cols, const uint16_t* scales_f16,
                                        int blocksize, int out_f16, void* output) {
  if (blocksize <= 0 || cols % blocksize != 0) return 1;
  const size_t num_blocks = static_cast<size_t>(cols) / blocksize;
  const int8_t* value_ptr = reinterpret_cast<const int8_t*>(table);
  for (int i = 0; i < count; ++i) {
    const int idx = lookup[i];
    if (idx >= rows || idx < 0) return -(i + 1);
    const size_t output_row_offset = static_cast<size_t>(i) * cols;
    const size_t scale_offset = static_cast<size_t>(idx) * num_blocks;
    const size_t value_offset = static_cast<size_t>(idx) * cols;
    for (size_t j = 0; j < num_blocks; ++j) {
      const float scaling_factor = orc_half_to_float(scales_f16[scale_offset + j]);
      const size_t val_off = value_offset + j * blocksize;
      EmbeddingUnpack4Bit(scaling_factor, blocksize, &value_ptr[val_off / 2], out_f16, output,
                          output_row_offset + j * blocksize);
    }
  }
  return 0;
}

// EMBEDDING_LOOKUP from an Int8 or Int4 table to floats: EvalHybrid,
// tflite/kernels/embedding_lookup.cc:309-395. One scale for the table, or one per row
// (row_scales, :376-383). value_bits is 8 or 4. Same return convention as above.
int orc_embedding_lookup_hybrid(const int32_t* lookup, int count, const void* table, int value_bits,
                                int rows, int cols, float scale, const float* row_scales,
                                int out_f16, void* output) {
  const int8_t* value_ptr = static_cast<const int8_t*>(table);
  for (int i = 0; i < count; ++i) {
    const int32_t idx = lookup[i];
    if (idx >= rows || idx < 0) return -(i + 1);
    const size_t out_off = static_cast<size_t>(i) * cols;
    const float scaling_factor = row_scales ? row_scales[idx] : scale;
    const size_t offset = static_cast<size_t>(cols) * idx;
    if (value_bits == 4) {
      EmbeddingUnpack4Bit(scaling_factor, cols, &value_ptr[offset >> 1], out_f16, output, out_off);
    } else {
      for (int j = 0; j < cols; ++j) {
        EmbeddingStore(value_ptr[offset + j] * scaling_factor, out_f16, output, out_off + j);
      }
    }
  }
  return 0;
}

}  // extern "C"

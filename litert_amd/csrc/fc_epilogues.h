// Output epilogues shared by the int8-weight kernels. Integer accumulators are exact, so
// these few lines are where bit-exactness with the reference is decided.
#ifndef LITERT_AMD_CSRC_FC_EPILOGUES_H_
#define LITERT_AMD_CSRC_FC_EPILOGUES_H_

#include "kernels.h"

namespace lrtfc {

// Requantization of one accumulator: reference/integer_ops/fully_connected.h:65-74.
// `acc` already holds every additive term (dot product, offset corrections, bias).
__device__ __forceinline__ int8_t RequantizeCore(int32_t acc, int32_t multiplier, int shift,
                                                 int32_t output_offset, int32_t act_min,
                                                 int32_t act_max) {
  const int32_t v = Mbqm(acc, multiplier, shift) + output_offset;
  return static_cast<int8_t>(ClampI32(v, act_min, act_max));
}

// The same value as RequantizeCore for the common case, in half the instructions: a right
// shift by right_shift = 1..31 bits, multiplier != INT32_MIN, |acc| < 2^30 and act_lo <= act_hi
// (the caller checks all four). SaturatingRoundingDoublingHighMul cannot saturate then and is
// floor((acc * multiplier + 2^30) / 2^31); RoundingDivideByPOT of r, nearest with ties away from
// zero, is (r + 2^(right_shift - 1) - (r < 0)) >> right_shift, a sum that stays below 2^31
// because |r| <= |acc|. half = 2^(right_shift - 1).
__device__ __forceinline__ int32_t RequantizeShort(int32_t acc, int32_t multiplier,
                                                   int right_shift, int32_t half,
                                                   int32_t output_offset, int32_t act_lo,
                                                   int32_t act_hi) {
  const int64_t t = static_cast<int64_t>(acc) * multiplier + (1ll << 30);
  const int32_t r = static_cast<int32_t>(t >> 31);
  const int32_t v = ((r + half + (r >> 31)) >> right_shift) + output_offset;
  int32_t out;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(out) : "v"(v), "v"(act_lo), "v"(act_hi));
  return out;
}

// The low bytes of four values as one dword, first value lowest.
__device__ __forceinline__ int32_t PackLowBytes(int32_t q0, int32_t q1, int32_t q2, int32_t q3) {
  const uint32_t lo = __builtin_amdgcn_perm(q1, q0, 0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm(q3, q2, 0x0c0c0400u);
  return static_cast<int32_t>(__builtin_amdgcn_perm(hi, lo, 0x05040100u));
}

// Hybrid output value: reference/portable_tensor_utils.cc:186-203 after the bias
// initialisation of fully_connected.cc:780-786, then ApplyActivationToVector.
// channel_scale is the per-channel scale, or the per-tensor filter scale.
__device__ __forceinline__ float HybridCore(int32_t dot, float batch_scale, float channel_scale,
                                            int32_t batch_zero_point, int32_t row_sum, float base,
                                            int activation) {
  const float scale = __fmul_rn(batch_scale, channel_scale);
  dot -= row_sum * batch_zero_point;
  const float out = __fadd_rn(base, __fmul_rn(static_cast<float>(dot), scale));
  return ApplyFloatActivation(out, activation);
}

// EvalHybridDense leaves the output at activation(bias) when the WHOLE input is zero and skips
// the product (tflite/kernels/fully_connected.cc:789-795). Adding the zero product instead gives
// the same bits except for a bias element of -0.0f (-0.0f + 0.0f is +0.0f). So the kernels add
// the product as always and repair that one case lazily: a thread that meets a -0.0f bias with a
// zero dot product scans the input; only a whole-zero input takes the scan to its end. A row of
// finite values quantizes to all-zero values exactly when it was all zero (any other row has a
// value at the far end of the int8 range), so the quantized rows can stand for the float ones.
// Not so for NaN: the row's min/max (fminf/fmaxf) drop NaNs, so a row of only zeros and NaNs
// quantizes to zeros and takes the exit here, while the reference's IsZeroVector (v != 0) counts
// a NaN as non-zero and adds the product; the difference shows only in a -0.0f bias element.
// The scans are
// real function calls: inlined into an unrolled epilogue their loops keep it from unrolling, and
// the accumulator tiles then land in scratch memory.
__device__ __attribute__((noinline)) bool AllZeroInt8(const int8_t* p, size_t n) {
  size_t i = 0;
  if ((reinterpret_cast<uintptr_t>(p) & 15) == 0) {
    const i32x4* v = reinterpret_cast<const i32x4*>(p);
    for (; i + 64 <= n; i += 64) {
      const i32x4 t = (v[i / 16] | v[i / 16 + 1]) | (v[i / 16 + 2] | v[i / 16 + 3]);
      if ((t.x | t.y | t.z | t.w) != 0) return false;
    }
  }
  for (; i < n; ++i) {
    if (p[i] != 0) return false;
  }
  return true;
}

// IsZeroVector: -0.0f counts as zero.
__device__ __attribute__((noinline)) bool AllZeroF32(const float* p, size_t n) {
  const uint32_t* u = reinterpret_cast<const uint32_t*>(p);
  size_t i = 0;
  for (; i + 4 <= n; i += 4) {
    if ((((u[i] | u[i + 1]) | (u[i + 2] | u[i + 3])) << 1) != 0) return false;
  }
  for (; i < n; ++i) {
    if ((u[i] << 1) != 0) return false;
  }
  return true;
}

__device__ __forceinline__ bool IsNegativeZero(float v) {
  return __float_as_uint(v) == 0x80000000u;
}

// Output value of the hybrid BATCH_MATMUL kernel, reference/batch_matmul.h:190-206: the
// zero-point correction `total -= row_sum * batch_offset` runs through float (batch_offset is a
// float there: int32 -> float, float product, float subtraction, truncation back to int32),
// then `out += scale * total` onto a zero-filled output. Differs from HybridCore as soon as a
// dot product or a correction exceeds 2^24.
__device__ __forceinline__ float HybridBatchMatMulCore(int32_t dot, float batch_scale,
                                                       float channel_scale,
                                                       int32_t batch_zero_point, int32_t row_sum) {
  const float corrected = __fsub_rn(
      static_cast<float>(dot),
      __fmul_rn(static_cast<float>(row_sum), static_cast<float>(batch_zero_point)));
  const int32_t total = static_cast<int32_t>(corrected);
  const float scale = __fmul_rn(batch_scale, channel_scale);
  return __fadd_rn(0.0f, __fmul_rn(scale, static_cast<float>(total)));
}

// HybridCore for kernels that run on already quantized rows (a.input), with the whole-zero-input
// case above when the caller asked for EvalHybridDense semantics (a.zero_input_exit), or the
// BATCH_MATMUL arithmetic (a.batch_matmul).
__device__ __forceinline__ float HybridCoreZeroAware(const FcInt8Args& a, int32_t dot,
                                                     float batch_scale, float channel_scale,
                                                     int32_t batch_zero_point, int32_t row_sum,
                                                     float base) {
  if (a.batch_matmul) {
    return HybridBatchMatMulCore(dot, batch_scale, channel_scale, batch_zero_point, row_sum);
  }
  if (a.zero_input_exit && dot == 0 && IsNegativeZero(base) &&
      AllZeroInt8(a.input, static_cast<size_t>(a.batches) * a.depth)) {
    return ApplyFloatActivation(base, a.activation);
  }
  return HybridCore(dot, batch_scale, channel_scale, batch_zero_point, row_sum, base,
                    a.activation);
}

// The same choice without a branch or a loop, for epilogues that must unroll completely (an
// accumulator tile indexed inside a loop that did not unroll lands in scratch memory): the
// caller has settled `zero_input` for the whole workgroup beforehand. Adding -0.0f instead of the
// zero product leaves every bias value as it is, -0.0f included, which is what the early exit
// amounts to.
__device__ __forceinline__ float HybridCoreSelect(int32_t dot, float batch_scale,
                                                  float channel_scale, int32_t batch_zero_point,
                                                  int32_t row_sum, float base, int activation,
                                                  bool batch_matmul, bool zero_input) {
  const float scale = __fmul_rn(batch_scale, channel_scale);
  const float as_bmm =
      HybridBatchMatMulCore(dot, batch_scale, channel_scale, batch_zero_point, row_sum);
  const int32_t corrected = dot - row_sum * batch_zero_point;
  const float term = zero_input ? -0.0f : __fmul_rn(static_cast<float>(corrected), scale);
  const float as_fc = ApplyFloatActivation(__fadd_rn(base, term), activation);
  return batch_matmul ? as_bmm : as_fc;
}

// Whole-input zero test by a whole workgroup (every thread must call it): threads scan
// interleaved 16-byte pieces and meet after every round, so a non-zero input ends the scan
// after the first round.
__device__ inline bool WorkgroupAllZeroInt8(const int8_t* p, size_t n) {
  const bool vec = (reinterpret_cast<uintptr_t>(p) & 15) == 0;
  const size_t pieces = vec ? n / 16 : 0;
  for (size_t base = 0; base < pieces; base += blockDim.x) {
    const size_t i = base + threadIdx.x;
    int nonzero = 0;
    if (i < pieces) {
      const i32x4 t = reinterpret_cast<const i32x4*>(p)[i];
      nonzero = (t.x | t.y | t.z | t.w) != 0;
    }
    if (__syncthreads_or(nonzero)) return false;
  }
  int nonzero = 0;
  for (size_t i = pieces * 16 + threadIdx.x; i < n; i += blockDim.x) nonzero |= p[i] != 0;
  return !__syncthreads_or(nonzero);
}

// Output value of the per-channel int4 hybrid path: ReferenceAssignBiasAndComputeOffsets and
// ReferenceUnpack (tflite/kernels/internal/optimized/4bit/fully_connected_reference.cc:182-272)
// followed by ApplyActivationToVector. `dot` is sum(w * q) over the depth with the signed
// weights; the reference accumulates sum((w + 7) * q) = dot + 7 * sum(q) = dot - input_offset.
__device__ __forceinline__ float Hybrid4BitCore(int32_t dot, float batch_scale,
                                                float channel_scale, int32_t input_offset,
                                                float bias, bool has_bias, int activation) {
  const float val = __fmul_rn(static_cast<float>(input_offset), batch_scale);
  float out = __fmul_rn(val, channel_scale);
  if (has_bias) out = __fadd_rn(out, bias);
  const float term = __fmul_rn(static_cast<float>(dot - input_offset), batch_scale);
  out = __fadd_rn(out, __fmul_rn(term, channel_scale));
  return ApplyFloatActivation(out, activation);
}

// Pointer forms used by the row-major kernels.
__device__ __forceinline__ void StoreRequantized(const FcInt8Args& a, int b, int n, int32_t dot,
                                                 int32_t xsum) {
  // sum (w + fo)(x + io) = dot + io * sum(w) + fo * sum(x) + depth * fo * io
  int32_t acc = dot;
  if (a.input_offset != 0) acc += a.input_offset * a.filter_row_sums[n];
  if (a.filter_offset != 0) {
    acc += a.filter_offset * xsum + a.depth * a.filter_offset * a.input_offset;
  }
  if (a.bias_i32) acc += a.bias_i32[n];
  const int32_t m = a.per_channel ? a.multipliers[n] : a.multipliers[0];
  const int s = a.per_channel ? a.shifts[n] : a.shifts[0];
  a.output_i8[static_cast<size_t>(b) * a.out_depth + n] =
      RequantizeCore(acc, m, s, a.output_offset, a.act_min, a.act_max);
}

__device__ __forceinline__ void StoreHybrid(const FcInt8Args& a, int b, int n, int32_t dot,
                                            float batch_scale, int32_t batch_zero_point) {
  const float channel_scale = a.per_channel_scales ? a.per_channel_scales[n] : a.filter_scale;
  const int32_t row_sum = batch_zero_point != 0 ? a.filter_row_sums[n] : 0;
  const float base = a.bias_f32 ? a.bias_f32[n] : 0.0f;
  a.output_f32[static_cast<size_t>(b) * a.out_depth + n] =
      HybridCoreZeroAware(a, dot, batch_scale, channel_scale, batch_zero_point, row_sum, base);
}

}  // namespace lrtfc

#endif  // LITERT_AMD_CSRC_FC_EPILOGUES_H_

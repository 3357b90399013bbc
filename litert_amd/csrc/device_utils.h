// Device-side helpers shared by the gfx950 FULLY_CONNECTED kernels.
#ifndef LITERT_AMD_CSRC_DEVICE_UTILS_H_
#define LITERT_AMD_CSRC_DEVICE_UTILS_H_

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace lrtfc {

constexpr int kWaveSize = 64;

// 128-bit register quad: the unit of every weight load (global_load_dwordx4).
using i32x4 = int __attribute__((ext_vector_type(4)));
using i32x2 = int __attribute__((ext_vector_type(2)));

// ---- integer requantization -------------------------------------------------

// SaturatingRoundingDoublingHighMul (gemmlowp fixedpoint, as used by
// tflite/kernels/internal/common.cc:83-89): (ab + nudge) / 2^31 with a truncating
// division, nudge = 2^30 for ab >= 0 and 1 - 2^30 otherwise. For either sign that
// quotient equals floor((ab + 2^30) / 2^31), which needs no sign test: one 64-bit
// multiply-add and an arithmetic shift.
__device__ __forceinline__ int32_t Srdhm(int32_t a, int32_t b) {
  const int64_t t = static_cast<int64_t>(a) * static_cast<int64_t>(b) + (1ll << 30);
  const int32_t r = static_cast<int32_t>(t >> 31);
  // The one product that does not fit (INT32_MIN squared) saturates; as a select, so that
  // the epilogues stay free of branches.
  return (a == INT32_MIN && b == INT32_MIN) ? INT32_MAX : r;
}

// RoundingDivideByPOT: shift right, nearest, ties away from zero.
__device__ __forceinline__ int32_t RoundingDivideByPot(int32_t x, int exponent) {
  const int32_t mask = static_cast<int32_t>((1ll << exponent) - 1);
  const int32_t remainder = x & mask;
  const int32_t threshold = (mask >> 1) + (x < 0 ? 1 : 0);
  return (x >> exponent) + (remainder > threshold ? 1 : 0);
}

// MultiplyByQuantizedMultiplier, double-rounding build
// (tflite/kernels/internal/common.cc:80-90). The left shift wraps as the
// reference's int32 multiply does.
__device__ __forceinline__ int32_t Mbqm(int32_t x, int32_t quantized_multiplier, int shift) {
  const int left_shift = shift > 0 ? shift : 0;
  const int right_shift = shift > 0 ? 0 : -shift;
  const int32_t shifted = static_cast<int32_t>(static_cast<uint32_t>(x) << left_shift);
  return RoundingDivideByPot(Srdhm(shifted, quantized_multiplier), right_shift);
}

__device__ __forceinline__ int32_t ClampI32(int32_t v, int32_t lo, int32_t hi) {
  return min(max(v, lo), hi);
}

// ---- float helpers (explicitly rounded: no FMA contraction) -----------------

__device__ __forceinline__ float ApplyFloatActivation(float v, int activation) {
  // tflite/kernels/internal/portable_tensor_utils.cc:41-71, written out as std::max(a, b) =
  // (a < b) ? b : a and std::min(a, b) = (b < a) ? b : a, which also fixes what a -0.0f or a NaN
  // turns into (std::max(0.0f, -0.0f) is +0.0f; std::max(-1.0f, -0.0f) is -0.0f).
  switch (activation) {
    case 1:
      return (0.0f < v) ? v : 0.0f;
    case 2: {
      const float t = (1.0f < v) ? 1.0f : v;
      return (-1.0f < t) ? t : -1.0f;
    }
    case 3: {
      const float t = (6.0f < v) ? 6.0f : v;
      return (0.0f < t) ? t : 0.0f;
    }
    case 5:  // kTfLiteActSignBit: std::signbit as a float
      return (__float_as_uint(v) >> 31) ? 1.0f : 0.0f;
    default:
      return v;
  }
}

// The same function without a branch, for epilogues whose few active lanes should not walk a
// switch per value: every clamp is `t = (hi < v) ? hi : v; (lo < t) ? t : lo` with its bounds
// (RELU: 0 and +infinity, whose upper test never holds, as in the form above), selected by
// wave-uniform conditions.
__device__ __forceinline__ float ApplyFloatActivationSelect(float v, int activation) {
  const float lo = activation == 2 ? -1.0f : 0.0f;
  const float hi = activation == 2 ? 1.0f : (activation == 3 ? 6.0f : __builtin_inff());
  const float t = (hi < v) ? hi : v;
  const float clamped = (lo < t) ? t : lo;
  const float sign = (__float_as_uint(v) >> 31) ? 1.0f : 0.0f;
  const bool clamps = activation >= 1 && activation <= 3;
  return clamps ? clamped : (activation == 5 ? sign : v);
}

// IEEE binary16 -> binary32, exact for every finite pattern, subnormals included.
__device__ __forceinline__ float HalfBitsToFloat(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1Fu;
  const uint32_t man = h & 0x3FFu;
  if (exp == 0) {
    // subnormal or zero: man * 2^-24, exact in float
    const float mag = static_cast<float>(man) * 5.9604644775390625e-08f;
    return __uint_as_float(__float_as_uint(mag) | sign);
  }
  if (exp == 31) return __uint_as_float(sign | 0x7F800000u | (man << 13));
  return __uint_as_float(sign | ((exp + 112u) << 23) | (man << 13));
}

// The same conversion through the hardware's half-to-float instruction, which handles
// subnormals, infinities and NaNs as IEEE 754 prescribes (the conversion is exact).
__device__ __forceinline__ float HalfBitsToFloatFast(uint16_t h) {
  return __half2float(__ushort_as_half(h));
}

// ---- wave64 reductions --------------------------------------------------------

// Sum over the 64 lanes of a wavefront; every lane receives the total. Integer
// addition is associative, so the order of the butterfly cannot change results.
__device__ __forceinline__ int32_t WaveSumI32(int32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWaveSize);
  return v;
}

// f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N - 1>{}): a loop whose
// index is a compile-time constant in the body.
template <int N, int I = 0, typename F>
__device__ __forceinline__ void StaticFor(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    StaticFor<N, I + 1>(f);
  }
}

// Float min / max over the 64 lanes; every lane receives the result (it is wave-uniform).
// Four data-parallel-primitive steps reduce each row of 16 lanes inside the vector ALU (lane
// swaps within quads, then the half-row and row mirrors), and the four row results are read
// out as scalars: 10 short instructions, where a butterfly of cross-lane shuffles goes
// through the LDS crossbar six times in sequence. min and max are exact and order-free.
template <int CTRL>
__device__ __forceinline__ float DppMoveF32(float v) {
  const int i = __float_as_int(v);
  return __int_as_float(__builtin_amdgcn_update_dpp(i, i, CTRL, 0xF, 0xF, false));
}

__device__ __forceinline__ float ReadLaneF32(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

constexpr int kDppQuadSwap1 = 0xB1;       // quad_perm [1, 0, 3, 2]
constexpr int kDppQuadSwap2 = 0x4E;       // quad_perm [2, 3, 0, 1]
constexpr int kDppRowHalfMirror = 0x141;  // lane i <-> 7 - i within each 8
constexpr int kDppRowMirror = 0x140;      // lane i <-> 15 - i within each 16

__device__ __forceinline__ float WaveMinF32(float v) {
  v = fminf(v, DppMoveF32<kDppQuadSwap1>(v));
  v = fminf(v, DppMoveF32<kDppQuadSwap2>(v));
  v = fminf(v, DppMoveF32<kDppRowHalfMirror>(v));
  v = fminf(v, DppMoveF32<kDppRowMirror>(v));
  return fminf(fminf(ReadLaneF32(v, 0), ReadLaneF32(v, 16)),
               fminf(ReadLaneF32(v, 32), ReadLaneF32(v, 48)));
}

__device__ __forceinline__ float WaveMaxF32(float v) {
  v = fmaxf(v, DppMoveF32<kDppQuadSwap1>(v));
  v = fmaxf(v, DppMoveF32<kDppQuadSwap2>(v));
  v = fmaxf(v, DppMoveF32<kDppRowHalfMirror>(v));
  v = fmaxf(v, DppMoveF32<kDppRowMirror>(v));
  return fmaxf(fmaxf(ReadLaneF32(v, 0), ReadLaneF32(v, 16)),
               fmaxf(ReadLaneF32(v, 32), ReadLaneF32(v, 48)));
}

// 4-way int8 dot product with int32 accumulate (v_dot4_i32_i8).
__device__ __forceinline__ int32_t Dot4(int32_t a, int32_t b, int32_t acc) {
  return __builtin_amdgcn_sdot4(a, b, acc, false);
}

}  // namespace lrtfc

#endif  // LITERT_AMD_CSRC_DEVICE_UTILS_H_

// Device-side pieces of the per-row activation quantizer, shared by the standalone
// BatchQuantizeFloats kernel and by the GEMV kernels that quantize their input rows in
// their own prologue. Semantics: tflite/kernels/internal/reference/portable_tensor_utils.cc
// :41-119 (portable, normative) and optimized/neon_tensor_utils.cc:2347-2552 (the two
// NEON-flavoured variants).
#ifndef LITERT_AMD_CSRC_QUANTIZE_DEVICE_H_
#define LITERT_AMD_CSRC_QUANTIZE_DEVICE_H_

#include "device_utils.h"
#include "../../include/litert_amd_fc.h"

namespace lrtfc {

struct RowQuantParams {
  float scale;     // scaling factor stored for the row
  float inv;       // multiplier applied to each element
  int32_t zero_point;
  bool all_zero;   // the row quantizes to zeros with scale 1 / zero point 0
};

// mn = min(0, min v), mx = max(0, max v) of the row.
template <int VARIANT>
__device__ __forceinline__ RowQuantParams AsymmetricRowParams(float mn, float mx) {
  RowQuantParams p;
  p.zero_point = 0;
  p.all_zero = false;
  if (mn == mx) {  // both 0
    p.all_zero = true;
    p.scale = 1.0f;
    p.inv = 1.0f;
    return p;
  }
  const double qmin = -128.0, qmax = 127.0;
  const double rmin = static_cast<double>(mn);
  const double rmax = static_cast<double>(mx);
  // Portable widens to double before subtracting (portable_tensor_utils.cc:81-87); the
  // NEON build subtracts in float (neon_tensor_utils.cc:2486).
  const double span = (VARIANT == LRTFC_QUANT_PORTABLE)
                          ? (rmax - rmin)
                          : static_cast<double>(__fsub_rn(mx, mn));
  const double scale = span / (qmax - qmin);
  const double zp_from_min = qmin - rmin / scale;
  const double zp_from_max = qmax - rmax / scale;
  const double err_from_min = fabs(qmin) + fabs(rmin / scale);
  const double err_from_max = fabs(qmax) + fabs(rmax / scale);
  const double zp_double = err_from_min < err_from_max ? zp_from_min : zp_from_max;
  if (zp_double <= qmin) {
    p.zero_point = -128;
  } else if (zp_double >= qmax) {
    p.zero_point = 127;
  } else {
    p.zero_point = static_cast<int8_t>(round(zp_double));
  }
  p.scale = static_cast<float>(scale);
  if (VARIANT == LRTFC_QUANT_PORTABLE) {
    p.inv = __fdiv_rn(1.0f, p.scale);
  } else {
    p.inv = p.scale == 0.0f ? 0.0f : static_cast<float>(1.0 / static_cast<double>(p.scale));
  }
  return p;
}

__device__ __forceinline__ RowQuantParams SymmetricRowParams(float mn, float mx) {
  RowQuantParams p;
  p.zero_point = 0;
  const float absmax = fmaxf(fabsf(mn), fabsf(mx));
  p.all_zero = absmax == 0.0f;
  if (p.all_zero) {
    p.scale = 1.0f;
    p.inv = 1.0f;
  } else {
    p.scale = __fdiv_rn(absmax, 127.0f);
    p.inv = __fdiv_rn(127.0f, absmax);
  }
  return p;
}

// std::round (nearest, ties away from zero) in three VALU operations: add the largest float
// below one half, with x's sign, and truncate. The sum is rounded to nearest even, and that
// rounding never carries a value across an integer: below a tie k + 0.5 the exact sum stays
// more than half an ulp under k + 1, and a tie's own sum k + 1 - 2^-25 is at most half an ulp
// under k + 1 (exactly half only at k = 0, where the even neighbour is 1.0). Adding 0.5
// itself would be wrong for the one float just below 0.5. Bit-identical to roundf on every
// float that is not a NaN (checked over all 2^32 bit patterns on the host).
__device__ __forceinline__ float RoundHalfAway(float x) {
  return truncf(__fadd_rn(x, copysignf(0x1.fffffep-2f, x)));
}

// The rounding used inside the NEON loops (neon_tensor_utils.cc:2347-2359).
template <int VARIANT>
__device__ __forceinline__ int32_t RoundToNearest(float x) {
  if (VARIANT == LRTFC_QUANT_NEON_LEGACY) {
    const float nudge = __fadd_rn(x < 0.0f ? -1.0f : 0.0f, 0.5f);
    return static_cast<int32_t>(__fadd_rn(x, nudge));  // truncation
  }
  return static_cast<int32_t>(RoundHalfAway(x));
}

// in_tail: the element belongs to the last n % 8 of the row, which the NEON builds
// finish with a scalar expression that rounds differently.
template <int VARIANT>
__device__ __forceinline__ int32_t QuantizeAsym(float v, float inv, int32_t zp, bool in_tail) {
  int32_t q;
  if (VARIANT == LRTFC_QUANT_PORTABLE) {
    // portable_tensor_utils.cc:112-118: float multiply, float add, then round half
    // away. An FMA here would change results.
    q = static_cast<int32_t>(RoundHalfAway(__fadd_rn(static_cast<float>(zp), __fmul_rn(v, inv))));
  } else if (in_tail) {
    q = static_cast<int32_t>(__fadd_rn(static_cast<float>(zp), RoundHalfAway(__fmul_rn(inv, v))));
  } else {
    q = RoundToNearest<VARIANT>(__fmul_rn(v, inv)) + zp;
  }
  return min(127, max(-128, q));
}

template <int VARIANT>
__device__ __forceinline__ int32_t QuantizeSym(float v, float inv, bool in_tail) {
  int32_t q;
  if (VARIANT == LRTFC_QUANT_PORTABLE || in_tail) {
    q = static_cast<int32_t>(RoundHalfAway(__fmul_rn(v, inv)));
  } else {
    q = RoundToNearest<VARIANT>(__fmul_rn(v, inv));
  }
  return min(127, max(-127, q));
}

// An all-zero row (scale 1, zero point 0, every value 0) needs no branch: callers pass
// inv = 0 for it (see ElementwiseInv), and round(0 + v * 0) is 0 for the finite zeros of such
// a row. With zero point 0 the asymmetric expression is also what the symmetric one computes,
// up to its clamp at -127, so one code path serves both.
template <int VARIANT>
__device__ __forceinline__ int32_t QuantizeElement(float v, const RowQuantParams& p,
                                                   bool asymmetric, bool in_tail) {
  const int32_t q = QuantizeAsym<VARIANT>(v, p.inv, p.zero_point, in_tail);
  return asymmetric ? q : max(q, -127);
}

// The quantized value of one element as an integral float, zero point included and not yet
// clamped: the same expressions as QuantizeAsym (adding the zero point to an integral float is
// exact, so the NEON forms' integer addition may happen in float).
template <int VARIANT>
__device__ __forceinline__ float QuantizedFloat(float v, float inv, float zp, bool in_tail) {
  if (VARIANT == LRTFC_QUANT_PORTABLE) {
    return RoundHalfAway(__fadd_rn(zp, __fmul_rn(v, inv)));
  }
  if (in_tail) return __fadd_rn(zp, RoundHalfAway(__fmul_rn(inv, v)));
  const float x = __fmul_rn(v, inv);
  if (VARIANT == LRTFC_QUANT_NEON_LEGACY) {
    const float nudge = __fadd_rn(x < 0.0f ? -1.0f : 0.0f, 0.5f);
    return __fadd_rn(truncf(__fadd_rn(x, nudge)), zp);
  }
  return __fadd_rn(RoundHalfAway(x), zp);
}

// Four elements quantized, clamped to [-128, 127] and packed little-endian into one dword.
// The clamp is the saturation of v_cvt_pk_u8_f32 on value + 128 (integral, so the
// instruction's own rounding never acts); flipping the four top bits afterwards takes the 128
// back out. A symmetric row (zero point 0, multiplier 127 / max|v|) cannot reach -128: every
// |v * inv| stays below 127.5, so its clamp at -127 never binds and needs no instruction.
template <int VARIANT>
__device__ __forceinline__ int32_t QuantizePack4(float a, float b, float c, float d,
                                                 const RowQuantParams& p, bool in_tail) {
  const float zp = static_cast<float>(p.zero_point);
  uint32_t w = 0;
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __fadd_rn(QuantizedFloat<VARIANT>(a, p.inv, zp, in_tail), 128.0f), 0, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __fadd_rn(QuantizedFloat<VARIANT>(b, p.inv, zp, in_tail), 128.0f), 1, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __fadd_rn(QuantizedFloat<VARIANT>(c, p.inv, zp, in_tail), 128.0f), 2, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(
      __fadd_rn(QuantizedFloat<VARIANT>(d, p.inv, zp, in_tail), 128.0f), 3, w);
  return static_cast<int32_t>(w ^ 0x80808080u);
}

// The multiplier the elementwise pass should use for a row.
__device__ __forceinline__ float ElementwiseInv(const RowQuantParams& p) {
  return p.all_zero ? 0.0f : p.inv;
}

// Four quantized values packed little-endian into one dword.
__device__ __forceinline__ int32_t PackBytes(int32_t a, int32_t b, int32_t c, int32_t d) {
  return (a & 0xFF) | ((b & 0xFF) << 8) | ((c & 0xFF) << 16) | (static_cast<uint32_t>(d) << 24);
}

// ---- one row by one workgroup (the standalone quantizer kernels) ------------------------

constexpr int kQuantizeThreads = 256;

struct RowRange {
  float mn;
  float mx;
};

// Rows deeper than kQuantizeDeepRow are given a workgroup of kQuantizeDeepThreads threads by the
// launchers: four loads, one row's worth of vector work per wavefront a quarter as long, where the
// narrow workgroup spends 7 us on a row of 16384 (one latency chain on one compute unit). Rows of
// 4096 are faster on the narrow one (0.4 us per launch at 9 to 128 rows).
constexpr int kQuantizeDeepThreads = 1024;
constexpr int kQuantizeDeepRow = 4096;

// Block-wide min and max. Every thread returns the same pair.
template <int THREADS = kQuantizeThreads>
__device__ __forceinline__ RowRange BlockMinMax(float mn, float mx) {
  __shared__ float s_min[THREADS / kWaveSize];
  __shared__ float s_max[THREADS / kWaveSize];
  mn = WaveMinF32(mn);
  mx = WaveMaxF32(mx);
  const int wave = threadIdx.x / kWaveSize;
  if ((threadIdx.x & (kWaveSize - 1)) == 0) {
    s_min[wave] = mn;
    s_max[wave] = mx;
  }
  __syncthreads();
  RowRange r{s_min[0], s_max[0]};
#pragma unroll
  for (int w = 1; w < THREADS / kWaveSize; ++w) {
    r.mn = fminf(r.mn, s_min[w]);
    r.mx = fmaxf(r.mx, s_max[w]);
  }
  return r;
}

// Where element i of a quantized row goes, as a byte offset from the row's base pointer.
// A placement keeps aligned groups of four elements together, in order.
struct RowMajorPlacement {
  __device__ __forceinline__ size_t operator()(int i) const { return static_cast<size_t>(i); }
};

// One row through BatchQuantizeFloats by one workgroup of THREADS threads: v[n_data]
// -> q[place(0 .. n_data-1)], *scaling_factor, *zero_point (may be null).
template <int VARIANT, typename PLACEMENT = RowMajorPlacement, int THREADS = kQuantizeThreads>
__device__ __forceinline__ void QuantizeRow(const float* __restrict__ v, int n_data,
                                            int8_t* __restrict__ q,
                                            float* __restrict__ scaling_factor,
                                            int32_t* __restrict__ zero_point, int do_asymmetric,
                                            PLACEMENT place = PLACEMENT()) {
  const bool vec_ok = (n_data % 4 == 0) && ((reinterpret_cast<uintptr_t>(v) & 15) == 0) &&
                      ((reinterpret_cast<uintptr_t>(q) & 3) == 0);
  // Rows and results are in global memory. Callers that read these pointers from a table in
  // memory hand them over without an address space, and accesses through such pointers would go
  // the flat path; so the address space is stated here.
  using Float4 = float __attribute__((ext_vector_type(4)));
  using GlobalF4 = const __attribute__((address_space(1))) Float4;
  using GlobalF = const __attribute__((address_space(1))) float;
  using GlobalI32 = __attribute__((address_space(1))) int32_t;
  using GlobalC = __attribute__((address_space(1))) int8_t;
  auto load4 = [](GlobalF4* at) {
    const Float4 r = *at;
    return make_float4(r.x, r.y, r.z, r.w);
  };
  GlobalF4* const gv4 = (GlobalF4*)v;
  GlobalF* const gv = (GlobalF*)v;
  GlobalC* const gq = (GlobalC*)q;

  // Pass 1: range of the row. Starting from 0 gives min(0, min v) / max(0, max v),
  // which is also what max(|min|, |max|) needs for the symmetric case.
  float mn = 0.0f, mx = 0.0f;
  // Rows of up to kRowRegs * THREADS * 4 values (16384) stay in registers between the
  // two passes instead of being read again, and all their loads are in flight at once: a deep
  // row read in a loop, twice, is a chain of memory latencies on the one workgroup that has it.
  // The loads of a row stand in ONE basic block (no test between them, or the compiler waits for
  // each before it issues the next); rows of up to 4096 values take a block of four.
  constexpr int kRowRegs = THREADS > 256 ? 4 : 16, kShortRegs = 4;
  const int n4 = n_data / 4;
  const bool in_regs = vec_ok && n4 <= kRowRegs * THREADS;
  const bool short_row = n4 <= kShortRegs * THREADS;
  float4 held[kRowRegs];
  if (in_regs) {
    GlobalF4* v4 = gv4;
    // Past the end: the row's last piece again (an unconditional load), then taken as zeros, which
    // the range (it always includes 0) does not notice.
    auto take = [&](int j) {
      const int i = threadIdx.x + j * THREADS;
      held[j] = load4(v4 + min(i, n4 - 1));
    };
    auto widen = [&](int j) {
      const int i = threadIdx.x + j * THREADS;
      const float4 t = i < n4 ? held[j] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
      mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
    };
    if (short_row) {
#pragma unroll
      for (int j = 0; j < kShortRegs; ++j) take(j);
#pragma unroll
      for (int j = 0; j < kShortRegs; ++j) widen(j);
    } else {
#pragma unroll
      for (int j = 0; j < kRowRegs; ++j) take(j);
#pragma unroll
      for (int j = 0; j < kRowRegs; ++j) widen(j);
    }
  } else if (vec_ok) {
    GlobalF4* v4 = gv4;
    for (int i = threadIdx.x; i < n_data / 4; i += THREADS) {
      const float4 t = load4(v4 + i);
      mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
      mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
    }
  } else {
    for (int i = threadIdx.x; i < n_data; i += THREADS) {
      mn = fminf(mn, gv[i]);
      mx = fmaxf(mx, gv[i]);
    }
  }
  const RowRange range = BlockMinMax<THREADS>(mn, mx);

  // Scale and zero point, every thread redundantly (a few dozen flops).
  const RowQuantParams qp = do_asymmetric ? AsymmetricRowParams<VARIANT>(range.mn, range.mx)
                                          : SymmetricRowParams(range.mn, range.mx);
  const float sf = qp.scale;
  const float inv = qp.inv;
  const int32_t zp = qp.zero_point;
  const bool all_zero = qp.all_zero;
  if (threadIdx.x == 0) {
    *(__attribute__((address_space(1))) float*)scaling_factor = sf;
    if (zero_point) *(__attribute__((address_space(1))) int32_t*)zero_point = zp;
  }

  // Pass 2: elementwise. The NEON builds process 8 floats per step and finish
  // the remaining n_data % 8 with a scalar expression that rounds differently.
  const int vector_end = n_data - (n_data % 8);
  // Elements 4 i .. 4 i + 3 of the row, given as t.
  auto emit4 = [&](int i, const float4& t) {
    int32_t word = 0;
    if (!all_zero) {
      const bool tail = 4 * i >= vector_end;
      if (do_asymmetric) {
        word = QuantizePack4<VARIANT>(t.x, t.y, t.z, t.w, qp, tail);
      } else {
        word = PackBytes(QuantizeSym<VARIANT>(t.x, inv, tail), QuantizeSym<VARIANT>(t.y, inv, tail),
                         QuantizeSym<VARIANT>(t.z, inv, tail), QuantizeSym<VARIANT>(t.w, inv, tail));
      }
    }
    *(GlobalI32*)(gq + place(4 * i)) = word;
  };
  if (in_regs) {
    if (short_row) {
#pragma unroll
      for (int j = 0; j < kShortRegs; ++j) {
        const int i = threadIdx.x + j * THREADS;
        if (i < n4) emit4(i, held[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < kRowRegs; ++j) {
        const int i = threadIdx.x + j * THREADS;
        if (i < n4) emit4(i, held[j]);
      }
    }
  } else if (vec_ok) {
    GlobalF4* v4 = gv4;
    for (int i = threadIdx.x; i < n_data / 4; i += THREADS) emit4(i, load4(v4 + i));
  } else {
    for (int i = threadIdx.x; i < n_data; i += THREADS) {
      int8_t o = 0;
      if (!all_zero) {
        const bool tail = i >= vector_end;
        o = static_cast<int8_t>(do_asymmetric ? QuantizeAsym<VARIANT>(gv[i], inv, zp, tail)
                                              : QuantizeSym<VARIANT>(gv[i], inv, tail));
      }
      gq[place(i)] = o;
    }
  }
}

}  // namespace lrtfc

#endif  // LITERT_AMD_CSRC_QUANTIZE_DEVICE_H_

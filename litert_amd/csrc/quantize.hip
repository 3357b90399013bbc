// Per-row activation quantization on the GPU with BatchQuantizeFloats semantics
// (tflite/kernels/internal/portable_tensor_utils.h:158-176): one workgroup per
// row, a min/max pass, the scale / zero-point derivation in double precision
// exactly as the CPU kernels do it, then the elementwise pass.
#include "kernels.h"

namespace lrtfc {
namespace {

constexpr int kThreads = 256;

struct RowRange {
  float mn;
  float mx;
};

// Block-wide min and max. Every thread returns the same pair.
__device__ __forceinline__ RowRange BlockMinMax(float mn, float mx) {
  __shared__ float s_min[kThreads / kWaveSize];
  __shared__ float s_max[kThreads / kWaveSize];
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
  for (int w = 1; w < kThreads / kWaveSize; ++w) {
    r.mn = fminf(r.mn, s_min[w]);
    r.mx = fmaxf(r.mx, s_max[w]);
  }
  return r;
}

// The rounding used inside the NEON loops
// (tflite/kernels/internal/optimized/neon_tensor_utils.cc:2347-2359).
template <int VARIANT>
__device__ __forceinline__ int32_t RoundToNearest(float x) {
  if (VARIANT == LRTFC_QUANT_NEON_LEGACY) {
    const float nudge = __fadd_rn(x < 0.0f ? -1.0f : 0.0f, 0.5f);
    return static_cast<int32_t>(__fadd_rn(x, nudge));  // truncation
  }
  return static_cast<int32_t>(roundf(x));
}

template <int VARIANT>
__device__ __forceinline__ int8_t QuantizeAsym(float v, float inv, int32_t zp, bool in_tail) {
  int32_t q;
  if (VARIANT == LRTFC_QUANT_PORTABLE) {
    // reference/portable_tensor_utils.cc:112-118: float multiply, float add,
    // then round half away. An FMA here would change results.
    q = static_cast<int32_t>(roundf(__fadd_rn(static_cast<float>(zp), __fmul_rn(v, inv))));
  } else if (in_tail) {
    // neon_tensor_utils.cc:2546-2551, scalar postamble.
    q = static_cast<int32_t>(__fadd_rn(static_cast<float>(zp), roundf(__fmul_rn(inv, v))));
  } else {
    q = RoundToNearest<VARIANT>(__fmul_rn(v, inv)) + zp;
  }
  return static_cast<int8_t>(min(127, max(-128, q)));
}

template <int VARIANT>
__device__ __forceinline__ int8_t QuantizeSym(float v, float inv, bool in_tail) {
  int32_t q;
  if (VARIANT == LRTFC_QUANT_PORTABLE || in_tail) {
    q = static_cast<int32_t>(roundf(__fmul_rn(v, inv)));
  } else {
    q = RoundToNearest<VARIANT>(__fmul_rn(v, inv));
  }
  return static_cast<int8_t>(min(127, max(-127, q)));
}

template <int VARIANT>
__global__ __launch_bounds__(kThreads) void BatchQuantizeKernel(
    const float* __restrict__ values, int n_data, int8_t* __restrict__ quantized,
    float* __restrict__ scaling_factors, int32_t* __restrict__ zero_points, int do_asymmetric) {
  const int row = blockIdx.x;
  const float* v = values + static_cast<size_t>(row) * n_data;
  int8_t* q = quantized + static_cast<size_t>(row) * n_data;
  const bool vec_ok = (n_data % 4 == 0) && ((reinterpret_cast<uintptr_t>(v) & 15) == 0) &&
                      ((reinterpret_cast<uintptr_t>(q) & 3) == 0);

  // Pass 1: range of the row. Starting from 0 gives min(0, min v) / max(0, max v),
  // which is also what max(|min|, |max|) needs for the symmetric case.
  float mn = 0.0f, mx = 0.0f;
  if (vec_ok) {
    const float4* v4 = reinterpret_cast<const float4*>(v);
    for (int i = threadIdx.x; i < n_data / 4; i += kThreads) {
      const float4 t = v4[i];
      mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
      mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
    }
  } else {
    for (int i = threadIdx.x; i < n_data; i += kThreads) {
      mn = fminf(mn, v[i]);
      mx = fmaxf(mx, v[i]);
    }
  }
  const RowRange range = BlockMinMax(mn, mx);

  // Scale and zero point, every thread redundantly (a few dozen flops).
  float sf;
  float inv;
  int32_t zp = 0;
  bool all_zero = false;
  if (do_asymmetric) {
    if (range.mn == range.mx) {
      all_zero = true;  // both are 0: memset, scale 1, offset 0
      sf = 1.0f;
      inv = 1.0f;
    } else {
      const double qmin = -128.0, qmax = 127.0;
      const double rmin = static_cast<double>(range.mn);
      const double rmax = static_cast<double>(range.mx);
      // Portable widens to double before subtracting
      // (reference/portable_tensor_utils.cc:81-87); the NEON build subtracts in
      // float (neon_tensor_utils.cc:2486).
      const double span = (VARIANT == LRTFC_QUANT_PORTABLE)
                              ? (rmax - rmin)
                              : static_cast<double>(__fsub_rn(range.mx, range.mn));
      const double scale = span / (qmax - qmin);
      const double zp_from_min = qmin - rmin / scale;
      const double zp_from_max = qmax - rmax / scale;
      const double err_from_min = fabs(qmin) + fabs(rmin / scale);
      const double err_from_max = fabs(qmax) + fabs(rmax / scale);
      const double zp_double = err_from_min < err_from_max ? zp_from_min : zp_from_max;
      if (zp_double <= qmin) {
        zp = -128;
      } else if (zp_double >= qmax) {
        zp = 127;
      } else {
        zp = static_cast<int8_t>(round(zp_double));
      }
      sf = static_cast<float>(scale);
      if (VARIANT == LRTFC_QUANT_PORTABLE) {
        inv = __fdiv_rn(1.0f, sf);
      } else {
        inv = sf == 0.0f ? 0.0f : static_cast<float>(1.0 / static_cast<double>(sf));
      }
    }
  } else {
    const float absmax = fmaxf(fabsf(range.mn), fabsf(range.mx));
    if (absmax == 0.0f) {
      all_zero = true;
      sf = 1.0f;
      inv = 1.0f;
    } else {
      sf = __fdiv_rn(absmax, 127.0f);
      inv = __fdiv_rn(127.0f, absmax);
    }
  }
  if (threadIdx.x == 0) {
    scaling_factors[row] = sf;
    if (zero_points) zero_points[row] = zp;
  }

  // Pass 2: elementwise. The NEON builds process 8 floats per step and finish
  // the remaining n_data % 8 with a scalar expression that rounds differently.
  const int vector_end = n_data - (n_data % 8);
  if (vec_ok) {
    const float4* v4 = reinterpret_cast<const float4*>(v);
    char4* q4 = reinterpret_cast<char4*>(q);
    for (int i = threadIdx.x; i < n_data / 4; i += kThreads) {
      char4 o;
      if (all_zero) {
        o = make_char4(0, 0, 0, 0);
      } else {
        const float4 t = v4[i];
        const bool tail = 4 * i >= vector_end;
        if (do_asymmetric) {
          o.x = QuantizeAsym<VARIANT>(t.x, inv, zp, tail);
          o.y = QuantizeAsym<VARIANT>(t.y, inv, zp, tail);
          o.z = QuantizeAsym<VARIANT>(t.z, inv, zp, tail);
          o.w = QuantizeAsym<VARIANT>(t.w, inv, zp, tail);
        } else {
          o.x = QuantizeSym<VARIANT>(t.x, inv, tail);
          o.y = QuantizeSym<VARIANT>(t.y, inv, tail);
          o.z = QuantizeSym<VARIANT>(t.z, inv, tail);
          o.w = QuantizeSym<VARIANT>(t.w, inv, tail);
        }
      }
      q4[i] = o;
    }
  } else {
    for (int i = threadIdx.x; i < n_data; i += kThreads) {
      int8_t o = 0;
      if (!all_zero) {
        const bool tail = i >= vector_end;
        o = do_asymmetric ? QuantizeAsym<VARIANT>(v[i], inv, zp, tail)
                          : QuantizeSym<VARIANT>(v[i], inv, tail);
      }
      q[i] = o;
    }
  }
}

}  // namespace

hipError_t LaunchBatchQuantize(const float* values, int n_batch, int n_data, int8_t* quantized,
                               float* scaling_factors, int32_t* zero_points, int do_asymmetric,
                               int variant, hipStream_t stream) {
  if (n_batch == 0 || n_data == 0) return hipSuccess;
  const dim3 grid(n_batch), block(kThreads);
  switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      hipLaunchKernelGGL(BatchQuantizeKernel<LRTFC_QUANT_NEON_V8>, grid, block, 0, stream, values,
                         n_data, quantized, scaling_factors, zero_points, do_asymmetric);
      break;
    case LRTFC_QUANT_NEON_LEGACY:
      hipLaunchKernelGGL(BatchQuantizeKernel<LRTFC_QUANT_NEON_LEGACY>, grid, block, 0, stream,
                         values, n_data, quantized, scaling_factors, zero_points, do_asymmetric);
      break;
    default:
      hipLaunchKernelGGL(BatchQuantizeKernel<LRTFC_QUANT_PORTABLE>, grid, block, 0, stream,
                         values, n_data, quantized, scaling_factors, zero_points, do_asymmetric);
      break;
  }
  return hipGetLastError();
}

}  // namespace lrtfc

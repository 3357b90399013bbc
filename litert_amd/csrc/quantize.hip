// Per-row activation quantization on the GPU with BatchQuantizeFloats semantics
// (tflite/kernels/internal/portable_tensor_utils.h:158-176): one workgroup per
// row, a min/max pass, the scale / zero-point derivation in double precision
// exactly as the CPU kernels do it, then the elementwise pass.
#include "kernels.h"
#include "quantize_device.h"

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
  const RowQuantParams qp = do_asymmetric ? AsymmetricRowParams<VARIANT>(range.mn, range.mx)
                                          : SymmetricRowParams(range.mn, range.mx);
  const float sf = qp.scale;
  const float inv = qp.inv;
  const int32_t zp = qp.zero_point;
  const bool all_zero = qp.all_zero;
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
          o.x = static_cast<char>(QuantizeAsym<VARIANT>(t.x, inv, zp, tail));
          o.y = static_cast<char>(QuantizeAsym<VARIANT>(t.y, inv, zp, tail));
          o.z = static_cast<char>(QuantizeAsym<VARIANT>(t.z, inv, zp, tail));
          o.w = static_cast<char>(QuantizeAsym<VARIANT>(t.w, inv, zp, tail));
        } else {
          o.x = static_cast<char>(QuantizeSym<VARIANT>(t.x, inv, tail));
          o.y = static_cast<char>(QuantizeSym<VARIANT>(t.y, inv, tail));
          o.z = static_cast<char>(QuantizeSym<VARIANT>(t.z, inv, tail));
          o.w = static_cast<char>(QuantizeSym<VARIANT>(t.w, inv, tail));
        }
      }
      q4[i] = o;
    }
  } else {
    for (int i = threadIdx.x; i < n_data; i += kThreads) {
      int8_t o = 0;
      if (!all_zero) {
        const bool tail = i >= vector_end;
        o = static_cast<int8_t>(do_asymmetric ? QuantizeAsym<VARIANT>(v[i], inv, zp, tail)
                                              : QuantizeSym<VARIANT>(v[i], inv, tail));
      }
      q[i] = o;
    }
  }
}

// The row quantizer of the per-channel int4 hybrid path (ReferenceBatchQuantizeFloats4Bit,
// tflite/kernels/internal/optimized/4bit/fully_connected_reference.cc:121-180): symmetric,
// scale_denom = max|x| (127 for an all-zero row), multiplier 127.0 / scale_denom and stored
// scale scale_denom / 127.0 both divided in double and rounded to float, q = (int8)round(x *
// multiplier) without a clamp, and input_offsets = sum(q) * zero_point_4bit (-7).
__global__ __launch_bounds__(kThreads) void BatchQuantize4BitKernel(
    const float* __restrict__ values, int n_data, int8_t* __restrict__ quantized,
    float* __restrict__ scaling_factors, int32_t* __restrict__ input_offsets) {
  __shared__ int32_t s_sum[kThreads / kWaveSize];
  const int row = blockIdx.x;
  const float* v = values + static_cast<size_t>(row) * n_data;
  int8_t* q = quantized + static_cast<size_t>(row) * n_data;
  float mn = 0.0f, mx = 0.0f;
  for (int i = threadIdx.x; i < n_data; i += kThreads) {
    mn = fminf(mn, v[i]);
    mx = fmaxf(mx, v[i]);
  }
  const RowRange range = BlockMinMax(mn, mx);
  float scale_denom = fmaxf(fabsf(range.mn), fabsf(range.mx));
  if (scale_denom == 0.0f) scale_denom = 127.0f;
  const float multiplier = static_cast<float>(127.0 / static_cast<double>(scale_denom));
  int32_t sum = 0;
  for (int i = threadIdx.x; i < n_data; i += kThreads) {
    const int32_t o = static_cast<int8_t>(RoundHalfAway(__fmul_rn(v[i], multiplier)));
    q[i] = static_cast<int8_t>(o);
    sum += o;
  }
  sum = WaveSumI32(sum);
  if ((threadIdx.x & (kWaveSize - 1)) == 0) s_sum[threadIdx.x / kWaveSize] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t total = 0;
#pragma unroll
    for (int w = 0; w < kThreads / kWaveSize; ++w) total += s_sum[w];
    scaling_factors[row] = static_cast<float>(static_cast<double>(scale_denom) / 127.0);
    input_offsets[row] = total * -7;
  }
}

}  // namespace

hipError_t LaunchBatchQuantize4Bit(const float* values, int n_batch, int n_data, int8_t* quantized,
                                   float* scaling_factors, int32_t* input_offsets,
                                   hipStream_t stream) {
  if (n_batch == 0 || n_data == 0) return hipSuccess;
  hipLaunchKernelGGL(BatchQuantize4BitKernel, dim3(n_batch), dim3(kThreads), 0, stream, values,
                     n_data, quantized, scaling_factors, input_offsets);
  return hipGetLastError();
}

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

// Per-row activation quantization on the GPU with BatchQuantizeFloats semantics
// (tflite/kernels/internal/portable_tensor_utils.h:158-176): one workgroup per
// row, a min/max pass, the scale / zero-point derivation in double precision
// exactly as the CPU kernels do it, then the elementwise pass.
#include "kernels.h"
#include "quantize_device.h"

namespace lrtfc {
namespace {

constexpr int kThreads = kQuantizeThreads;

template <int VARIANT, int THREADS = kThreads>
__global__ __launch_bounds__(THREADS) void BatchQuantizeKernel(
    const float* __restrict__ values, int n_data, int8_t* __restrict__ quantized,
    float* __restrict__ scaling_factors, int32_t* __restrict__ zero_points, int do_asymmetric) {
  const int row = blockIdx.x;
  QuantizeRow<VARIANT, RowMajorPlacement, THREADS>(
      values + static_cast<size_t>(row) * n_data, n_data,
      quantized + static_cast<size_t>(row) * n_data, scaling_factors + row,
      zero_points ? zero_points + row : nullptr, do_asymmetric);
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

// BATCH_MATMUL with adj_x: the op transposes the last two dimensions of its left operand into a
// temporary before anything else (TransposeRowsColumns, tflite/kernels/batch_matmul.cc:811-813).
// Per matrix, src [in_rows, in_cols] -> dst [in_cols, in_rows], through a 32 x 32 tile in LDS so
// that reads and writes both run along rows (one padding column keeps the transposed reads off
// a single bank).
constexpr int kTransposeTile = 32;
__global__ __launch_bounds__(kTransposeTile * 8) void TransposeLastTwoF32Kernel(
    const float* __restrict__ src, int in_rows, int in_cols, float* __restrict__ dst) {
  __shared__ float tile[kTransposeTile][kTransposeTile + 1];
  const size_t matrix = static_cast<size_t>(blockIdx.z) * in_rows * in_cols;
  const int c0 = blockIdx.x * kTransposeTile, r0 = blockIdx.y * kTransposeTile;
  const int tx = threadIdx.x & (kTransposeTile - 1), ty = threadIdx.x / kTransposeTile;
  for (int j = ty; j < kTransposeTile; j += 8) {
    const int r = r0 + j, c = c0 + tx;
    if (r < in_rows && c < in_cols) tile[j][tx] = src[matrix + static_cast<size_t>(r) * in_cols + c];
  }
  __syncthreads();
  for (int j = ty; j < kTransposeTile; j += 8) {
    const int c = c0 + j, r = r0 + tx;  // dst row = source column
    if (r < in_rows && c < in_cols) dst[matrix + static_cast<size_t>(c) * in_rows + r] = tile[tx][j];
  }
}

}  // namespace

hipError_t LaunchTransposeLastTwoF32(const float* src, int matrices, int in_rows, int in_cols,
                                     float* dst, hipStream_t stream) {
  if (matrices == 0 || in_rows == 0 || in_cols == 0) return hipSuccess;
  if (matrices > 65535) return hipErrorInvalidValue;
  const dim3 grid((in_cols + kTransposeTile - 1) / kTransposeTile,
                  (in_rows + kTransposeTile - 1) / kTransposeTile, matrices);
  if (grid.y > 65535) return hipErrorInvalidValue;
  hipLaunchKernelGGL(TransposeLastTwoF32Kernel, grid, dim3(kTransposeTile * 8), 0, stream, src,
                     in_rows, in_cols, dst);
  return hipGetLastError();
}

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
  const dim3 grid(n_batch);
  const bool deep = n_data > kQuantizeDeepRow;
  auto launch = [&](auto narrow, auto wide) {
    if (deep) {
      hipLaunchKernelGGL(wide, grid, dim3(kQuantizeDeepThreads), 0, stream, values, n_data, quantized,
                         scaling_factors, zero_points, do_asymmetric);
    } else {
      hipLaunchKernelGGL(narrow, grid, dim3(kThreads), 0, stream, values, n_data, quantized,
                         scaling_factors, zero_points, do_asymmetric);
    }
  };
  switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      launch(BatchQuantizeKernel<LRTFC_QUANT_NEON_V8>,
             BatchQuantizeKernel<LRTFC_QUANT_NEON_V8, kQuantizeDeepThreads>);
      break;
    case LRTFC_QUANT_NEON_LEGACY:
      launch(BatchQuantizeKernel<LRTFC_QUANT_NEON_LEGACY>,
             BatchQuantizeKernel<LRTFC_QUANT_NEON_LEGACY, kQuantizeDeepThreads>);
      break;
    default:
      launch(BatchQuantizeKernel<LRTFC_QUANT_PORTABLE>,
             BatchQuantizeKernel<LRTFC_QUANT_PORTABLE, kQuantizeDeepThreads>);
      break;
  }
  return hipGetLastError();
}

}  // namespace lrtfc

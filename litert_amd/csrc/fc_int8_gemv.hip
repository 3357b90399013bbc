// Decode-regime FULLY_CONNECTED with int8 weights: a bandwidth-bound GEMV.
//
// Layout: filter [out_depth, depth] row-major int8, read exactly once per call
// with 128-bit loads (one wavefront covers 1 KiB of a filter row per load
// instruction); the activation rows of the batch tile are staged once per
// workgroup in LDS and re-read from there for every filter row. Each wavefront
// owns R filter rows per pass and keeps R x BT int32 accumulators; lanes split
// the depth, so a wave64 butterfly finishes each dot product. Integer sums are
// exact, so any summation order gives the reference's accumulator; only the
// epilogues below have an order that matters.
#include "fc_epilogues.h"
#include "kernels.h"

namespace lrtfc {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / kWaveSize;

template <int R, int BT, Int8Epilogue EPI, bool FILTER_OFFSET>
__global__ __launch_bounds__(kThreads) void FcInt8GemvKernel(FcInt8Args a, int batch0) {
  extern __shared__ i32x4 lds_q[];  // [BT][depth / 16]
  const int kvec = a.depth / 16;
  for (int i = threadIdx.x; i < BT * kvec; i += kThreads) {
    const int b = i / kvec;
    const int j = i - b * kvec;
    const int bb = batch0 + b;
    i32x4 v = {0, 0, 0, 0};
    if (bb < a.batches) {
      v = reinterpret_cast<const i32x4*>(a.input + static_cast<size_t>(bb) * a.depth)[j];
    }
    lds_q[i] = v;
  }
  __syncthreads();

  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int num_passes = (a.out_depth + R - 1) / R;
  for (int pass = blockIdx.x * kWavesPerBlock + wave; pass < num_passes;
       pass += gridDim.x * kWavesPerBlock) {
    const int n0 = pass * R;
    int32_t acc[R][BT];
    int32_t xsum[BT];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int b = 0; b < BT; ++b) acc[r][b] = 0;
    }
#pragma unroll
    for (int b = 0; b < BT; ++b) xsum[b] = 0;

    const i32x4* rows[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = min(n0 + r, a.out_depth - 1);  // clamped rows are computed and dropped
      rows[r] = reinterpret_cast<const i32x4*>(a.filter + static_cast<size_t>(n) * a.depth);
    }

#pragma unroll 2
    for (int j = lane; j < kvec; j += kWaveSize) {
      i32x4 wv[R];
#pragma unroll
      for (int r = 0; r < R; ++r) wv[r] = __builtin_nontemporal_load(rows[r] + j);
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        const i32x4 qv = lds_q[b * kvec + j];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          int32_t t = acc[r][b];
          t = Dot4(wv[r].x, qv.x, t);
          t = Dot4(wv[r].y, qv.y, t);
          t = Dot4(wv[r].z, qv.z, t);
          t = Dot4(wv[r].w, qv.w, t);
          acc[r][b] = t;
        }
        if (FILTER_OFFSET) {
          int32_t t = xsum[b];
          t = Dot4(qv.x, 0x01010101, t);
          t = Dot4(qv.y, 0x01010101, t);
          t = Dot4(qv.z, 0x01010101, t);
          t = Dot4(qv.w, 0x01010101, t);
          xsum[b] = t;
        }
      }
    }

    // Finish the dot products across lanes; lane r * BT + b keeps (row r, batch b).
    int32_t mine = 0, mine_xsum = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        const int32_t total = WaveSumI32(acc[r][b]);
        if (lane == r * BT + b) mine = total;
      }
    }
    if (FILTER_OFFSET) {
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        const int32_t total = WaveSumI32(xsum[b]);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (lane == r * BT + b) mine_xsum = total;
        }
      }
    }
    if (lane < R * BT) {
      const int r = lane / BT;
      const int b = batch0 + (lane - r * BT);
      const int n = n0 + r;
      if (n < a.out_depth && b < a.batches) {
        if (EPI == Int8Epilogue::kRequantize) {
          StoreRequantized(a, b, n, mine, mine_xsum);
        } else {
          StoreHybrid(a, b, n, mine, a.scaling_factors[b], a.zero_points ? a.zero_points[b] : 0);
        }
      }
    }
  }
}

// Any shape, any alignment: one thread per output element. Used for shapes the
// vector kernel cannot take (depth not a multiple of 16, unaligned pointers).
template <Int8Epilogue EPI>
__global__ __launch_bounds__(kThreads) void FcInt8GenericKernel(FcInt8Args a) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= static_cast<int64_t>(a.batches) * a.out_depth) return;
  const int b = static_cast<int>(idx / a.out_depth);
  const int n = static_cast<int>(idx - static_cast<int64_t>(b) * a.out_depth);
  const int8_t* w = a.filter + static_cast<size_t>(n) * a.depth;
  const int8_t* x = a.input + static_cast<size_t>(b) * a.depth;
  int32_t dot = 0, xsum = 0;
  for (int k = 0; k < a.depth; ++k) {
    dot += static_cast<int32_t>(w[k]) * static_cast<int32_t>(x[k]);
    xsum += x[k];
  }
  if (EPI == Int8Epilogue::kRequantize) {
    StoreRequantized(a, b, n, dot, xsum);
  } else {
    StoreHybrid(a, b, n, dot, a.scaling_factors[b], a.zero_points ? a.zero_points[b] : 0);
  }
}

__global__ __launch_bounds__(kThreads) void RowSumsInt8Kernel(const int8_t* __restrict__ filter,
                                                              int out_depth, int depth,
                                                              int32_t* __restrict__ row_sums) {
  // one wavefront per row
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int row = blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
  if (row >= out_depth) return;
  const int8_t* w = filter + static_cast<size_t>(row) * depth;
  int32_t s = 0;
  if (depth % 16 == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
    const i32x4* w4 = reinterpret_cast<const i32x4*>(w);
    for (int j = lane; j < depth / 16; j += kWaveSize) {
      const i32x4 v = w4[j];
      s = Dot4(v.x, 0x01010101, s);
      s = Dot4(v.y, 0x01010101, s);
      s = Dot4(v.z, 0x01010101, s);
      s = Dot4(v.w, 0x01010101, s);
    }
  } else {
    for (int k = lane; k < depth; k += kWaveSize) s += w[k];
  }
  s = WaveSumI32(s);
  if (lane == 0) row_sums[row] = s;
}

__global__ __launch_bounds__(kThreads) void UnpackInt4Kernel(const uint8_t* __restrict__ packed,
                                                             int64_t num_elements,
                                                             int8_t* __restrict__ unpacked) {
  // tflite/kernels/internal/portable_tensor_utils.cc:96-127: element 2i is the
  // low nibble of byte i, element 2i+1 the high nibble, both sign-extended.
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t num_bytes = (num_elements + 1) / 2;
  if (i >= num_bytes) return;
  const int8_t byte = static_cast<int8_t>(packed[i]);
  unpacked[2 * i] = static_cast<int8_t>(static_cast<int8_t>(byte << 4) >> 4);
  if (2 * i + 1 < num_elements) unpacked[2 * i + 1] = static_cast<int8_t>(byte >> 4);
}

__global__ __launch_bounds__(kThreads) void UnpackInt2Kernel(const uint8_t* __restrict__ packed,
                                                             int64_t num_elements,
                                                             int8_t* __restrict__ unpacked) {
  // tflite/kernels/internal/portable_tensor_utils.cc:128-163: element 4i + k is field k of byte
  // i (bits 2k, 2k + 1), sign-extended; a last partial byte gives num_elements % 4 elements.
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t num_bytes = (num_elements + 3) / 4;
  if (i >= num_bytes) return;
  const uint32_t byte = packed[i];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int8_t value =
        static_cast<int8_t>(static_cast<int8_t>((byte << (6 - 2 * k)) & 0xFF) >> 6);
    if (4 * i + k < num_elements) unpacked[4 * i + k] = value;
  }
}

// uint8 <-> int8 as a change of representation: value - 128 one way, value + 128 the other, both
// the same flip of the top bit. 16 bytes per thread where the pointers allow it.
__global__ __launch_bounds__(kThreads) void XorSignBitKernel(const uint8_t* __restrict__ src,
                                                             uint8_t* __restrict__ dst,
                                                             size_t bytes, bool vectors) {
  const size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (vectors) {
    const size_t at = i * 16;
    if (at + 16 <= bytes) {
      i32x4 v = *reinterpret_cast<const i32x4*>(src + at);
      const int32_t flip = static_cast<int32_t>(0x80808080u);
      v = i32x4{v[0] ^ flip, v[1] ^ flip, v[2] ^ flip, v[3] ^ flip};
      *reinterpret_cast<i32x4*>(dst + at) = v;
    } else {
      for (size_t j = at; j < bytes; ++j) dst[j] = src[j] ^ 0x80;
    }
  } else if (i < bytes) {
    dst[i] = src[i] ^ 0x80;
  }
}

__global__ __launch_bounds__(kThreads) void ZeroFillKernel(uint8_t* __restrict__ dst, size_t bytes) {
  const size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < bytes) dst[i] = 0;
}

template <int R, int BT>
hipError_t LaunchVariant(const FcInt8Args& a, Int8Epilogue epilogue, int batch0, int grid,
                         size_t lds_bytes, hipStream_t stream) {
  const dim3 g(grid), blk(kThreads);
  if (epilogue == Int8Epilogue::kHybrid) {
    hipLaunchKernelGGL((FcInt8GemvKernel<R, BT, Int8Epilogue::kHybrid, false>), g, blk, lds_bytes,
                       stream, a, batch0);
  } else if (a.filter_offset != 0) {
    hipLaunchKernelGGL((FcInt8GemvKernel<R, BT, Int8Epilogue::kRequantize, true>), g, blk,
                       lds_bytes, stream, a, batch0);
  } else {
    hipLaunchKernelGGL((FcInt8GemvKernel<R, BT, Int8Epilogue::kRequantize, false>), g, blk,
                       lds_bytes, stream, a, batch0);
  }
  return hipGetLastError();
}

template <int BT>
hipError_t LaunchForBatchTile(const FcInt8Args& a, Int8Epilogue epilogue, int batch0,
                              hipStream_t stream) {
  const size_t lds_bytes = static_cast<size_t>(BT) * a.depth;
  // Enough wavefronts to cover the chip several times over; fewer rows per pass
  // when the filter is short.
  constexpr int kTargetWaves = 256 * 8;
  if (a.out_depth >= 4 * kTargetWaves) {
    const int passes = (a.out_depth + 3) / 4;
    const int grid = min((passes + kWavesPerBlock - 1) / kWavesPerBlock, 4096);
    return LaunchVariant<4, BT>(a, epilogue, batch0, grid, lds_bytes, stream);
  }
  if (a.out_depth >= 2 * kTargetWaves) {
    const int passes = (a.out_depth + 1) / 2;
    const int grid = min((passes + kWavesPerBlock - 1) / kWavesPerBlock, 4096);
    return LaunchVariant<2, BT>(a, epilogue, batch0, grid, lds_bytes, stream);
  }
  const int grid = min((a.out_depth + kWavesPerBlock - 1) / kWavesPerBlock, 4096);
  return LaunchVariant<1, BT>(a, epilogue, batch0, grid, lds_bytes, stream);
}

}  // namespace

hipError_t LaunchZeroFill(void* dst, size_t bytes, hipStream_t stream) {
  // A kernel rather than hipMemsetAsync, so that a caller may capture it in a graph.
  if (bytes == 0) return hipSuccess;
  const size_t grid = (bytes + kThreads - 1) / kThreads;
  hipLaunchKernelGGL(ZeroFillKernel, dim3(static_cast<unsigned>(grid)), dim3(kThreads), 0, stream,
                     static_cast<uint8_t*>(dst), bytes);
  return hipGetLastError();
}

hipError_t LaunchRowSumsInt8(const int8_t* filter, int out_depth, int depth, int32_t* row_sums,
                             hipStream_t stream) {
  if (out_depth == 0) return hipSuccess;
  const int grid = (out_depth + kWavesPerBlock - 1) / kWavesPerBlock;
  hipLaunchKernelGGL(RowSumsInt8Kernel, dim3(grid), dim3(kThreads), 0, stream, filter, out_depth,
                     depth, row_sums);
  return hipGetLastError();
}

hipError_t LaunchUnpackInt4(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                            hipStream_t stream) {
  if (num_elements == 0) return hipSuccess;
  const int64_t num_bytes = (num_elements + 1) / 2;
  const int grid = static_cast<int>((num_bytes + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(UnpackInt4Kernel, dim3(grid), dim3(kThreads), 0, stream, packed, num_elements,
                     unpacked);
  return hipGetLastError();
}

hipError_t LaunchXorSignBit(const uint8_t* src, uint8_t* dst, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  const bool vectors = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
  const size_t threads = vectors ? (bytes + 15) / 16 : bytes;
  const size_t grid = (threads + kThreads - 1) / kThreads;
  if (grid > 0x7fffffffull) return hipErrorInvalidValue;
  hipLaunchKernelGGL(XorSignBitKernel, dim3(static_cast<unsigned>(grid)), dim3(kThreads), 0, stream,
                     src, dst, bytes, vectors);
  return hipGetLastError();
}

hipError_t LaunchUnpackInt2(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                            hipStream_t stream) {
  if (num_elements == 0) return hipSuccess;
  const int64_t num_bytes = (num_elements + 3) / 4;
  const int grid = static_cast<int>((num_bytes + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(UnpackInt2Kernel, dim3(grid), dim3(kThreads), 0, stream, packed, num_elements,
                     unpacked);
  return hipGetLastError();
}

hipError_t LaunchFcInt8Gemv(const FcInt8Args& a, Int8Epilogue epilogue, hipStream_t stream) {
  if (a.batches == 0 || a.out_depth == 0) return hipSuccess;
  const bool aligned = (a.depth % 16 == 0) && a.depth > 0 &&
                       ((reinterpret_cast<uintptr_t>(a.filter) & 15) == 0) &&
                       ((reinterpret_cast<uintptr_t>(a.input) & 15) == 0);
  constexpr size_t kMaxLds = 64 * 1024;
  if (!aligned || static_cast<size_t>(a.depth) > kMaxLds) {
    const int64_t total = static_cast<int64_t>(a.batches) * a.out_depth;
    const int grid = static_cast<int>((total + kThreads - 1) / kThreads);
    if (epilogue == Int8Epilogue::kHybrid) {
      hipLaunchKernelGGL(FcInt8GenericKernel<Int8Epilogue::kHybrid>, dim3(grid), dim3(kThreads), 0,
                         stream, a);
    } else {
      hipLaunchKernelGGL(FcInt8GenericKernel<Int8Epilogue::kRequantize>, dim3(grid),
                         dim3(kThreads), 0, stream, a);
    }
    return hipGetLastError();
  }
  // Walk the batch in tiles of up to 8 rows that fit in LDS; each tile streams the
  // filter once.
  int batch0 = 0;
  while (batch0 < a.batches) {
    const int left = a.batches - batch0;
    int bt = left >= 8 ? 8 : left >= 4 ? 4 : left >= 2 ? 2 : 1;
    while (static_cast<size_t>(bt) * a.depth > kMaxLds) bt /= 2;
    hipError_t err;
    switch (bt) {
      case 8:
        err = LaunchForBatchTile<8>(a, epilogue, batch0, stream);
        break;
      case 4:
        err = LaunchForBatchTile<4>(a, epilogue, batch0, stream);
        break;
      case 2:
        err = LaunchForBatchTile<2>(a, epilogue, batch0, stream);
        break;
      default:
        err = LaunchForBatchTile<1>(a, epilogue, batch0, stream);
        break;
    }
    if (err != hipSuccess) return err;
    batch0 += bt;
  }
  return hipSuccess;
}

}  // namespace lrtfc

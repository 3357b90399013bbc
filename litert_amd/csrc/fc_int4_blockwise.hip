// Blockwise-int4-weight FULLY_CONNECTED (EvalBlockwise4Bit semantics,
// tflite/kernels/fully_connected.cc:1014-1086) as a bandwidth-bound GEMV.
//
// Layout in HBM is the reference's: each filter row is depth/2 bytes, two signed
// nibbles per byte with the even k in the low nibble; scales are fp16
// [out_depth, depth/blocksize]. With blocksize 32 one block of one row is exactly
// 16 bytes, i.e. one 128-bit load: lane L of a wavefront owns block (64*c + L) of
// a row, so one load instruction covers 1 KiB of the row and the lane finishes
// that block's int32 sum on its own (8 dot4, no cross-lane traffic).
//
// The reference then adds float(block_sum) * scale over the blocks of a row in
// block order, in float32. Float addition is not associative, so the products
// are parked in LDS and one lane per (row, batch) walks them in order; that
// chain is the only sequential part and runs while other workgroups stream.
//
// Signed nibbles are not sign-extended: (nibble ^ 8) = w + 8 is a small positive
// byte, so sum(w * q) = dot4(nibble ^ 8, q) - 8 * sum(q), with sum(q) per block
// computed once per activation block.
#include "kernels.h"

namespace lrtfc {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWaveSize;
constexpr int kBlock = 32;  // weights per quantization block on the fast path

__device__ __forceinline__ int PStride(int nblk) { return nblk | 1; }

template <int R, int BT, int WC>
__global__ __launch_bounds__(kThreads) void FcBlockwiseInt4Kernel(FcInt4Args a, int batch0) {
  constexpr int WR = kWaves / WC;  // waves splitting the rows
  constexpr int RW = R / WR;       // rows per wave
  static_assert(R % WR == 0, "rows must divide over the row-splitting waves");
  extern __shared__ int32_t lds[];
  const int depth = a.depth;
  const int nblk = depth / kBlock;
  const int qdw = depth / 4;  // dwords of quantized activations per batch row
  int32_t* q_lds = lds;       // [BT][qdw], each group of 8 k stored as (even k, odd k)
  float* p_lds = reinterpret_cast<float*>(lds + BT * qdw);  // [R * BT][PStride(nblk)]
  const int pstride = PStride(nblk);

  // Stage the batch tile's activations: 8 consecutive int8 per step, split into
  // the four even-k bytes and the four odd-k bytes to line up with the nibbles.
  for (int i = threadIdx.x; i < BT * (depth / 8); i += kThreads) {
    const int b = i / (depth / 8);
    const int g = i - b * (depth / 8);
    const int bb = batch0 + b;
    uint32_t lo = 0, hi = 0;
    if (bb < a.batches) {
      const i32x2 v = reinterpret_cast<const i32x2*>(a.input + static_cast<size_t>(bb) * depth)[g];
      lo = static_cast<uint32_t>(v.x);
      hi = static_cast<uint32_t>(v.y);
    }
    const uint32_t even = (lo & 0xFFu) | ((lo >> 8) & 0xFF00u) | ((hi & 0xFFu) << 16) |
                          ((hi << 8) & 0xFF000000u);
    const uint32_t odd = ((lo >> 8) & 0xFFu) | ((lo >> 16) & 0xFF00u) | ((hi << 8) & 0xFF0000u) |
                         (hi & 0xFF000000u);
    q_lds[b * qdw + 2 * g] = static_cast<int32_t>(even);
    q_lds[b * qdw + 2 * g + 1] = static_cast<int32_t>(odd);
  }
  __syncthreads();

  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int wc = wave % WC;
  const int wr = wave / WC;
  const int n0 = blockIdx.x * R;
  const size_t row_bytes = static_cast<size_t>(depth) / 2;

  for (int c = wc; c * kWaveSize < nblk; c += WC) {
    const int blk = c * kWaveSize + lane;
    if (blk < nblk) {
      // Issue every global load of this step before any arithmetic.
      i32x4 wv[RW];
      uint16_t sc[RW];
#pragma unroll
      for (int i = 0; i < RW; ++i) {
        const int n = min(n0 + wr * RW + i, a.out_depth - 1);
        wv[i] = __builtin_nontemporal_load(
            reinterpret_cast<const i32x4*>(a.packed_filter + n * row_bytes) + blk);
        sc[i] = __builtin_nontemporal_load(a.scales_f16 + static_cast<size_t>(n) * nblk + blk);
      }
      i32x4 qe[BT], qo[BT];  // qe/qo: dwords (e0,o0,e1,o1) and (e2,o2,e3,o3)
      int32_t qsum8[BT];
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        const i32x4* qp = reinterpret_cast<const i32x4*>(q_lds + b * qdw + blk * 8);
        qe[b] = qp[0];
        qo[b] = qp[1];
        int32_t s = 0;
        s = Dot4(qe[b].x, 0x01010101, s);
        s = Dot4(qe[b].y, 0x01010101, s);
        s = Dot4(qe[b].z, 0x01010101, s);
        s = Dot4(qe[b].w, 0x01010101, s);
        s = Dot4(qo[b].x, 0x01010101, s);
        s = Dot4(qo[b].y, 0x01010101, s);
        s = Dot4(qo[b].z, 0x01010101, s);
        s = Dot4(qo[b].w, 0x01010101, s);
        qsum8[b] = 8 * s;
      }
#pragma unroll
      for (int i = 0; i < RW; ++i) {
        const float scale = HalfBitsToFloat(sc[i]);
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t wx = static_cast<uint32_t>(wv[i][d]) ^ 0x88888888u;
          lo[d] = wx & 0x0F0F0F0Fu;
          hi[d] = (wx >> 4) & 0x0F0F0F0Fu;
        }
        const int r = wr * RW + i;
#pragma unroll
        for (int b = 0; b < BT; ++b) {
          int32_t acc = -qsum8[b];
          acc = Dot4(lo[0], qe[b].x, acc);
          acc = Dot4(hi[0], qe[b].y, acc);
          acc = Dot4(lo[1], qe[b].z, acc);
          acc = Dot4(hi[1], qe[b].w, acc);
          acc = Dot4(lo[2], qo[b].x, acc);
          acc = Dot4(hi[2], qo[b].y, acc);
          acc = Dot4(lo[3], qo[b].z, acc);
          acc = Dot4(hi[3], qo[b].w, acc);
          p_lds[(r * BT + b) * pstride + blk] = __fmul_rn(static_cast<float>(acc), scale);
        }
      }
    }
  }
  __syncthreads();

  // Ordered float32 accumulation over blocks, one lane per (row, batch), spread
  // over the four wavefronts.
  const int item = lane * kWaves + wave;
  if (item < R * BT) {
    const int r = item / BT;
    const int b = item - r * BT;
    const int n = n0 + r;
    const int bb = batch0 + b;
    if (n < a.out_depth && bb < a.batches) {
      const float* p = p_lds + item * pstride;
      float out = 0.0f;
      for (int j = 0; j < nblk; ++j) out = __fadd_rn(out, p[j]);
      // fully_connected.cc:1078-1082
      out = __fsub_rn(out, __fmul_rn(static_cast<float>(a.zero_points[bb]), a.kfsum[n]));
      out = __fmul_rn(out, a.scaling_factors[bb]);
      if (a.bias) out = __fadd_rn(out, a.bias[n]);
      a.output[static_cast<size_t>(bb) * a.out_depth + n] = out;
    }
  }
}

__device__ __forceinline__ int32_t NibbleAt(const uint8_t* row, int k) {
  const uint8_t byte = row[k >> 1];
  const int nib = (k & 1) ? (byte >> 4) : (byte & 0xF);
  return (nib ^ 8) - 8;
}

// Any block size: one thread per output element, everything in source order.
__global__ __launch_bounds__(kThreads) void FcBlockwiseInt4GenericKernel(FcInt4Args a) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= static_cast<int64_t>(a.batches) * a.out_depth) return;
  const int m = static_cast<int>(idx / a.out_depth);
  const int n = static_cast<int>(idx - static_cast<int64_t>(m) * a.out_depth);
  const int nblk = a.depth / a.blocksize;
  const size_t k2 = (static_cast<size_t>(a.depth) + 1) & ~static_cast<size_t>(1);
  const uint8_t* row = a.packed_filter + n * (k2 / 2);
  const int8_t* q = a.input + static_cast<size_t>(m) * a.depth;
  float out = 0.0f;
  for (int bi = 0; bi < nblk; ++bi) {
    int32_t acc = 0;
    for (int ki = 0; ki < a.blocksize; ++ki) {
      const int k = bi * a.blocksize + ki;
      acc += static_cast<int32_t>(q[k]) * NibbleAt(row, k);
    }
    const float scale = HalfBitsToFloat(a.scales_f16[static_cast<size_t>(n) * nblk + bi]);
    out = __fadd_rn(out, __fmul_rn(static_cast<float>(acc), scale));
  }
  out = __fsub_rn(out, __fmul_rn(static_cast<float>(a.zero_points[m]), a.kfsum[n]));
  out = __fmul_rn(out, a.scaling_factors[m]);
  if (a.bias) out = __fadd_rn(out, a.bias[n]);
  a.output[idx] = out;
}

// kfsum[n] = sum over blocks, in block order, of scale * float(sum of the block's weights)
// (tflite/kernels/fully_connected.cc:1056-1077). One wavefront per channel: lane L forms the
// products of blocks L, L + 64, ... in parallel, and the products are then added one by one in
// block order (each read out of its lane as a scalar), which is the order the result depends on.
__global__ __launch_bounds__(kThreads) void BlockwiseInt4KfsumKernel(
    const uint8_t* __restrict__ packed_filter, const uint16_t* __restrict__ scales_f16,
    int out_depth, int depth, int blocksize, float* __restrict__ kfsum) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int n = blockIdx.x * (kThreads / kWaveSize) +
                __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
  if (n >= out_depth) return;
  const int nblk = depth / blocksize;
  const size_t k2 = (static_cast<size_t>(depth) + 1) & ~static_cast<size_t>(1);
  const uint8_t* row = packed_filter + n * (k2 / 2);
  float total = 0.0f;
  for (int base = 0; base < nblk; base += kWaveSize) {
    const int bi = base + lane;
    float product = 0.0f;
    if (bi < nblk) {
      int32_t ksum = 0;
      for (int ki = 0; ki < blocksize; ++ki) ksum += NibbleAt(row, bi * blocksize + ki);
      const float scale = HalfBitsToFloat(scales_f16[static_cast<size_t>(n) * nblk + bi]);
      product = __fmul_rn(scale, static_cast<float>(ksum));
    }
    const int count = min(kWaveSize, nblk - base);
#pragma unroll
    for (int j = 0; j < kWaveSize; ++j) {
      if (j < count) {
        total = __fadd_rn(total, __int_as_float(__builtin_amdgcn_readlane(__float_as_int(product), j)));
      }
    }
  }
  if (lane == 0) kfsum[n] = total;
}

template <int R, int BT, int WC>
hipError_t LaunchVariant(const FcInt4Args& a, int batch0, hipStream_t stream) {
  const int nblk = a.depth / kBlock;
  const size_t lds_bytes = static_cast<size_t>(BT) * a.depth +
                           static_cast<size_t>(R) * BT * (nblk | 1) * sizeof(float);
  auto kernel = FcBlockwiseInt4Kernel<R, BT, WC>;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds_bytes)) return err;
  const int grid = (a.out_depth + R - 1) / R;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds_bytes, stream, a, batch0);
  return hipGetLastError();
}

template <int BT>
hipError_t LaunchForBatchTile(const FcInt4Args& a, int batch0, hipStream_t stream) {
  const int nblk = a.depth / kBlock;
  const int nchunks = (nblk + kWaveSize - 1) / kWaveSize;
  // Rows per workgroup: as many as keep >= ~1024 workgroups in the grid.
  const int r_pref = a.out_depth >= 8192 ? 8 : a.out_depth >= 4096 ? 4 : 2;
  if (nchunks >= 4) {  // four wavefronts split the depth
    if (r_pref == 8) return LaunchVariant<8, BT, 4>(a, batch0, stream);
    if (r_pref == 4) return LaunchVariant<4, BT, 4>(a, batch0, stream);
    return LaunchVariant<2, BT, 4>(a, batch0, stream);
  }
  if (nchunks >= 2) {  // two split the depth, two split the rows
    if (r_pref == 8) return LaunchVariant<8, BT, 2>(a, batch0, stream);
    if (r_pref == 4) return LaunchVariant<4, BT, 2>(a, batch0, stream);
    return LaunchVariant<2, BT, 2>(a, batch0, stream);
  }
  if (r_pref == 8) return LaunchVariant<8, BT, 1>(a, batch0, stream);
  return LaunchVariant<4, BT, 1>(a, batch0, stream);
}

}  // namespace

hipError_t LaunchBlockwiseInt4Kfsum(const uint8_t* packed_filter, const uint16_t* scales_f16,
                                    int out_depth, int depth, int blocksize, float* kfsum,
                                    hipStream_t stream) {
  if (out_depth == 0) return hipSuccess;
  const int channels_per_wg = kThreads / kWaveSize;
  const int grid = (out_depth + channels_per_wg - 1) / channels_per_wg;
  hipLaunchKernelGGL(BlockwiseInt4KfsumKernel, dim3(grid), dim3(kThreads), 0, stream,
                     packed_filter, scales_f16, out_depth, depth, blocksize, kfsum);
  return hipGetLastError();
}

hipError_t LaunchFcBlockwiseInt4(const FcInt4Args& a, hipStream_t stream) {
  if (a.batches == 0 || a.out_depth == 0) return hipSuccess;
  constexpr size_t kMaxLds = 150 * 1024;
  const bool fast = a.blocksize == kBlock && a.depth % kBlock == 0 && a.depth > 0 &&
                    ((reinterpret_cast<uintptr_t>(a.packed_filter) & 15) == 0) &&
                    ((reinterpret_cast<uintptr_t>(a.input) & 7) == 0) &&
                    // one batch row + its products must fit in LDS
                    (static_cast<size_t>(a.depth) + 8 * ((a.depth / kBlock) | 1) * 4 <= kMaxLds);
  if (!fast) {
    const int64_t total = static_cast<int64_t>(a.batches) * a.out_depth;
    const int grid = static_cast<int>((total + kThreads - 1) / kThreads);
    hipLaunchKernelGGL(FcBlockwiseInt4GenericKernel, dim3(grid), dim3(kThreads), 0, stream, a);
    return hipGetLastError();
  }
  int batch0 = 0;
  while (batch0 < a.batches) {
    const int left = a.batches - batch0;
    int bt = left >= 8 ? 8 : left >= 4 ? 4 : left >= 2 ? 2 : 1;
    // keep activations + products inside the LDS budget
    while (bt > 1 && static_cast<size_t>(bt) * a.depth +
                             8u * bt * ((a.depth / kBlock) | 1) * 4 > kMaxLds) {
      bt /= 2;
    }
    hipError_t err;
    switch (bt) {
      case 8:
        err = LaunchForBatchTile<8>(a, batch0, stream);
        break;
      case 4:
        err = LaunchForBatchTile<4>(a, batch0, stream);
        break;
      case 2:
        err = LaunchForBatchTile<2>(a, batch0, stream);
        break;
      default:
        err = LaunchForBatchTile<1>(a, batch0, stream);
        break;
    }
    if (err != hipSuccess) return err;
    batch0 += bt;
  }
  return hipSuccess;
}

}  // namespace lrtfc

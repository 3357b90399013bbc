// Prefill-regime full-integer FULLY_CONNECTED: a dense int8 GEMM on the gfx950
// matrix cores (v_mfma_i32_32x32x32_i8) with the per-channel requantization of
// reference/integer_ops/fully_connected.h:65-74 fused into the epilogue.
//
//   out[m, n] = requant(sum_k in[m, k] * w[n, k])     in [M, K], w [N, K], both K-major
//
// Both operands are K-contiguous in HBM, which is exactly what the MFMA A and B
// register layouts want (lane L holds 16 consecutive k of row/column L % 32), so
// tiles go to LDS unchanged. One 256-thread workgroup owns a 128 x 256 output
// tile (16 x 16 tiles = 256 workgroups for the 2048 x 4096 prefill shape: one per
// CU); its four wavefronts each own 64 x 128, i.e. 2 x 4 MFMA tiles and 128
// accumulator registers. K advances in slabs of 128 through two LDS buffers: the
// global loads of slab k+1 are in flight while slab k feeds the matrix cores.
// LDS rows are padded from 128 to 144 bytes so the 16-byte operand reads of 8
// consecutive rows fall in distinct banks.
//
// int32 accumulation is exact, so tiling order cannot change the accumulator;
// bit-exactness rests only on the epilogue.
#include "kernels.h"

namespace lrtfc {
namespace {

using i32x16 = int __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BM = 128;  // output rows (batch) per workgroup
constexpr int BN = 256;  // output columns (filter rows) per workgroup
constexpr int BK = 128;  // depth per LDS slab
constexpr int kLdsStride = BK + 16;
constexpr int kChunksPerRow = BK / 16;                        // 16-byte chunks per slab row
constexpr int kALoads = BM * kChunksPerRow / kThreads;        // 4
constexpr int kBLoads = BN * kChunksPerRow / kThreads;        // 8
constexpr int kStageBytes = (BM + BN) * kLdsStride;           // 55296
constexpr int kGroupM = 4;  // M-tiles per rasterization group (with 8 N-tiles: one XCD)

struct ChannelParams {
  int32_t multiplier;
  int32_t left_shift;
  int32_t right_shift;
  int32_t addend;  // bias + input_offset * row_sum
};

__device__ __forceinline__ int32_t Requantize(int32_t acc, const ChannelParams& p,
                                              int32_t output_offset, int32_t act_min,
                                              int32_t act_max) {
  const int32_t x =
      static_cast<int32_t>(static_cast<uint32_t>(acc + p.addend) << p.left_shift);
  const int32_t y = RoundingDivideByPot(Srdhm(x, p.multiplier), p.right_shift);
  return ClampI32(y + output_offset, act_min, act_max);
}

__global__ __launch_bounds__(kThreads, 1) void FcInt8GemmKernel(FcInt8Args a) {
  extern __shared__ __align__(16) int8_t smem[];
  const int M = a.batches, N = a.out_depth, K = a.depth;
  const int tiles_m = M / BM, tiles_n = N / BN;
  const int total = tiles_m * tiles_n;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // range of tile ids, and order ids so that a range is a compact rectangle whose
  // operand slabs stay in that XCD's L2.
  int id = blockIdx.x;
  if (total % 8 == 0) id = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
  const int width = kGroupM * tiles_n;
  const int group = id / width;
  const int first_m = group * kGroupM;
  const int gsize = min(tiles_m - first_m, kGroupM);
  const int tm = first_m + (id % width) % gsize;
  const int tn = (id % width) / gsize;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1;  // 0..1 -> 64 rows each
  const int wave_n = wave & 1;   // 0..1 -> 128 columns each

  const int ld_row = tid / kChunksPerRow;  // 0..31
  const int ld_chunk = tid % kChunksPerRow;
  const int8_t* a_src = a.input + static_cast<size_t>(m0 + ld_row) * K + ld_chunk * 16;
  const int8_t* b_src = a.filter + static_cast<size_t>(n0 + ld_row) * K + ld_chunk * 16;
  const size_t row_step = static_cast<size_t>(32) * K;  // 32 rows per pass of 256 threads
  const int lds_off = ld_row * kLdsStride + ld_chunk * 16;

  i32x4 a_reg[kALoads], b_reg[kBLoads];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      a_reg[i] = *reinterpret_cast<const i32x4*>(a_src + i * row_step + k0);
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      b_reg[i] = *reinterpret_cast<const i32x4*>(b_src + i * row_step + k0);
    }
  };
  auto store_lds = [&](int buf) {
    int8_t* as = smem + buf * kStageBytes;
    int8_t* bs = as + BM * kLdsStride;
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      *reinterpret_cast<i32x4*>(as + lds_off + i * 32 * kLdsStride) = a_reg[i];
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      *reinterpret_cast<i32x4*>(bs + lds_off + i * 32 * kLdsStride) = b_reg[i];
    }
  };

  i32x16 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    }
  }

  // Operand fragment addresses: lane L reads 16 bytes of row (L % 32) at k offset
  // 16 * (L / 32) inside each 32-deep MFMA step.
  const int frag_off = (lane & 31) * kLdsStride + (lane >> 5) * 16;
  const int a_frag = (wave_m * 64) * kLdsStride + frag_off;
  const int b_frag = BM * kLdsStride + (wave_n * 128) * kLdsStride + frag_off;

  load_global(0);
  store_lds(0);
  __syncthreads();

  const int num_slabs = K / BK;
  for (int kt = 0; kt < num_slabs; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < num_slabs) load_global((kt + 1) * BK);
    const int8_t* stage = smem + buf * kStageBytes;
#pragma unroll
    for (int kk = 0; kk < BK / 32; ++kk) {
      i32x4 af[2], bf[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = *reinterpret_cast<const i32x4*>(stage + a_frag + i * 32 * kLdsStride + kk * 32);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        bf[j] = *reinterpret_cast<const i32x4*>(stage + b_frag + j * 32 * kLdsStride + kk * 32);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
      }
    }
    if (kt + 1 < num_slabs) store_lds(buf ^ 1);
    __syncthreads();
  }

  // Epilogue. Accumulator register e of a 32x32 tile holds
  // row = 8 * (e / 4) + 4 * (lane / 32) + e % 4, column = lane % 32.
  const int col_in_tile = lane & 31;
  const int row_base = 4 * (lane >> 5);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + wave_n * 128 + j * 32 + col_in_tile;
    ChannelParams p;
    p.multiplier = a.per_channel ? a.multipliers[n] : a.multipliers[0];
    const int shift = a.per_channel ? a.shifts[n] : a.shifts[0];
    p.left_shift = shift > 0 ? shift : 0;
    p.right_shift = shift > 0 ? 0 : -shift;
    p.addend = a.bias_i32 ? a.bias_i32[n] : 0;
    if (a.input_offset != 0) p.addend += a.input_offset * a.filter_row_sums[n];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m_tile = m0 + wave_m * 64 + i * 32 + row_base;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m_tile + 8 * (e / 4) + (e % 4);
        const int32_t v = Requantize(acc[i][j][e], p, a.output_offset, a.act_min, a.act_max);
        a.output_i8[static_cast<size_t>(m) * N + n] = static_cast<int8_t>(v);
      }
    }
  }
}

}  // namespace

bool FcInt8GemmMfmaSupports(const FcInt8Args& a) {
  return a.batches >= BM && a.batches % BM == 0 && a.out_depth % BN == 0 && a.depth % BK == 0 &&
         a.depth > 0 && a.filter_offset == 0 &&
         ((reinterpret_cast<uintptr_t>(a.filter) & 15) == 0) &&
         ((reinterpret_cast<uintptr_t>(a.input) & 15) == 0);
}

hipError_t LaunchFcInt8GemmMfma(const FcInt8Args& a, hipStream_t stream) {
  if (!FcInt8GemmMfmaSupports(a)) return hipErrorNotSupported;
  const int lds_bytes = 2 * kStageBytes;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(FcInt8GemmKernel),
                                        lds_bytes)) {
    return err;
  }
  const int grid = (a.batches / BM) * (a.out_depth / BN);
  hipLaunchKernelGGL(FcInt8GemmKernel, dim3(grid), dim3(kThreads), lds_bytes, stream, a);
  return hipGetLastError();
}

}  // namespace lrtfc

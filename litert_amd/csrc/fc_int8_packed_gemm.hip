// Prefill-regime FULLY_CONNECTED on the re-tiled int8 filter: a dense int8 GEMM on the
// gfx950 matrix cores (v_mfma_i32_32x32x32_i8, the int8 instruction with the highest rate)
// that shares its weight layout with the decode GEMV, so a filter is kept in ONE form for
// every batch size.
//
//   out[m, n] = epilogue(sum_k x[m, k] * w[n, k])        x [M, K] row-major int8
//
// The filter is stored in 1 KiB tiles of 16 channels x 64 depth (lane L of a tile: channel
// L % 16, depth 16 * (L / 16) .. +16). A 32x32x32 operand (lane L: channel L % 32, 16 depth
// bytes of half L / 32) is gathered from two such tiles by per-lane addresses; each quarter
// of the wavefront still reads 256 consecutive bytes, so the load is as efficient as a
// contiguous one. Each wavefront owns 64 output channels and loads their operands straight
// from global memory into registers, three depth steps ahead -- the weights never touch
// LDS, because no other wavefront of the workgroup needs them. Only the activation rows are
// shared: the workgroup stages 128 rows x 64 depth per step in LDS (two buffers, rows padded
// to 80 bytes so that the 16-byte operand reads are conflict-free) and every wavefront reads
// its eight operands from there. Per step and wavefront: 4 global loads, 8 LDS reads, 16
// MFMAs (512 matrix-core cycles), one barrier placed between the two halves of the MFMAs.
// Launches that this 128 x 256 tile would cut into fewer workgroups than half the chip's CUs
// (batches of a few dozen to a few hundred rows) run the same kernel with 64 rows x 128
// channels per workgroup (32 channels per wavefront).
//
// int32 accumulation is exact, so tiling cannot change the accumulator; bit-exactness rests
// on the epilogues, which are the ones of the GEMV kernels (fc_epilogues.h).
#include <type_traits>
#include <utility>

#include "fc_epilogues.h"
#include "kernels.h"

namespace lrtfc {
namespace {

using i32x16 = int __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kStep = 64;                     // depth per step = one slab of the packed filter
constexpr int kXStride = kStep + 16;          // padded LDS row
constexpr int kSub = kStep / 32;              // MFMA depth sub-steps per step
constexpr int kRing = 4;                      // weight register ring, in steps (even)
constexpr int kGroupM = 4;                    // M-tiles per rasterization group

// f(std::integral_constant<int, 0>{}), f(<1>), ... : a loop whose index is a constant in
// every iteration, so that register arrays indexed by it stay in fixed registers.
template <int... Is, typename F>
__device__ __forceinline__ void ForEachConst(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}

// BM: batch rows per workgroup (128, or 64 for launches the large tile would leave with few
// workgroups); kWaveTiles: 32-channel MFMA tiles per wavefront (2 or 1).
template <Int8Epilogue EPI, int BM, int kWaveTiles>
__global__ __launch_bounds__(kThreads, 1) void FcInt8PackedGemmKernel(FcInt8Args a) {
  constexpr int BN = kWaves * kWaveTiles * 32;  // output channels per workgroup
  constexpr int kStageBytes = BM * kXStride;
  constexpr int kBatchTiles = BM / 32;
  constexpr int kXChunks = BM / 64;  // 16-byte chunks of activations a thread stages per step
  static_assert(BM % 64 == 0 && BN <= kThreads, "tile shape");
  __shared__ __align__(16) int8_t smem[2 * kStageBytes];
  __shared__ i32x4 chan_params[BN];  // per output channel of the tile, for the epilogue
  const int M = a.batches, N = a.out_depth, K = a.depth;
  const int slabs = (K + kStep - 1) / kStep;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous range of tile
  // ids, ordered so that a range is a compact rectangle whose operands stay in that XCD's L2.
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
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // Per-channel epilogue inputs, one channel per thread, fetched now so that their latency
  // hides behind the main loop: {multiplier, shift, bias + input_offset * row_sum, -} or
  // {channel scale, bias, row sum, -}.
  i32x4 chan_p;
  {
    const int n = min(n0 + tid, N - 1);
    i32x4 p = {0, 0, 0, 0};
    if (EPI == Int8Epilogue::kRequantize) {
      p[0] = a.per_channel ? a.multipliers[n] : a.multipliers[0];
      p[1] = a.per_channel ? a.shifts[n] : a.shifts[0];
      p[2] = a.bias_i32 ? a.bias_i32[n] : 0;
      if (a.input_offset != 0) p[2] += a.input_offset * a.filter_row_sums[n];
    } else {
      p[0] = __float_as_int(a.per_channel_scales ? a.per_channel_scales[n] : a.filter_scale);
      p[1] = __float_as_int(a.bias_f32 ? a.bias_f32[n] : 0.0f);
      p[2] = (EPI == Int8Epilogue::kHybrid && a.zero_points) ? a.filter_row_sums[n] : 0;
    }
    chan_p = p;
  }
  // EvalHybridDense's early exit for a whole-zero input (fully_connected.cc:789-795) matters only
  // where a bias element is -0.0f: a workgroup that stages such a channel settles the question
  // here, once, outside the loops that must unroll.
  bool zero_input = false;
  if (EPI == Int8Epilogue::kHybrid && a.zero_input_exit) {
    const bool mine = tid < BN && n0 + tid < N && a.bias_f32 != nullptr &&
                      IsNegativeZero(__int_as_float(chan_p[1]));
    if (__syncthreads_or(mine)) {
      zero_input = WorkgroupAllZeroInt8(a.input, static_cast<size_t>(M) * K);
    }
  }

  // Weight operands of this wavefront: lane L addresses channel L % 32 of MFMA tile i (tile
  // index clamped at the last 16-channel tile: duplicates are computed and never stored) and
  // the 16 bytes of depth half L / 32 within a 32-deep sub-step.
  const int ctiles = (N + 15) / 16;
  const int8_t* wp[kWaveTiles];
#pragma unroll
  for (int i = 0; i < kWaveTiles; ++i) {
    const int ct = min(n0 / 16 + (wave * kWaveTiles + i) * 2 + ((lane & 31) >> 4), ctiles - 1);
    wp[i] = a.filter + static_cast<size_t>(ct) * slabs * 1024 + (lane & 15) * 16 + (lane >> 5) * 256;
  }
  // Activation staging: 16-byte chunks per thread and step, rows tid / 4 (and 64 + tid / 4).
  const int ld_chunk = tid & 3;
  const int8_t* xp[kXChunks];
#pragma unroll
  for (int i = 0; i < kXChunks; ++i) {
    const int row = min(m0 + (tid >> 2) + 64 * i, M - 1);
    xp[i] = a.input + static_cast<size_t>(row) * K;
  }
  const int st_off = (tid >> 2) * kXStride + ld_chunk * 16;

  i32x4 wring[kRing][kWaveTiles][kSub];
  i32x4 xr[2][kXChunks];  // two sets: rows are requested two steps before they are staged
  auto load_w = [&](int step, auto slot) {
    const int s = min(step, slabs - 1);
#pragma unroll
    for (int i = 0; i < kWaveTiles; ++i) {
#pragma unroll
      for (int h = 0; h < kSub; ++h) {
        wring[decltype(slot)::value][i][h] =
            *reinterpret_cast<const i32x4*>(wp[i] + static_cast<size_t>(s) * 1024 + h * 512);
      }
    }
  };
  auto load_x = [&](int step, auto set) {
    // Past the end of a row (last partial slab, steps beyond the last) the address is clamped
    // into the row: whatever it reads meets zero padding in the packed filter or is unused.
    const int k = min(min(step, slabs - 1) * kStep + ld_chunk * 16, K - 16);
#pragma unroll
    for (int i = 0; i < kXChunks; ++i) {
      xr[decltype(set)::value][i] = *reinterpret_cast<const i32x4*>(xp[i] + k);
    }
  };
  auto store_x = [&](int stage, auto set) {
#pragma unroll
    for (int i = 0; i < kXChunks; ++i) {
      *reinterpret_cast<i32x4*>(smem + stage * kStageBytes + st_off + i * 64 * kXStride) =
          xr[decltype(set)::value][i];
    }
  };
  // Operand of batch tile j, sub-step h: lane L reads row 32 j + L % 32, bytes
  // 32 h + 16 * (L / 32) .. +16 of the staged 64.
  const int frag_off = (lane & 31) * kXStride + (lane >> 5) * 16;
  auto read_frag = [&](int stage, int j, int h) {
    return *reinterpret_cast<const i32x4*>(smem + stage * kStageBytes + frag_off +
                                           j * 32 * kXStride + h * 32);
  };

  i32x16 acc[kWaveTiles][kBatchTiles];
#pragma unroll
  for (int i = 0; i < kWaveTiles; ++i) {
#pragma unroll
    for (int j = 0; j < kBatchTiles; ++j) {
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    }
  }

  // Prologue: step 0 staged, steps 1 and 2 in registers, weights of steps 0 .. kRing - 2 in
  // flight.
  // (Same issue order as inside the loop: activation rows first, then weights.)
  load_x(0, std::integral_constant<int, 0>{});
  store_x(0, std::integral_constant<int, 0>{});
  asm volatile("" ::: "memory");
  load_x(1, std::integral_constant<int, 1>{});
  load_x(2, std::integral_constant<int, 0>{});
  asm volatile("" ::: "memory");
  ForEachConst(std::make_integer_sequence<int, kRing - 1>{}, [&](auto u) { load_w(u, u); });
  asm volatile("" ::: "memory");
  if (tid < BN) chan_params[tid] = chan_p;
  __syncthreads();
  i32x4 fa[kBatchTiles][kSub];
#pragma unroll
  for (int j = 0; j < kBatchTiles; ++j) {
#pragma unroll
    for (int h = 0; h < kSub; ++h) fa[j][h] = read_frag(0, j, h);
  }

  auto step_body = [&](int s, auto slot) {
    constexpr int kSlot = decltype(slot)::value;
    constexpr int kNext = (kSlot + kRing - 1) % kRing;
    const int next_stage = (s + 1) & 1;
    constexpr int kXSet = (kSlot + 1) % 2;  // set of step s + 1, and then of step s + 3
    store_x(next_stage, std::integral_constant<int, kXSet>{});  // rows requested two steps ago
    // Vector memory returns in issue order and the next step's store_x waits for these rows,
    // so they must be requested before the weights; the fences pin that order.
    asm volatile("" ::: "memory");
    load_x(s + 3, std::integral_constant<int, kXSet>{});
    asm volatile("" ::: "memory");
    load_w(s + kRing - 1, std::integral_constant<int, kNext>{});
    asm volatile("" ::: "memory");
    // The scheduling fences keep the instruction order written here: each group of LDS reads
    // is followed by eight MFMAs that do not depend on it, which hides the read latency; left
    // alone, the compiler moves every read next to its first use.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < kBatchTiles; ++j) {
#pragma unroll
      for (int i = 0; i < kWaveTiles; ++i) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wring[kSlot][i][0], fa[j][0], acc[i][j], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();  // step s + 1 is staged; the other buffer is free for step s + 2
#pragma unroll
    for (int j = 0; j < kBatchTiles; ++j) fa[j][0] = read_frag(next_stage, j, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < kBatchTiles; ++j) {
#pragma unroll
      for (int i = 0; i < kWaveTiles; ++i) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wring[kSlot][i][1], fa[j][1], acc[i][j], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < kBatchTiles; ++j) fa[j][1] = read_frag(next_stage, j, 1);
    __builtin_amdgcn_sched_barrier(0);
  };

  // Whole groups of kRing steps run without branches so that the ring slots stay fixed
  // registers; the remainder repeats the first slots.
  int s0 = 0;
  for (; s0 + kRing <= slabs; s0 += kRing) {
    ForEachConst(std::make_integer_sequence<int, kRing>{}, [&](auto u) { step_body(s0 + u, u); });
  }
  ForEachConst(std::make_integer_sequence<int, kRing - 1>{}, [&](auto u) {
    if (s0 + u < slabs) step_body(s0 + u, u);
  });

  // Epilogue. Register e of acc[i][j] holds channel 32 i + 8 * (e / 4) + 4 * (L / 32) + e % 4 of
  // the wavefront's 64 and batch row 32 j + L % 32 of the workgroup's 128: four groups (g) of
  // four consecutive channels per lane and tile.
  const int row_in_tile = lane & 31;
  const bool vec_ok = (N & 3) == 0;
  // Interior tiles (the common case) store whole dwords without any bounds test.
  auto epilogue = [&](auto full_tag) {
  constexpr bool kFull = decltype(full_tag)::value;
#pragma unroll
  for (int i = 0; i < kWaveTiles; ++i) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int c0 = n0 + (wave * kWaveTiles + i) * 32 + 8 * g + 4 * (lane >> 5);
      const int local = (wave * kWaveTiles + i) * 32 + 8 * g + 4 * (lane >> 5);
      if (EPI == Int8Epilogue::kRequantize) {
        int32_t mult[4], shift[4], addend[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const i32x4 p = chan_params[local + r];
          mult[r] = p[0];
          shift[r] = p[1];
          addend[r] = p[2];
        }
#pragma unroll
        for (int j = 0; j < kBatchTiles; ++j) {
          const int m = m0 + j * 32 + row_in_tile;
          int32_t q[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            q[r] = RequantizeCore(acc[i][j][4 * g + r] + addend[r], mult[r], shift[r],
                                  a.output_offset, a.act_min, a.act_max);
          }
          if (kFull || m < M) {
            int8_t* dst = a.output_i8 + static_cast<size_t>(m) * N + c0;
            if (kFull || (vec_ok && c0 + 3 < N)) {
              *reinterpret_cast<int32_t*>(dst) =
                  (q[0] & 0xFF) | ((q[1] & 0xFF) << 8) | ((q[2] & 0xFF) << 16) |
                  static_cast<int32_t>(static_cast<uint32_t>(q[3]) << 24);
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                if (c0 + r < N) dst[r] = static_cast<int8_t>(q[r]);
              }
            }
          }
        }
      } else {
        float cscale[4], base[4];
        int32_t rsum[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const i32x4 p = chan_params[local + r];
          cscale[r] = __int_as_float(p[0]);
          base[r] = __int_as_float(p[1]);
          rsum[r] = p[2];
        }
#pragma unroll
        for (int j = 0; j < kBatchTiles; ++j) {
          const int m = m0 + j * 32 + row_in_tile;
          const int mc = min(m, M - 1);
          const float bscale = a.scaling_factors[mc];
          const int32_t bzp = a.zero_points ? a.zero_points[mc] : 0;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            v[r] = EPI == Int8Epilogue::kHybrid4Bit
                       ? Hybrid4BitCore(acc[i][j][4 * g + r], bscale, cscale[r], bzp, base[r],
                                        a.bias_f32 != nullptr, a.activation)
                       : HybridCoreSelect(acc[i][j][4 * g + r], bscale, cscale[r], bzp, rsum[r],
                                          base[r], a.activation, a.batch_matmul != 0, zero_input);
          }
          if (kFull || m < M) {
            float* dst = a.output_f32 + static_cast<size_t>(m) * N + c0;
            if (kFull || (vec_ok && c0 + 3 < N)) {
              *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                if (c0 + r < N) dst[r] = v[r];
              }
            }
          }
        }
      }
    }
  }
  };
  if (vec_ok && m0 + BM <= M && n0 + BN <= N) {
    epilogue(std::true_type{});
  } else {
    epilogue(std::false_type{});
  }
}

template <int BM, int kWaveTiles>
hipError_t LaunchShape(const FcInt8Args& a, Int8Epilogue epilogue, int grid, hipStream_t stream) {
  if (epilogue == Int8Epilogue::kRequantize) {
    hipLaunchKernelGGL((FcInt8PackedGemmKernel<Int8Epilogue::kRequantize, BM, kWaveTiles>),
                       dim3(grid), dim3(kThreads), 0, stream, a);
  } else if (epilogue == Int8Epilogue::kHybrid) {
    hipLaunchKernelGGL((FcInt8PackedGemmKernel<Int8Epilogue::kHybrid, BM, kWaveTiles>),
                       dim3(grid), dim3(kThreads), 0, stream, a);
  } else {
    hipLaunchKernelGGL((FcInt8PackedGemmKernel<Int8Epilogue::kHybrid4Bit, BM, kWaveTiles>),
                       dim3(grid), dim3(kThreads), 0, stream, a);
  }
  return hipGetLastError();
}

constexpr int kMinLargeTiles = 128;

}  // namespace

bool FcInt8PackedGemmSupports(const FcInt8Args& a) {
  return a.depth >= 16 && a.depth % 16 == 0 && a.filter_offset == 0 && a.batches > 0 &&
         a.out_depth > 0 && ((reinterpret_cast<uintptr_t>(a.filter) & 15) == 0) &&
         ((reinterpret_cast<uintptr_t>(a.input) & 15) == 0);
}

hipError_t LaunchFcInt8PackedGemm(const FcInt8Args& a, Int8Epilogue epilogue, hipStream_t stream) {
  if (!FcInt8PackedGemmSupports(a)) return hipErrorNotSupported;
  // 128 x 256 tiles move the fewest bytes per MFMA; a launch they would cut into fewer
  // workgroups than half the chip's CUs takes 64 x 128 tiles instead (four times as many).
  const int large = ((a.batches + 127) / 128) * ((a.out_depth + 255) / 256);
  if (large >= kMinLargeTiles) return LaunchShape<128, 2>(a, epilogue, large, stream);
  return LaunchShape<64, 1>(a, epilogue, ((a.batches + 63) / 64) * ((a.out_depth + 127) / 128),
                            stream);
}

}  // namespace lrtfc

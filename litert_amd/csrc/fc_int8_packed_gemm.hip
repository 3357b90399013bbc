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
// from global memory into registers, two depth steps ahead -- the weights never touch LDS,
// because no other wavefront of the workgroup needs them. Only the activation rows are
// shared: the workgroup stages 128 rows x 128 depth per step in LDS (two buffers, rows padded
// to 144 bytes so that the 16-byte operand reads are conflict-free; 128 bytes of a row are one
// whole cache line) and every wavefront reads its sixteen operands from there. Per step and
// wavefront: 12 global loads, 16 LDS reads, 4 LDS writes, 32 MFMAs (1024 matrix-core cycles)
// and one barrier, all dealt out singly between the MFMAs: a wavefront is alone on its SIMD,
// so whatever holds up its instruction stream idles the matrix pipe.
// Launches that this 128 x 256 tile would cut into fewer workgroups than half the chip's CUs
// (batches of a few dozen to a few hundred rows) run the same kernel with 64 rows x 128
// channels per workgroup (32 channels per wavefront).
//
// The int8 outputs of an interior tile are put together in LDS (the row buffers, free by then)
// and stored in 16-byte pieces, whole cache lines per row.
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
constexpr int kSlab = 64;                     // depth of one tile of the packed filter
constexpr int kStep = 128;                    // depth per step: two slabs, one cache line of a row
constexpr int kXStride = kStep + 16;          // padded LDS row
constexpr int kSub = kStep / 32;              // MFMA depth sub-steps per step
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
  constexpr int kXChunks = BM / 32;  // 16-byte chunks of activations a thread stages per step
  static_assert(BM % 64 == 0 && BN <= kThreads, "tile shape");
  __shared__ __align__(16) int8_t smem[2 * kStageBytes];
  __shared__ i32x4 chan_params[BN];  // per output channel of the tile, for the epilogue
  const int M = a.batches, N = a.out_depth, K = a.depth;
  const int slabs = (K + kSlab - 1) / kSlab;
  const int steps = (slabs + 1) / 2;
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
  // hides behind the main loop: {multiplier, shift, bias + input_offset * row_sum, rounding
  // term of the right shift} or {channel scale, bias, row sum, -}.
  i32x4 chan_p;
  bool plain_channel = true;  // this thread's channel allows the short requantization
  {
    const int n = min(n0 + tid, N - 1);
    i32x4 p = {0, 0, 0, 0};
    if (EPI == Int8Epilogue::kRequantize) {
      p[0] = a.per_channel ? a.multipliers[n] : a.multipliers[0];
      p[1] = a.per_channel ? a.shifts[n] : a.shifts[0];
      p[2] = a.bias_i32 ? a.bias_i32[n] : 0;
      if (a.input_offset != 0) p[2] += a.input_offset * a.filter_row_sums[n];
      p[3] = (p[1] < 0 && p[1] >= -31) ? (1 << (-p[1] - 1)) : 0;
      plain_channel = p[1] <= -1 && p[1] >= -31 && p[0] != INT32_MIN &&
                      p[2] > -(1 << 29) && p[2] < (1 << 29);
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
  // Activation staging: 16-byte chunks per thread and step, chunk tid % 8 of rows tid / 8 + 32 p
  // (eight consecutive lanes read one whole 128-byte line of a row).
  const int ld_chunk = tid & 7;
  const int8_t* xp[kXChunks];
#pragma unroll
  for (int p = 0; p < kXChunks; ++p) {
    const int row = min(m0 + (tid >> 3) + 32 * p, M - 1);
    xp[p] = a.input + static_cast<size_t>(row) * K;
  }
  const int st_off = (tid >> 3) * kXStride + ld_chunk * 16;
  // An odd number of slabs leaves the second half of the last step without a filter tile: the
  // weight addresses are clamped to the last tile and the rows' half is staged as zeros.
  const bool upper_chunk = ld_chunk >= 4;
  const int half_step = (slabs & 1) ? steps - 1 : -1;

  // Weights: wring[step % 2] holds a step's operands; a piece is requested again, for two steps
  // later, right after the last MFMA that reads it. Rows: xr[step % 2], requested three steps
  // before their use, staged two steps before it, read into fa during the step before it.
  i32x4 wring[2][kWaveTiles][kSub];
  i32x4 xr[2][kXChunks];
  auto load_w_piece = [&](int step, auto slot, auto tile, auto sub) {
    constexpr int i = decltype(tile)::value, h = decltype(sub)::value;
    const int slab = min(2 * step + h / 2, slabs - 1);
    wring[decltype(slot)::value][i][h] = *reinterpret_cast<const i32x4*>(
        wp[i] + static_cast<size_t>(slab) * 1024 + (h & 1) * 512);
  };
  auto load_x_piece = [&](int step, auto set, auto piece) {
    // Past the end of a row (last partial slab, steps beyond the last) the address is clamped
    // into the row: whatever it reads meets zero padding in the packed filter, is replaced by
    // zeros when staged, or is never used.
    const int k = min(min(step, steps - 1) * kStep + ld_chunk * 16, K - 16);
    xr[decltype(set)::value][decltype(piece)::value] =
        *reinterpret_cast<const i32x4*>(xp[decltype(piece)::value] + k);
  };
  auto store_x_piece = [&](int step, auto set, auto piece) {
    constexpr int p = decltype(piece)::value;
    i32x4 v = xr[decltype(set)::value][p];
    if (upper_chunk && step == half_step) v = i32x4{0, 0, 0, 0};
    *reinterpret_cast<i32x4*>(smem + decltype(set)::value * kStageBytes + st_off +
                              p * 32 * kXStride) = v;
  };
  // Operand of batch tile j, sub-step h: lane L reads row 32 j + L % 32, bytes
  // 32 h + 16 * (L / 32) .. +16 of the staged 128.
  const int frag_off = (lane & 31) * kXStride + (lane >> 5) * 16;
  auto read_frag = [&](auto stage, int j, int h) {
    return *reinterpret_cast<const i32x4*>(smem + decltype(stage)::value * kStageBytes + frag_off +
                                           j * 32 * kXStride + h * 32);
  };
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  constexpr auto kTiles = std::make_integer_sequence<int, kWaveTiles>{};
  constexpr auto kSubs = std::make_integer_sequence<int, kSub>{};
  constexpr auto kChunks = std::make_integer_sequence<int, kXChunks>{};

  i32x16 acc[kWaveTiles][kBatchTiles];
#pragma unroll
  for (int i = 0; i < kWaveTiles; ++i) {
#pragma unroll
    for (int j = 0; j < kBatchTiles; ++j) {
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    }
  }

  // Prologue: rows of steps 0 and 1 staged, those of step 2 requested, weights of steps 0 and 1
  // requested, operands of step 0 read.
  ForEachConst(kChunks, [&](auto p) { load_x_piece(0, C0{}, p); });
  ForEachConst(kChunks, [&](auto p) { load_x_piece(1, C1{}, p); });
  asm volatile("" ::: "memory");
  ForEachConst(kTiles, [&](auto i) { ForEachConst(kSubs, [&](auto h) { load_w_piece(0, C0{}, i, h); }); });
  ForEachConst(kTiles, [&](auto i) { ForEachConst(kSubs, [&](auto h) { load_w_piece(1, C1{}, i, h); }); });
  asm volatile("" ::: "memory");
  ForEachConst(kChunks, [&](auto p) { store_x_piece(0, C0{}, p); });
  ForEachConst(kChunks, [&](auto p) { store_x_piece(1, C1{}, p); });
  asm volatile("" ::: "memory");
  ForEachConst(kChunks, [&](auto p) { load_x_piece(2, C0{}, p); });
  asm volatile("" ::: "memory");
  if (tid < BN) chan_params[tid] = chan_p;
  // The short requantization (RequantizeShort) needs every channel of the tile to shift right by
  // 1..31 bits and |accumulator + addend| < 2^30, which |addend| < 2^29 and a depth of at most
  // 32768 guarantee; one channel outside that sends the whole workgroup down the general form.
  const bool general_requantize =
      __syncthreads_or(EPI == Int8Epilogue::kRequantize &&
                       ((tid < BN && !plain_channel) || K > 32768 || a.act_min > a.act_max));
  i32x4 fa[kBatchTiles][kSub];
#pragma unroll
  for (int j = 0; j < kBatchTiles; ++j) {
#pragma unroll
    for (int h = 0; h < kSub; ++h) fa[j][h] = read_frag(C0{}, j, h);
  }

  // One depth step s (slot = s % 2). MFMA number m works on sub-step h = m / kHalf, channel tile
  // i = (m % kHalf) / kBatchTiles, batch tile j = m % kBatchTiles; what follows it:
  //   * after the first MFMA that frees an operand of the rows: the barrier that publishes the
  //     rows of step s + 1 (staged at the end of step s - 1);
  //   * after the last use of fa[j][h] (i = last tile): its LDS read for step s + 1;
  //   * after the last use of weight piece (i, h) (j = last batch tile): its load for step s + 2;
  //   * spread over the step: the loads of the rows of step s + 3;
  //   * from the middle of the step on, one every few MFMAs: the LDS writes of the rows of step
  //     s + 2, into the buffer whose readers all passed this step's barrier (behind the last
  //     MFMAs instead they are still in the LDS queue when the next step's barrier waits for
  //     them: 1.6 us per launch of config 4 at the nominal clock).
  // The scheduling fences keep exactly this order. Vector memory returns in issue order, which
  // the waits the compiler derives from the registers respect.
  constexpr int kHalf = kBatchTiles * kWaveTiles;
  constexpr int kMfmas = kSub * kHalf;
  constexpr int kFirstFree = (kWaveTiles - 1) * kBatchTiles;
  constexpr int kStoreAt = kMfmas / 4, kStoreEvery = (kMfmas / 2) / kXChunks;
  auto step_body = [&](int s, auto slot) {
    constexpr int kSlot = decltype(slot)::value;
    using Slot = std::integral_constant<int, kSlot>;
    using Other = std::integral_constant<int, 1 - kSlot>;
    ForEachConst(std::make_integer_sequence<int, kMfmas>{}, [&](auto index) {
      constexpr int m = decltype(index)::value;
      constexpr int h = m / kHalf, i = (m % kHalf) / kBatchTiles, j = m % kBatchTiles;
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wring[kSlot][i][h], fa[j][h], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (m == kFirstFree) {
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (i == kWaveTiles - 1) {
        fa[j][h] = read_frag(Other{}, j, h);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (j == kBatchTiles - 1) {
        load_w_piece(s + 2, Slot{}, std::integral_constant<int, i>{}, std::integral_constant<int, h>{});
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (m % (kMfmas / kXChunks) == 1) {
        load_x_piece(s + 3, Other{}, std::integral_constant<int, m / (kMfmas / kXChunks)>{});
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (m >= kStoreAt && (m - kStoreAt) % kStoreEvery == 0 &&
                    (m - kStoreAt) / kStoreEvery < kXChunks) {
        store_x_piece(s + 2, Slot{},
                      std::integral_constant<int, (m - kStoreAt) / kStoreEvery>{});
        __builtin_amdgcn_sched_barrier(0);
      }
    });
  };

  // Pairs of steps run without branches so that the two slots stay fixed registers.
  int s0 = 0;
  for (; s0 + 2 <= steps; s0 += 2) {
    step_body(s0, C0{});
    step_body(s0 + 1, C1{});
  }
  if (s0 < steps) step_body(s0, C0{});

  // Epilogue. Register e of acc[i][j] holds channel 32 i + 8 * (e / 4) + 4 * (L / 32) + e % 4 of
  // the wavefront's 64 and batch row 32 j + L % 32 of the workgroup's 128: four groups (g) of
  // four consecutive channels per lane and tile.
  const int row_in_tile = lane & 31;
  const bool vec_ok = (N & 3) == 0;
  // The clamp bounds in vector registers: v_med3_i32 takes at most one scalar operand.
  int32_t act_lo = a.act_min, act_hi = a.act_max;
  asm volatile("" : "+v"(act_lo), "+v"(act_hi));
  // Interior tiles (the common case) store whole dwords without any bounds test.
  // kStaged (int8 outputs of an interior tile): the tile is put together in LDS and leaves in
  // 16-byte pieces, sixteen lanes to a row, i.e. in whole cache lines. Stored from the
  // accumulator layout a store instruction touches 32 rows with 8 bytes each, and the 8 MB of
  // config 4's output reach L2 as a million partial-line writes behind the last MFMA.
  constexpr int kOutStride = BN + 16;
  static_assert(BM * kOutStride <= 2 * kStageBytes, "output tile does not fit the row buffers");
  auto epilogue = [&](auto full_tag, auto short_tag, auto staged_tag) {
  constexpr bool kFull = decltype(full_tag)::value;
  constexpr bool kShort = decltype(short_tag)::value;
  constexpr bool kStaged = decltype(staged_tag)::value;
  if (kStaged) __syncthreads();  // every wavefront has read its last row operands
#pragma unroll
  for (int i = 0; i < kWaveTiles; ++i) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int c0 = n0 + (wave * kWaveTiles + i) * 32 + 8 * g + 4 * (lane >> 5);
      const int local = (wave * kWaveTiles + i) * 32 + 8 * g + 4 * (lane >> 5);
      if (EPI == Int8Epilogue::kRequantize) {
        int32_t mult[4], shift[4], addend[4], half[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const i32x4 p = chan_params[local + r];
          mult[r] = p[0];
          shift[r] = kShort ? -p[1] : p[1];
          addend[r] = p[2];
          half[r] = p[3];
        }
#pragma unroll
        for (int j = 0; j < kBatchTiles; ++j) {
          const int m = m0 + j * 32 + row_in_tile;
          int32_t q[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            q[r] = kShort ? RequantizeShort(acc[i][j][4 * g + r] + addend[r], mult[r], shift[r],
                                            half[r], a.output_offset, act_lo, act_hi)
                          : RequantizeCore(acc[i][j][4 * g + r] + addend[r], mult[r], shift[r],
                                           a.output_offset, a.act_min, a.act_max);
          }
          if (kStaged) {
            *reinterpret_cast<int32_t*>(smem + (j * 32 + row_in_tile) * kOutStride + local) =
                PackLowBytes(q[0], q[1], q[2], q[3]);
          } else if (kFull || m < M) {
            int8_t* dst = a.output_i8 + static_cast<size_t>(m) * N + c0;
            if (kFull || (vec_ok && c0 + 3 < N)) {
              *reinterpret_cast<int32_t*>(dst) = PackLowBytes(q[0], q[1], q[2], q[3]);
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
  if (kStaged) {
    __syncthreads();
    constexpr int kPiecesPerRow = BN / 16;
#pragma unroll
    for (int k = 0; k < BM * kPiecesPerRow / kThreads; ++k) {
      const int piece = k * kThreads + tid;
      const int row = piece / kPiecesPerRow, at = (piece % kPiecesPerRow) * 16;
      *reinterpret_cast<i32x4*>(a.output_i8 + static_cast<size_t>(m0 + row) * N + n0 + at) =
          *reinterpret_cast<const i32x4*>(smem + row * kOutStride + at);
    }
  }
  };
  // The float outputs of an interior tile take the same way, 32 rows (one batch tile) at a time:
  // a wavefront then stores one row's whole kilobyte per instruction instead of 32 bytes in each
  // of 32 rows.
  auto epilogue_float_staged = [&]() {
    constexpr int kRowBytes = BN * 4 + 16;
    static_assert(32 * kRowBytes <= 2 * kStageBytes, "a batch tile of floats does not fit");
    constexpr int kPiecesPerRow = BN / 4;
#pragma unroll
    for (int j = 0; j < kBatchTiles; ++j) {
      const int m = m0 + j * 32 + row_in_tile;
      const float bscale = a.scaling_factors[m];
      const int32_t bzp = a.zero_points ? a.zero_points[m] : 0;
      __syncthreads();  // the buffer's last readers (main loop, previous batch tile) are through
#pragma unroll
      for (int i = 0; i < kWaveTiles; ++i) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int local = (wave * kWaveTiles + i) * 32 + 8 * g + 4 * (lane >> 5);
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const i32x4 p = chan_params[local + r];
            v[r] = EPI == Int8Epilogue::kHybrid4Bit
                       ? Hybrid4BitCore(acc[i][j][4 * g + r], bscale, __int_as_float(p[0]), bzp,
                                        __int_as_float(p[1]), a.bias_f32 != nullptr, a.activation)
                       : HybridCoreSelect(acc[i][j][4 * g + r], bscale, __int_as_float(p[0]), bzp,
                                          p[2], __int_as_float(p[1]), a.activation,
                                          a.batch_matmul != 0, zero_input);
          }
          *reinterpret_cast<float4*>(smem + row_in_tile * kRowBytes + local * 4) =
              make_float4(v[0], v[1], v[2], v[3]);
        }
      }
      __syncthreads();
#pragma unroll
      for (int k = 0; k < 32 * kPiecesPerRow / kThreads; ++k) {
        const int piece = k * kThreads + tid;
        const int row = piece / kPiecesPerRow, at = (piece % kPiecesPerRow) * 16;
        *reinterpret_cast<i32x4*>(reinterpret_cast<int8_t*>(a.output_f32) +
                                  (static_cast<size_t>(m0 + j * 32 + row) * N + n0) * 4 + at) =
            *reinterpret_cast<const i32x4*>(smem + row * kRowBytes + at);
      }
    }
  };
  const bool interior = vec_ok && m0 + BM <= M && n0 + BN <= N;
  if (EPI != Int8Epilogue::kRequantize && interior &&
      (reinterpret_cast<uintptr_t>(a.output_f32) & 15) == 0) {
    epilogue_float_staged();
    return;
  }
  if (EPI == Int8Epilogue::kRequantize && !general_requantize) {
    const bool staged =
        interior && (N & 15) == 0 && (reinterpret_cast<uintptr_t>(a.output_i8) & 15) == 0;
    if (staged) {
      epilogue(std::true_type{}, std::true_type{}, std::true_type{});
    } else if (interior) {
      epilogue(std::true_type{}, std::true_type{}, std::false_type{});
    } else {
      epilogue(std::false_type{}, std::true_type{}, std::false_type{});
    }
  } else if (interior) {
    epilogue(std::true_type{}, std::false_type{}, std::false_type{});
  } else {
    epilogue(std::false_type{}, std::false_type{}, std::false_type{});
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

// 33 to 128 rows that arrive quantized, on the re-tiled int8 filter (`tile16x64`): the filter is
// streamed ONCE, as in the decode GEMV, where the matrix-core GEMM of the prefill regime cuts a
// launch of this size into too few workgroups to reach the memory system's rate (14336 x 4096:
// 112 or 224 workgroups behind one barrier per 128 depth).
//
// A workgroup of eight wavefronts owns four 16-channel tiles over the whole depth. The rows do
// not fit LDS at once (128 rows x 4096 = 512 KB), so the depth is walked in chunks of 64 / RT
// slabs (RT = 16-row tiles per weight tile: 4 or 8), and each chunk's rows (64 KB) are staged in
// one of two LDS buffers while the other is multiplied: global -> registers at the top of a
// chunk, registers -> LDS behind its products, one barrier per chunk. Inside a chunk a wavefront
// takes a PAIR of channel tiles over a quarter of the chunk's depth, so that every row operand
// read from LDS feeds two products (LDS bandwidth is what bounds a compute unit here: at eight
// row tiles, 8 KB of operands per KB of weights without the pairing). Weights go from global
// memory straight to registers through a ring of two chunks' worth of 1 KiB tiles per wavefront;
// every turn of the chunk loop issues the same loads in the same order (past the end: one
// 16-byte piece), so the compiler's waits are exact. 224 workgroups for 14336 channels: one
// round on 256 compute units, each staging the rows once, which keeps the L2-to-LDS traffic at
// rows x depth x 224 (57 MB at 64 rows).
//
// int32 accumulation is exact, so the result is that of the other kernels bit for bit; the
// epilogue's arithmetic is the shared one (fc_epilogues.h).
#include "fc_epilogues.h"
#include "kernels.h"

namespace lrtfc {
namespace {

constexpr int kRowsWaves = 8;
constexpr int kRowsThreads = kRowsWaves * kWaveSize;
constexpr int kTileRows = 16;
constexpr int kSlabDepth = 64;
constexpr int kRowPad = 16;  // bytes behind a staged row: spreads the rows over the LDS banks

template <int RT>
struct RowsShape {
  static constexpr int kChunkSlabs = 64 / RT;             // 16 (1024 deep) or 8 (512 deep)
  static constexpr int kQuarter = kChunkSlabs / 4;        // slabs per wavefront and chunk
  static constexpr int kRing = 2 * kQuarter;              // weight tiles per wavefront and chunk
  static constexpr int kRows = RT * kTileRows;
  static constexpr int kStride = kChunkSlabs * kSlabDepth + kRowPad;
  static constexpr int kBufferBytes = kRows * kStride;
  // 16-byte pieces of a chunk's rows per thread
  static constexpr int kPieces = kRows * kChunkSlabs * kSlabDepth / (kRowsThreads * 16);
  // The partial sums of all eight wavefronts meet in the two row buffers at the end.
  static_assert(kRowsWaves * 2 * RT * 1024 <= 2 * kBufferBytes, "partial sums do not fit");
};

template <Int8Epilogue EPI, int RT>
__global__ __launch_bounds__(kRowsThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void FcInt8RowsGemvKernel(FcInt8Args a, int slabs, int batch0, int bt) {
  using S = RowsShape<RT>;
  extern __shared__ __align__(16) int8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWaveSize);
  const int col = lane & 15;
  const int kgroup = lane >> 4;
  const int depth = a.depth;
  const int tiles = (a.out_depth + kTileRows - 1) / kTileRows;
  const int pair = wave >> 2;  // which two of the workgroup's four tiles
  const int part = wave & 3;   // which quarter of every chunk's depth
  const int tile0 = blockIdx.x * 4 + pair * 2;
  const int chunks = (slabs + S::kChunkSlabs - 1) / S::kChunkSlabs;
  const int8_t* tile_base[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    tile_base[u] = a.filter + static_cast<size_t>(min(tile0 + u, tiles - 1)) * slabs * 1024;
  }

  // Slab s of this wavefront's quarter of chunk c, of tile u of its pair. Every turn of the chunk
  // loop requests two chunks ahead, so the last two turns ask past the depth: those requests all
  // read one 16-byte piece (a cache hit that moves no data), and their product meets zeros in LDS.
  auto request = [&](int c, int s, int u) {
    const int slab = min(c * S::kChunkSlabs + part * S::kQuarter + s, slabs - 1);
    const size_t at = c < chunks ? static_cast<size_t>(slab) * 1024 + lane * 16 : 0;
    return __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(tile_base[u] + at));
  };
  // Piece p of a chunk's rows: row p / (pieces per row), 16 bytes at depth 16 * (p % ...). Past
  // the last chunk: one piece for all, as above.
  constexpr int kPiecesPerRow = S::kChunkSlabs * kSlabDepth / 16;
  i32x4 staged[S::kPieces];
  auto load_rows = [&](int c) {
#pragma unroll
    for (int j = 0; j < S::kPieces; ++j) {
      const int p = j * kRowsThreads + tid;
      const int row = min(p / kPiecesPerRow, bt - 1);  // rows past the batch: a copy, never stored
      const int at = c * S::kChunkSlabs * kSlabDepth + (p % kPiecesPerRow) * 16;
      const size_t from = c < chunks ? static_cast<size_t>(batch0 + row) * depth + min(at, depth - 16)
                                     : static_cast<size_t>(batch0) * depth;
      staged[j] = *reinterpret_cast<const i32x4*>(a.input + from);
    }
  };
  auto store_rows = [&](int c, int8_t* buffer) {
#pragma unroll
    for (int j = 0; j < S::kPieces; ++j) {
      const int p = j * kRowsThreads + tid;
      const int piece = p % kPiecesPerRow;
      const int at = c * S::kChunkSlabs * kSlabDepth + piece * 16;
      *reinterpret_cast<i32x4*>(buffer + (p / kPiecesPerRow) * S::kStride + piece * 16) =
          at < depth ? staged[j] : i32x4{0, 0, 0, 0};
    }
  };

  // The epilogue's constants, requested ahead of the depth walk. A wavefront finishes the row
  // tiles of its own parity (r % 2 == part % 2) of ONE tile of its pair: parts 0 and 1 the first.
  const int tile = tile0 + (part >> 1);
  const int n0 = tile * kTileRows + 4 * kgroup;  // this lane's four channels: n0 .. n0 + 3
  float ep_scale[4], ep_bias[4];
  int32_t ep_sum[4], ep_mult[4], ep_shift[4], ep_bias_i[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = min(n0 + i, a.out_depth - 1);
    ep_sum[i] = a.filter_row_sums ? a.filter_row_sums[n] : 0;
    if (EPI == Int8Epilogue::kRequantize) {
      ep_mult[i] = a.multipliers[a.per_channel ? n : 0];
      ep_shift[i] = a.shifts[a.per_channel ? n : 0];
      ep_bias_i[i] = a.bias_i32 ? a.bias_i32[n] : 0;
    } else {
      ep_scale[i] = a.per_channel_scales ? a.per_channel_scales[n] : a.filter_scale;
      ep_bias[i] = a.bias_f32 ? a.bias_f32[n] : 0.0f;
    }
  }
  float row_scale[RT / 2];
  int32_t row_zp[RT / 2];
  if (EPI != Int8Epilogue::kRequantize) {
#pragma unroll
    for (int rr = 0; rr < RT / 2; ++rr) {
      const int b = batch0 + min(col + kTileRows * (2 * rr + (part & 1)), bt - 1);
      row_scale[rr] = a.scaling_factors[b];
      row_zp[rr] = a.zero_points ? a.zero_points[b] : 0;
    }
  }

  i32x4 ring[2][S::kRing];
  load_rows(0);
#pragma unroll
  for (int j = 0; j < S::kRing; ++j) ring[0][j] = request(0, j >> 1, j & 1);
#pragma unroll
  for (int j = 0; j < S::kRing; ++j) ring[1][j] = request(1, j >> 1, j & 1);
  store_rows(0, smem);
  __syncthreads();

  i32x4 acc[2][RT];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[u][r] = i32x4{0, 0, 0, 0};
  }
  const int operand_at = col * S::kStride + part * S::kQuarter * kSlabDepth + kgroup * 16;
  // One chunk: rows of the next chunk on their way, this chunk's products (each consumed ring
  // slot is requested again for the chunk after next), the next rows into the other buffer.
  auto chunk = [&](int c, auto parity_c) {
    constexpr int kParity = decltype(parity_c)::value;
    const int8_t* buffer = smem + kParity * S::kBufferBytes;
    load_rows(c + 1);
    // The rows are requested BEFORE this chunk's weight requests: waiting for them at the end of
    // the chunk then leaves the weight requests in flight (loads return in order).
    __builtin_amdgcn_sched_barrier(0);
    // The operands of step s + 1 are read from LDS while step s multiplies; the fences keep the
    // compiler from reading a whole chunk's operands ahead.
    i32x4 operand[2][RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      operand[0][r] = *reinterpret_cast<const i32x4*>(buffer + operand_at + r * kTileRows * S::kStride);
    }
#pragma unroll
    for (int s = 0; s < S::kQuarter; ++s) {
      if (s + 1 < S::kQuarter) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
          operand[(s + 1) & 1][r] = *reinterpret_cast<const i32x4*>(
              buffer + operand_at + r * kTileRows * S::kStride + (s + 1) * kSlabDepth);
        }
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
          acc[u][r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ring[kParity][2 * s + u],
                                                            operand[s & 1][r], acc[u][r], 0, 0, 0);
        }
      }
      // Requested again behind their last product, so that the loads may land in the registers
      // the tiles occupied (requested ahead of it they need others, and the loop's back edge
      // then copies every tile home behind a full wait).
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 2; ++u) ring[kParity][2 * s + u] = request(c + 2, s, u);
      __builtin_amdgcn_sched_barrier(0);
    }
    // Nothing of the staging (its zero-fill selects wait for the rows just requested) may move
    // up into the products.
    __builtin_amdgcn_sched_barrier(0);
    store_rows(c + 1, smem + (1 - kParity) * S::kBufferBytes);
    __syncthreads();
  };
  // Always in pairs, so that every turn of the loop is the same straight line: with an odd count
  // the last chunk of the last pair multiplies (finite) weights by the zeros that store_rows puts
  // behind the depth.
  for (int c = 0; c < chunks; c += 2) {
    chunk(c, std::integral_constant<int, 0>{});
    chunk(c + 1, std::integral_constant<int, 1>{});
  }

  // The four quarters of a tile's depth meet in LDS (the row buffers are free now): every
  // wavefront leaves all its sums there and adds up the ones it finishes.
  i32x4* partial = reinterpret_cast<i32x4*>(smem);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
#pragma unroll
    for (int r = 0; r < RT; ++r) partial[((wave * 2 + u) * RT + r) * 64 + lane] = acc[u][r];
  }
  __syncthreads();
  if (tile >= tiles) return;
  // A lane holds four neighbouring channels of one row: one 16-byte (int8: 4-byte) store.
#pragma unroll
  for (int rr = 0; rr < RT / 2; ++rr) {
    const int r = 2 * rr + (part & 1);
    i32x4 sum = i32x4{0, 0, 0, 0};
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      sum += partial[(((pair * 4 + p) * 2 + (part >> 1)) * RT + r) * 64 + lane];
    }
    const int row = col + kTileRows * r;
    if (row >= bt) continue;
    const int b = batch0 + row;
    if (EPI == Int8Epilogue::kRequantize) {
      // StoreRequantized with a zero filter offset
      int32_t q[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        q[i] = RequantizeCore(sum[i] + a.input_offset * ep_sum[i] + ep_bias_i[i], ep_mult[i],
                              ep_shift[i], a.output_offset, a.act_min, a.act_max);
      }
      int8_t* out = a.output_i8 + static_cast<size_t>(b) * a.out_depth + n0;
      if (n0 + 4 <= a.out_depth && (reinterpret_cast<uintptr_t>(out) & 3) == 0) {
        *reinterpret_cast<int32_t*>(out) = PackLowBytes(q[0], q[1], q[2], q[3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (n0 + i < a.out_depth) out[i] = static_cast<int8_t>(q[i]);
        }
      }
      continue;
    }
    const float batch_scale = row_scale[rr];
    const int32_t batch_zp = row_zp[rr];
    float value[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (EPI == Int8Epilogue::kHybrid) {
        value[i] = HybridCoreZeroAware(a, sum[i], batch_scale, ep_scale[i], batch_zp,
                                       batch_zp != 0 ? ep_sum[i] : 0, ep_bias[i]);
      } else {
        value[i] = Hybrid4BitCore(sum[i], batch_scale, ep_scale[i], batch_zp, ep_bias[i],
                                  a.bias_f32 != nullptr, a.activation);
      }
    }
    float* out = a.output_f32 + static_cast<size_t>(b) * a.out_depth + n0;
    if (n0 + 4 <= a.out_depth && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
      *reinterpret_cast<float4*>(out) = make_float4(value[0], value[1], value[2], value[3]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n0 + i < a.out_depth) out[i] = value[i];
      }
    }
  }
}

template <Int8Epilogue EPI, int RT>
hipError_t LaunchRows(const FcInt8Args& a, int batch0, int bt, hipStream_t stream) {
  const size_t lds = 2 * static_cast<size_t>(RowsShape<RT>::kBufferBytes);
  auto kernel = FcInt8RowsGemvKernel<EPI, RT>;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds)) return err;
  const int tiles = (a.out_depth + kTileRows - 1) / kTileRows;
  const int slabs = (a.depth + kSlabDepth - 1) / kSlabDepth;
  hipLaunchKernelGGL(kernel, dim3((tiles + 3) / 4), dim3(kRowsThreads), lds, stream, a, slabs,
                     batch0, bt);
  return hipGetLastError();
}

template <Int8Epilogue EPI>
hipError_t LaunchRowsEpilogue(const FcInt8Args& a, hipStream_t stream) {
  // Passes of at most 128 rows; a pass of up to 64 rows takes four row tiles per weight tile.
  for (int batch0 = 0; batch0 < a.batches; batch0 += 128) {
    const int bt = min(128, a.batches - batch0);
    const hipError_t err = bt <= 64 ? LaunchRows<EPI, 4>(a, batch0, bt, stream)
                                    : LaunchRows<EPI, 8>(a, batch0, bt, stream);
    if (err != hipSuccess) return err;
  }
  return hipSuccess;
}

}  // namespace

bool FcInt8RowsGemvTakes(const FcInt8Args& a) {
  // Wide filters only: four channel tiles per workgroup must still give the chip a round of
  // workgroups, and the chunked walk wants a few chunks of depth.
  const int tiles = (a.out_depth + kTileRows - 1) / kTileRows;
  return a.batches > 32 && a.batches <= 128 && a.filter_offset == 0 && a.depth >= 1024 &&
         a.depth % 16 == 0 && tiles >= 4 * 160 &&
         (reinterpret_cast<uintptr_t>(a.input) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(a.filter) & 15) == 0;
}

hipError_t LaunchFcInt8RowsGemv(const FcInt8Args& a, Int8Epilogue epilogue, hipStream_t stream) {
  if (!FcInt8RowsGemvTakes(a)) return hipErrorNotSupported;
  if (epilogue == Int8Epilogue::kRequantize) {
    return LaunchRowsEpilogue<Int8Epilogue::kRequantize>(a, stream);
  }
  if (epilogue == Int8Epilogue::kHybrid4Bit) {
    return LaunchRowsEpilogue<Int8Epilogue::kHybrid4Bit>(a, stream);
  }
  return LaunchRowsEpilogue<Int8Epilogue::kHybrid>(a, stream);
}

}  // namespace lrtfc

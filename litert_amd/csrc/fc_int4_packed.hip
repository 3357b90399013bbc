// Blockwise-int4 FULLY_CONNECTED (EvalBlockwise4Bit, tflite/kernels/fully_connected.cc
// :1014-1086) on a re-tiled filter, block size 32: the streaming form used for decode.
//
// HBM layout ("tile8x64b", built once per constant filter by PackInt4BlockwiseKernel):
// the filter is cut into tiles of 8 output channels x 64 quantization blocks (2048
// depth). A tile is nine consecutive 1 KiB planes: plane j < 8 holds, for lane L, the 16
// bytes (32 nibbles) of channel j, block L; plane 8 holds, for lane L, the eight fp16
// scales of block L for the tile's channels. Nibbles are stored as (w + 8), i.e. XOR 8,
// so that they are small positive bytes for dot4; tiles of one channel group are
// consecutive along the depth. Every load instruction of a wavefront therefore reads
// 1 KiB of consecutive bytes, weights and scales alike, and one lane finishes a block's
// int32 sum alone (8 dot4): sum(w * q) = dot4(w + 8, q) - 8 * sum(q).
//
// A wavefront owns 8 channels over the whole depth. All loads of its first two tiles go
// out first (a ring that is refilled tile by tile for deeper filters); the activation
// rows are quantized (BatchQuantizeFloats, always asymmetric on this path) and staged in
// LDS, split into planes of high and low nibbles that line up with the filter's dwords,
// while the ring fills. The reference then adds float(block_sum) * scale over the blocks
// of a row in block order in float32; that order is kept: the products of a tile are
// parked in LDS and 8 x batch lanes walk them in order, tile after tile, each walk
// overlapping the wait for the next tile's bytes.
#include <type_traits>

#include "kernels.h"
#include "quantize_device.h"

namespace lrtfc {
namespace {

#define LRTFC_GLOBAL __attribute__((address_space(1)))
using f32x4 = float __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWaveSize;
constexpr int kBlock = 32;       // weights per quantization block
constexpr int kTileRows = 8;
constexpr int kTileBlocks = 64;
constexpr int kPlanes = kTileRows + 1;
constexpr int kTileBytes = kPlanes * 1024;
constexpr int kTileVecs = kPlanes * 64;  // i32x4 per tile
constexpr int kRingTiles = 2;
constexpr int kPStride = kTileBlocks + 4;  // floats per (row, batch) line of parked products
constexpr int kMaxGroupNodes = LRTFC_INT4_GROUP_MAX;
constexpr int kMaxGroupsPerWave = 8;  // 64 channels: one lane each when their kfsum is staged
constexpr int kSplitShallowMinBlocks = 1024;  // grouped launches: see PrepareInt4Group
constexpr int kRowPairsSideBySide = 2;        // lrtfc_int4_group_launch.split_quantize
constexpr int kSideBySideMaxBlocks = 256;
constexpr int64_t kSideBySideMaxFilterBytes = 24 << 20;

__global__ __launch_bounds__(kThreads) void PackInt4BlockwiseKernel(
    const uint8_t* __restrict__ filter, const uint16_t* __restrict__ scales, int out_depth,
    int depth, int chunks, int64_t total_vecs, uint8_t* __restrict__ dst) {
  const int64_t v = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (v >= total_vecs) return;
  const int lane = static_cast<int>(v & 63);
  const int64_t plane_index = v >> 6;
  const int plane = static_cast<int>(plane_index % kPlanes);
  const int64_t tile = plane_index / kPlanes;
  const int chunk = static_cast<int>(tile % chunks);
  const int group = static_cast<int>(tile / chunks);
  const int nblk = depth / kBlock;
  const int blk = chunk * kTileBlocks + lane;
  const size_t row_bytes = static_cast<size_t>(depth) / 2;
  uint8_t out[16];
  if (plane < kTileRows) {
    const int row = group * kTileRows + plane;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      uint8_t byte = 0;  // weight 0, weight 0
      if (row < out_depth && blk < nblk) byte = filter[row * row_bytes + blk * 16 + t];
      out[t] = byte ^ 0x88;
    }
  } else {
#pragma unroll
    for (int j = 0; j < kTileRows; ++j) {
      const int row = group * kTileRows + j;
      uint16_t s = 0;
      if (row < out_depth && blk < nblk) s = scales[static_cast<size_t>(row) * nblk + blk];
      out[2 * j] = static_cast<uint8_t>(s & 0xFF);
      out[2 * j + 1] = static_cast<uint8_t>(s >> 8);
    }
  }
  *reinterpret_cast<i32x4*>(dst + v * 16) = *reinterpret_cast<const i32x4*>(out);
}

struct Int4PackedArgs {
  const uint8_t* packed;       // tile8x64b
  const float* input_f32;      // fused form
  const int8_t* input_q;       // unfused form: quantized rows + their scales / zero points
  const float* scaling_factors;
  const int32_t* zero_points;
  const float* kfsum;
  const float* bias;
  float* output;
  int batches, depth, out_depth, chunks;
};

// Nibble planes of eight consecutive int8 activations (lo = q0..q3, hi = q4..q7 as packed
// bytes): `high` holds (q >> 4) & 15 and `low` holds q & 15 of element i in bits 4i .. 4i + 3,
// the order in which a dword of the filter holds its eight weights. With q = 16 * qh + ql
// (qh signed, ql unsigned) a block's sum(w * q) is 16 * sdot8(w, qh) + udot8(w + 8, ql) -
// 8 * sum(ql): eight 8-way dot products per 32 weights and no nibble unpacking at all.
__device__ __forceinline__ uint32_t CompressNibbles(uint32_t t) {  // bytes 0x0n -> 16 bits
  t = (t | (t >> 4)) & 0x00FF00FFu;
  return (t | (t >> 8)) & 0xFFFFu;
}
__device__ __forceinline__ void NibblePlanes(uint32_t lo, uint32_t hi, int32_t* high,
                                             int32_t* low) {
  *low = static_cast<int32_t>(CompressNibbles(lo & 0x0F0F0F0Fu) |
                              (CompressNibbles(hi & 0x0F0F0F0Fu) << 16));
  *high = static_cast<int32_t>(CompressNibbles((lo >> 4) & 0x0F0F0F0Fu) |
                               (CompressNibbles((hi >> 4) & 0x0F0F0F0Fu) << 16));
}
__device__ __forceinline__ int32_t SDot8(int32_t a, int32_t b, int32_t acc) {
  return __builtin_amdgcn_sdot8(a, b, acc, false);
}
__device__ __forceinline__ uint32_t UDot8(uint32_t a, uint32_t b, uint32_t acc) {
  return __builtin_amdgcn_udot8(a, b, acc, false);
}

// LDS map: [BT][padded depth] activations as nibble planes (per block of 32: four dwords of
// high nibbles, then four of low nibbles); per wavefront [8 * BT][kPStride]
// parked products; per-row quantization state.
template <int BT>
struct Int4Shared {
  int32_t* q;   // dwords: per row padded_depth / 4
  float* p;     // [waves][8 * BT][kPStride]
  float* sf;    // [BT]
  float* inv;   // [BT]
  int32_t* zp;  // [BT]
  int32_t* zero;
  float* mm;    // [BT][waves][2]
  float* kb;    // [waves][2][64]: kfsum and bias of the channels a wavefront covers
  float* ob;    // [waves][64 * BT]: finished outputs of those channels
  // Floats of parked products: one tile per wavefront when a wavefront owns a channel group
  // alone; every tile of the group when `ksplit` wavefronts share it (the ordered walk then
  // needs them all).
  __host__ __device__ static size_t ProductFloats(int chunks, int ksplit) {
    constexpr int waves = kWaves;
    const size_t tile = static_cast<size_t>(8) * BT * kPStride;
    return ksplit == 1 ? waves * tile : (waves / ksplit) * static_cast<size_t>(chunks) * tile;
  }
  __device__ Int4Shared(int8_t* base, int padded, int chunks, int ksplit) {
    constexpr int waves = kWaves;
    q = reinterpret_cast<int32_t*>(base);
    size_t off = static_cast<size_t>(BT) * padded;
    p = reinterpret_cast<float*>(base + off);
    off += ProductFloats(chunks, ksplit) * 4;
    sf = reinterpret_cast<float*>(base + off);
    inv = sf + 8;
    zp = reinterpret_cast<int32_t*>(inv + 8);
    zero = zp + 8;
    mm = reinterpret_cast<float*>(zero + 8);
    kb = mm + BT * waves * 2;
    ob = kb + waves * 2 * 64;
  }
  static size_t Bytes(int padded, int ksplit) {
    constexpr int waves = kWaves;
    const int chunks = padded / (kTileBlocks * kBlock);
    return static_cast<size_t>(BT) * padded + ProductFloats(chunks, ksplit) * 4 + 4 * 8 * 4 +
           BT * waves * 2 * 4 + waves * 2 * 64 * 4 + waves * 64 * BT * 4;
  }
};

// GPT: groups of 8 depth positions each thread keeps in registers between the two passes of
// the prologue; the register form covers depth <= GPT * 256 * 8.
// The work of one workgroup; `block` is its index among the workgroups of this filter.
// gpw: consecutive channel groups one wavefront works through (ksplit == 1 only). Their
// tiles are one contiguous stretch of the filter, so the ring of loads runs on across group
// boundaries and the prologue (the row quantizer) is paid once for all of them.
// ALL > 0: a wavefront has at most ALL tiles (ksplit == 1, gpw * chunks <= ALL) and requests
// every one of them before it does anything else: no refills, one memory round trip per
// wavefront, and straight-line code whose waits for each tile are exact.
template <int N, class F>
__device__ __forceinline__ void StaticFor(F&& f) {
  if constexpr (N > 0) {
    StaticFor<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// PRE of them go out ahead of the prologue, the rest behind it: a compute unit accepts only
// some tens of KiB of outstanding loads, and a wavefront whose load issue blocks cannot do its
// share of the row quantizer (14336 x 4096, one row: two tiles per wavefront, one ahead, 8.3 us;
// both ahead 9.0 us; four tiles per wavefront all ahead 9.9 us; the refilled ring of two 8.5 us).
template <int BT, bool FUSED, int VARIANT, int GPT, int ALL = 0, int PRE = 0>
__device__ __forceinline__ void FcInt4PackedBody(const Int4PackedArgs& a, int block, int batch0,
                                                 int bt, int ksplit, int gpw, int8_t* smem) {

  // Every tensor is in global memory. Pointers that a kernel read from a table in memory
  // carry no address space, and accesses through them would go the flat path, whose waits
  // cannot leave a ring of loads in flight; so the address space is stated here.
  const LRTFC_GLOBAL i32x4* g_packed = (const LRTFC_GLOBAL i32x4*)a.packed;
  const LRTFC_GLOBAL float* g_input_f32 = (const LRTFC_GLOBAL float*)a.input_f32;
  const LRTFC_GLOBAL int8_t* g_input_q = (const LRTFC_GLOBAL int8_t*)a.input_q;
  const LRTFC_GLOBAL float* g_scaling_factors = (const LRTFC_GLOBAL float*)a.scaling_factors;
  const LRTFC_GLOBAL int32_t* g_zero_points = (const LRTFC_GLOBAL int32_t*)a.zero_points;
  const LRTFC_GLOBAL float* g_kfsum = (const LRTFC_GLOBAL float*)a.kfsum;
  const LRTFC_GLOBAL float* g_bias = (const LRTFC_GLOBAL float*)a.bias;
  LRTFC_GLOBAL float* g_output = (LRTFC_GLOBAL float*)a.output;
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = tid / kWaveSize;
  const int depth = a.depth;
  const int chunks = a.chunks;
  const int padded = chunks * kTileBlocks * kBlock;  // depth padded to whole tiles
  const int groups = (a.out_depth + kTileRows - 1) / kTileRows;
  // ksplit wavefronts share one channel group and take its tiles round-robin (deep, narrow
  // filters would otherwise leave most of the chip without a wavefront).
  const int kpart = wave % ksplit;
  const int group_in_wg = wave / ksplit;
  const int group0 = (block * (kWaves / ksplit) + group_in_wg) * gpw;  // may run past the last
  const int my_groups = max(0, min(gpw, groups - group0));
  const int ntiles = my_groups * chunks;  // tiles of this wavefront and its depth partners
  const int first_group = min(group0, groups - 1);
  const LRTFC_GLOBAL i32x4* tbase = g_packed +
                       static_cast<size_t>(first_group) * chunks * kTileVecs + lane;
  Int4Shared<BT> sh(smem, padded, chunks, ksplit);
  // Per-channel epilogue inputs of every channel this wavefront covers (lane = channel),
  // requested ahead of the weights and parked in LDS once the prologue is through.
  const int my_n = min(first_group * kTileRows + lane, a.out_depth - 1);
  const float kfsum_raw = g_kfsum[my_n];
  const float bias_raw = a.bias ? g_bias[my_n] : 0.0f;

  // Activation loads first (raw, branch-free): whatever the prologue waits for must be
  // requested before the weight ring, because vector memory returns in issue order.
  // Each thread owns groups of 8 consecutive depth positions: g = tid + 256 * j.
  constexpr int kGroupsPerThread = GPT;
  float4 xr[BT][kGroupsPerThread][2];
  i32x2 qr[BT][kGroupsPerThread];
  const int groups8 = depth / 8;
  bool in_regs;
  if (FUSED) {
    in_regs = ((reinterpret_cast<uintptr_t>(a.input_f32) & 15) == 0) &&
              groups8 <= kGroupsPerThread * kThreads;
    if (in_regs) {
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        const LRTFC_GLOBAL float* x = g_input_f32 + static_cast<size_t>(batch0 + min(b, bt - 1)) * depth;
#pragma unroll
        for (int j = 0; j < kGroupsPerThread; ++j) {
          const int g = min(j * kThreads + tid, groups8 - 1);
          const f32x4 lo = *reinterpret_cast<const LRTFC_GLOBAL f32x4*>(x + g * 8);
          const f32x4 hi = *reinterpret_cast<const LRTFC_GLOBAL f32x4*>(x + g * 8 + 4);
          xr[b][j][0] = make_float4(lo.x, lo.y, lo.z, lo.w);
          xr[b][j][1] = make_float4(hi.x, hi.y, hi.z, hi.w);
        }
      }
    } else {
      for (int b = 0; b < bt; ++b) {  // slow form: min/max from memory before the ring
        const LRTFC_GLOBAL float* x = g_input_f32 + static_cast<size_t>(batch0 + b) * depth;
        float mn = 0.0f, mx = 0.0f;
        for (int i = tid; i < depth; i += kThreads) {
          mn = fminf(mn, x[i]);
          mx = fmaxf(mx, x[i]);
        }
        mn = WaveMinF32(mn);
        mx = WaveMaxF32(mx);
        if (lane == 0) {
          sh.mm[(b * kWaves + wave) * 2] = mn;
          sh.mm[(b * kWaves + wave) * 2 + 1] = mx;
        }
      }
    }
  } else {
    in_regs = ((reinterpret_cast<uintptr_t>(a.input_q) & 7) == 0) &&
              groups8 <= kGroupsPerThread * kThreads;
    if (in_regs) {
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        const LRTFC_GLOBAL int8_t* x = g_input_q + static_cast<size_t>(batch0 + min(b, bt - 1)) * depth;
#pragma unroll
        for (int j = 0; j < kGroupsPerThread; ++j) {
          const int g = min(j * kThreads + tid, groups8 - 1);
          qr[b][j] = *reinterpret_cast<const LRTFC_GLOBAL i32x2*>(x + g * 8);
        }
      }
    } else {
      for (int b = 0; b < bt; ++b) {
        const LRTFC_GLOBAL int8_t* x = g_input_q + static_cast<size_t>(batch0 + b) * depth;
        for (int g = tid; g < padded / 8; g += kThreads) {
          uint32_t lo = 0, hi = 0;
          if (g < groups8) {
            for (int t = 0; t < 4; ++t) {
              lo |= static_cast<uint32_t>(static_cast<uint8_t>(x[g * 8 + t])) << (8 * t);
              hi |= static_cast<uint32_t>(static_cast<uint8_t>(x[g * 8 + 4 + t])) << (8 * t);
            }
          }
          int32_t high, low;
          NibblePlanes(lo, hi, &high, &low);
          sh.q[b * (padded / 4) + (g >> 2) * 8 + (g & 3)] = high;
          sh.q[b * (padded / 4) + (g >> 2) * 8 + 4 + (g & 3)] = low;
        }
      }
    }
  }

  // The ring: two tiles (18 KiB) per wavefront in flight. With several batch rows the second
  // tile is requested after the prologue's arithmetic, which then overlaps the time load issue
  // spends blocked on a full memory pipeline (measured: 15.4 -> 14.2 us at four rows); with one
  // row the prologue is too short for that to pay (9.0 -> 9.5 us), so both go out at once.
  constexpr int kRing = ALL > 0 ? ALL : kRingTiles;
  i32x4 ring[kRing][kPlanes];
  auto request_tile = [&](int t) {
    const int lin = min(kpart + t * ksplit, max(ntiles, 1) - 1);
    // The plane of scales goes first: loads return in issue order, so the rows of a tile can
    // then be worked through as they arrive instead of after the whole tile.
#pragma unroll
    for (int jj = 0; jj < kPlanes; ++jj) {
      const int j = (jj + kTileRows) % kPlanes;
      ring[t][j] =
          __builtin_nontemporal_load(tbase + static_cast<size_t>(lin) * kTileVecs + j * 64);
    }
  };
  constexpr int kPre = ALL > 0 ? PRE : (BT == 1 ? kRing : 1);
#pragma unroll
  for (int t = 0; t < kPre; ++t) request_tile(t);
  // Chain lanes: lane = row * BT + batch.
  const int chain_row = lane / BT;
  const int chain_b = lane - chain_row * BT;
  const bool chain_lane = lane < kTileRows * BT;

  // Activation rows into LDS.
  if (FUSED) {
    if (in_regs) {
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        float mn = 0.0f, mx = 0.0f;
#pragma unroll
        for (int j = 0; j < kGroupsPerThread; ++j) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const float4 t = xr[b][j][h];  // clamped duplicates past the row are harmless here
            mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
            mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
          }
        }
        mn = WaveMinF32(mn);
        mx = WaveMaxF32(mx);
        if (lane == 0) {
          sh.mm[(b * kWaves + wave) * 2] = mn;
          sh.mm[(b * kWaves + wave) * 2 + 1] = mx;
        }
      }
    }
    __syncthreads();
    if (tid < bt) {
      float mn = sh.mm[tid * kWaves * 2], mx = sh.mm[tid * kWaves * 2 + 1];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) {
        mn = fminf(mn, sh.mm[(tid * kWaves + w) * 2]);
        mx = fmaxf(mx, sh.mm[(tid * kWaves + w) * 2 + 1]);
      }
      const RowQuantParams qp = AsymmetricRowParams<VARIANT>(mn, mx);
      sh.sf[tid] = qp.scale;
      sh.inv[tid] = ElementwiseInv(qp);
      sh.zp[tid] = qp.zero_point;
      sh.zero[tid] = qp.all_zero ? 1 : 0;
    }
    __syncthreads();
    const int vector_end = depth - (depth % 8);
    if (in_regs) {
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        if (b < bt) {
          RowQuantParams qp;
          qp.scale = sh.sf[b];
          qp.inv = sh.inv[b];
          qp.zero_point = sh.zp[b];
          qp.all_zero = sh.zero[b] != 0;
#pragma unroll
          for (int j = 0; j < kGroupsPerThread; ++j) {
            const int g = j * kThreads + tid;
            if (g < padded / 8) {
              int32_t high = 0, low = 0;
              if (g < groups8) {
                const float4 lo = xr[b][j][0], hi = xr[b][j][1];
                const bool tail = g * 8 >= vector_end;
                NibblePlanes(
                    static_cast<uint32_t>(QuantizePack4<VARIANT>(lo.x, lo.y, lo.z, lo.w, qp, tail)),
                    static_cast<uint32_t>(QuantizePack4<VARIANT>(hi.x, hi.y, hi.z, hi.w, qp, tail)),
                    &high, &low);
              }
              sh.q[b * (padded / 4) + (g >> 2) * 8 + (g & 3)] = high;
              sh.q[b * (padded / 4) + (g >> 2) * 8 + 4 + (g & 3)] = low;
            }
          }
        }
      }
    } else {
      for (int b = 0; b < bt; ++b) {
        const LRTFC_GLOBAL float* x = g_input_f32 + static_cast<size_t>(batch0 + b) * depth;
        RowQuantParams qp;
        qp.scale = sh.sf[b];
        qp.inv = sh.inv[b];
        qp.zero_point = sh.zp[b];
        qp.all_zero = sh.zero[b] != 0;
        for (int g = tid; g < padded / 8; g += kThreads) {
          int32_t v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
          if (g < groups8) {
            for (int t = 0; t < 8; ++t) {
              v[t] = QuantizeElement<VARIANT>(x[g * 8 + t], qp, true, g * 8 + t >= vector_end);
            }
          }
          int32_t high, low;
          NibblePlanes(static_cast<uint32_t>(PackBytes(v[0], v[1], v[2], v[3])),
                       static_cast<uint32_t>(PackBytes(v[4], v[5], v[6], v[7])), &high, &low);
          sh.q[b * (padded / 4) + (g >> 2) * 8 + (g & 3)] = high;
          sh.q[b * (padded / 4) + (g >> 2) * 8 + 4 + (g & 3)] = low;
        }
      }
    }
  } else if (in_regs) {
#pragma unroll
    for (int b = 0; b < BT; ++b) {
      if (b < bt) {
#pragma unroll
        for (int j = 0; j < kGroupsPerThread; ++j) {
          const int g = j * kThreads + tid;
          if (g < padded / 8) {
            int32_t high = 0, low = 0;
            if (g < groups8) {
              NibblePlanes(static_cast<uint32_t>(qr[b][j].x), static_cast<uint32_t>(qr[b][j].y),
                           &high, &low);
            }
            sh.q[b * (padded / 4) + (g >> 2) * 8 + (g & 3)] = high;
            sh.q[b * (padded / 4) + (g >> 2) * 8 + 4 + (g & 3)] = low;
          }
        }
      }
    }
  }
  __syncthreads();

#pragma unroll
  for (int t = kPre; t < kRing; ++t) request_tile(t);

  float* kb = sh.kb + wave * 2 * 64;
  kb[lane] = kfsum_raw;
  kb[64 + lane] = bias_raw;

  float row_scale = 0.0f;
  float row_zp = 0.0f;
  if (chain_lane && chain_b < bt) {
    row_scale = FUSED ? sh.sf[chain_b] : g_scaling_factors[batch0 + chain_b];
    row_zp = static_cast<float>(FUSED ? sh.zp[chain_b] : g_zero_points[batch0 + chain_b]);
  }

  // Tile loop. Lane L owns block L of the tile for each of the 8 channels.
  constexpr int kTileFloats = 8 * BT * kPStride;
  float* pgroup = sh.p + static_cast<size_t>(group_in_wg) * chunks * kTileFloats;  // ksplit > 1
  float out = 0.0f;
  const int nblk = depth / kBlock;
  // One tile's 64 products per chain lane, added in block order.
  auto walk_tile = [&](const float* tile, int c) {
    const int count = min(kTileBlocks, nblk - c * kTileBlocks);
    const float* line = tile + lane * kPStride;
    if (count == kTileBlocks) {
      // Whole tile: fetch the 64 products with back-to-back LDS reads, then add in order.
      float4 v[kTileBlocks / 4];
#pragma unroll
      for (int j = 0; j < kTileBlocks / 4; ++j) v[j] = reinterpret_cast<const float4*>(line)[j];
#pragma unroll
      for (int j = 0; j < kTileBlocks / 4; ++j) {
        out = __fadd_rn(out, v[j].x);
        out = __fadd_rn(out, v[j].y);
        out = __fadd_rn(out, v[j].z);
        out = __fadd_rn(out, v[j].w);
      }
    } else {
      for (int j = 0; j < count; ++j) out = __fadd_rn(out, line[j]);
    }
  };
  // fully_connected.cc:1078-1082 for the channel group at offset `goff` from the first. The
  // value is parked in LDS and leaves in one store at the end: a store inside the tile loop
  // would make the number of outstanding memory operations depend on the path taken, and
  // the waits for the ring would have to assume the worst.
  float* ob = sh.ob + wave * (kMaxGroupsPerWave * kTileRows * BT);
  auto finish_group = [&](int goff) {
    float o = __fsub_rn(out, __fmul_rn(row_zp, kb[goff * kTileRows + chain_row]));
    o = __fmul_rn(o, row_scale);
    if (a.bias) o = __fadd_rn(o, kb[64 + goff * kTileRows + chain_row]);
    ob[goff * kTileRows * BT + lane] = o;
  };
  // One tile: ring slot SLOT holds tile `lin` of this wavefront's stretch. REFILL requests the
  // tile two turns ahead into the same slot -- always, so that every turn of the main loop
  // issues the same number of loads and the wait for a slot can leave exactly the other slot's
  // loads in flight; past the end the request goes to one hot cache line instead.
  auto process = [&](auto slot_tag, auto refill_tag, int lin, int c) {
    constexpr int SLOT = decltype(slot_tag)::value;
    constexpr bool REFILL = decltype(refill_tag)::value;
    float* pw = ksplit == 1 ? sh.p + static_cast<size_t>(wave) * kTileFloats
                            : pgroup + static_cast<size_t>(c) * kTileFloats;
    // This block's activations (four dwords of high nibbles, four of low ones, per batch row)
    // and -8 * sum(low nibbles), the seed of the unsigned dot product.
    i32x4 qh[BT], ql[BT];
    uint32_t seed[BT];
    const int blk = c * kTileBlocks + lane;
#pragma unroll
    for (int b = 0; b < BT; ++b) {
      const i32x4* qp = reinterpret_cast<const i32x4*>(sh.q + b * (padded / 4) + blk * 8);
      qh[b] = qp[0];
      ql[b] = qp[1];
      uint32_t t = 0;
#pragma unroll
      for (int d = 0; d < 4; ++d) t = UDot8(static_cast<uint32_t>(ql[b][d]), 0x11111111u, t);
      seed[b] = 0u - 8u * t;
    }
    const i32x4 sc = ring[SLOT][kTileRows];
#pragma unroll
    for (int j = 0; j < kTileRows; ++j) {
      const uint32_t pair = static_cast<uint32_t>(sc[j >> 1]);
      const float scale =
          HalfBitsToFloatFast(static_cast<uint16_t>((j & 1) ? (pair >> 16) : (pair & 0xFFFF)));
      const i32x4 wv = ring[SLOT][j];  // nibbles stored as w + 8
      int32_t ws[4];                   // the same weights as signed nibbles
#pragma unroll
      for (int d = 0; d < 4; ++d) ws[d] = wv[d] ^ static_cast<int32_t>(0x88888888u);
#pragma unroll
      for (int b = 0; b < BT; ++b) {
        int32_t sd = 0;
        uint32_t ud = seed[b];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          sd = SDot8(ws[d], qh[b][d], sd);
          ud = UDot8(static_cast<uint32_t>(wv[d]), static_cast<uint32_t>(ql[b][d]), ud);
        }
        const int32_t acc = (sd << 4) + static_cast<int32_t>(ud);
        pw[(j * BT + b) * kPStride + lane] = __fmul_rn(static_cast<float>(acc), scale);
      }
    }
    if (REFILL) {
      const int next = lin + kRingTiles * ksplit;
      const LRTFC_GLOBAL i32x4* src =
          next < ntiles ? tbase + static_cast<size_t>(next) * kTileVecs : g_packed;
#pragma unroll
      for (int jj = 0; jj < kPlanes; ++jj) {
        const int j = (jj + kTileRows) % kPlanes;
        ring[SLOT][j] = __builtin_nontemporal_load(src + j * 64);
      }
    }
    // Ordered float32 accumulation over this tile's blocks (same wavefront wrote them).
    if (ksplit == 1 && chain_lane) walk_tile(pw, c);
  };
  // Moves on to the next tile of the stretch; closes a channel group after its last tile.
#define LRTFC_INT4_ADVANCE()                      \
  do {                                            \
    if (ksplit == 1) {                            \
      if (++c == chunks) {                        \
        if (chain_lane) finish_group(goff);       \
        out = 0.0f;                               \
        c = 0;                                    \
        ++goff;                                   \
      }                                           \
    } else {                                      \
      c += ksplit;                                \
    }                                             \
  } while (0)
  int c = kpart;  // tile index within the current channel group
  int goff = 0;
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;
  int lin = kpart;
  if constexpr (ALL > 0) {
    StaticFor<ALL>([&](auto t) {
      if (decltype(t)::value < ntiles) {
        process(t, std::false_type{}, decltype(t)::value, c);
        LRTFC_INT4_ADVANCE();
      }
    });
  } else {
    for (; lin + ksplit < ntiles; lin += kRingTiles * ksplit) {
      process(Slot0{}, std::true_type{}, lin, c);
      LRTFC_INT4_ADVANCE();
      process(Slot1{}, std::true_type{}, lin + ksplit, c);
      LRTFC_INT4_ADVANCE();
    }
    if (lin < ntiles) {
      process(Slot0{}, std::false_type{}, lin, c);
      LRTFC_INT4_ADVANCE();
    }
  }
#undef LRTFC_INT4_ADVANCE
  if (ksplit > 1) {
    // Every tile of the group is parked; its first wavefront walks them in depth order.
    __syncthreads();
    if (kpart == 0 && chain_lane && my_groups > 0) {
      for (int cc = 0; cc < chunks; ++cc) {
        walk_tile(pgroup + static_cast<size_t>(cc) * kTileFloats, cc);
      }
      finish_group(0);
    }
  }
  // Outputs of this wavefront's channel groups: index = (group offset, row, batch).
  if (kpart == 0) {
    for (int i = lane; i < my_groups * kTileRows * BT; i += kWaveSize) {
      const int b = i % BT;
      const int row = i / BT;  // channel offset from the first group's first channel
      const int n = group0 * kTileRows + row;
      if (b < bt && n < a.out_depth) {
        g_output[static_cast<size_t>(batch0 + b) * a.out_depth + n] = ob[i];
      }
    }
  }
}

// The leading scalar arguments repeat what the first loads need (filter and row addresses,
// shapes): the library is built with kernel-argument preloading, which hands the leading scalar
// arguments to a wavefront in registers when it starts; the rest of the argument block is read
// from memory as usual while the first loads are already under way.
template <int BT, bool FUSED, int VARIANT, int GPT, int ALL, int PRE>
__global__ __launch_bounds__(kThreads) void FcInt4PackedKernel(
    const uint8_t* early_packed, const float* early_input_f32, const int8_t* early_input_q,
    int early_depth, int early_out_depth, int early_chunks, int batch0, int bt, int ksplit,
    int gpw, Int4PackedArgs rest) {
  extern __shared__ __align__(16) int8_t smem[];
  Int4PackedArgs a = rest;
  a.packed = early_packed;
  a.input_f32 = early_input_f32;
  a.input_q = early_input_q;
  a.depth = early_depth;
  a.out_depth = early_out_depth;
  a.chunks = early_chunks;
  FcInt4PackedBody<BT, FUSED, VARIANT, GPT, ALL, PRE>(a, blockIdx.x, batch0, bt, ksplit, gpw, smem);
}

// Several filters of the same depth in one launch (nodes of a graph that do not depend on
// each other: the q/k/v or gate/up projections of a decoder layer). The table lives in device
// memory: per node its arguments and the index of its first workgroup. One launch instead of
// `count` removes count - 1 launch gaps and lets small filters overlap large ones.
struct Int4GroupTable {
  int first_block[kMaxGroupNodes + 1];
  int reserved[3];
  Int4PackedArgs node[kMaxGroupNodes];
};

template <int BT, bool FUSED, int VARIANT, int GPT>
__global__ __launch_bounds__(kThreads) void FcInt4PackedGroupedKernel(
    const Int4GroupTable* __restrict__ table, int count, int batch0, int bt, int ksplit,
    int gpw) {
  extern __shared__ __align__(16) int8_t smem[];
  // first_block is ascending: the node of this workgroup is the number of later nodes whose
  // first workgroup is not beyond it. Vector loads and ballots (64 nodes per turn) instead of
  // a scalar walk.
  const int lane = threadIdx.x & (kWaveSize - 1);
  int node = 0;
  for (int base = 0; base + 1 < count; base += kWaveSize) {
    const int probe = base + lane + 1;
    const bool not_beyond =
        probe < count && static_cast<int>(blockIdx.x) >= table->first_block[min(probe, count)];
    node += __popcll(__ballot(not_beyond));
  }
  node = __builtin_amdgcn_readfirstlane(node);
  const Int4PackedArgs a = table->node[node];
  // Row tiles side by side (gridDim.y > 1): slice y of the grid takes rows batch0 + y * bt on.
  const int first_row = batch0 + static_cast<int>(blockIdx.y) * bt;
  const int rows = min(bt, a.batches - first_row);
  FcInt4PackedBody<BT, FUSED, VARIANT, GPT>(a, blockIdx.x - table->first_block[node], first_row,
                                            rows, ksplit, gpw, smem);
}

// The row quantizer for a whole group: workgroup r quantizes row r % batches of node
// r / batches into that node's workspace (EvalBlockwise4Bit always quantizes asymmetrically,
// tflite/kernels/fully_connected.cc:1044-1047).
template <int VARIANT, int THREADS = kQuantizeThreads>
__global__ __launch_bounds__(THREADS) void QuantizeGroupRowsKernel(
    const Int4GroupTable* __restrict__ table, int batches) {
  const int node = blockIdx.x / batches;
  const int row = blockIdx.x - node * batches;
  const Int4PackedArgs& a = table->node[node];
  QuantizeRow<VARIANT, RowMajorPlacement, THREADS>(
                       a.input_f32 + static_cast<size_t>(row) * a.depth, a.depth,
                       const_cast<int8_t*>(a.input_q) + static_cast<size_t>(row) * a.depth,
                       const_cast<float*>(a.scaling_factors) + row,
                       const_cast<int32_t*>(a.zero_points) + row, /*do_asymmetric=*/1);
}

// Wavefronts per channel group: one while that already gives the chip ~1000 wavefronts;
// otherwise the depth is shared out, as long as each wavefront keeps at least two tiles.
int ChooseKsplit(int out_depth, int chunks) {
  const int groups = (out_depth + kTileRows - 1) / kTileRows;
  int ksplit = 1;
  while (ksplit < kWaves && groups * ksplit < 1024 && chunks >= 4 * ksplit) ksplit *= 2;
  return ksplit;
}

// Channel groups per wavefront. Measured on launches from 7 MB to 340 MB: a wavefront should
// stream up to 8 tiles (its ring then runs long enough to amortize the prologue), as long as
// the launch keeps about one workgroup per CU (224 of them) to spread over the chip.
int ChooseGroupsPerWave(int total_groups, int chunks, int ksplit) {
  if (ksplit > 1) return 1;
  int gpw = 1;
  while (gpw * 2 <= kMaxGroupsPerWave && gpw * 2 * chunks <= 8 &&
         total_groups / (kWaves * gpw * 2) >= 224) {
    gpw *= 2;
  }
  return gpw;
}

template <int BT, bool FUSED, int VARIANT, int GPT, int ALL, int PRE>
hipError_t LaunchSized(const Int4PackedArgs& a, int batch0, int bt, int ksplit, int gpw,
                       hipStream_t stream) {
  const int padded = a.chunks * kTileBlocks * kBlock;
  const size_t lds = Int4Shared<BT>::Bytes(padded, ksplit);
  auto kernel = FcInt4PackedKernel<BT, FUSED, VARIANT, GPT, ALL, PRE>;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds)) return err;
  const int groups = (a.out_depth + kTileRows - 1) / kTileRows;
  const int groups_per_wg = kWaves / ksplit * gpw;
  const int grid = (groups + groups_per_wg - 1) / groups_per_wg;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, a.packed, a.input_f32,
                     a.input_q, a.depth, a.out_depth, a.chunks, batch0, bt, ksplit, gpw, a);
  return hipGetLastError();
}

// A single node of up to two batch rows whose wavefronts can be given at most two tiles each
// (depth up to 4096) runs the straight-line form: first tile ahead of the prologue, second
// behind it.
constexpr int kStraightTiles = 2;

template <int BT, bool FUSED, int VARIANT, int GPT>
hipError_t LaunchOne(const Int4PackedArgs& a, int batch0, int bt, hipStream_t stream) {
  const int ksplit = ChooseKsplit(a.out_depth, a.chunks);
  const int groups = (a.out_depth + kTileRows - 1) / kTileRows;
  int gpw = ChooseGroupsPerWave(groups, a.chunks, ksplit);
  if constexpr (BT <= 2) {
    if (ksplit == 1 && a.chunks <= kStraightTiles) {
      gpw = min(gpw, kStraightTiles / a.chunks);
      return LaunchSized<BT, FUSED, VARIANT, GPT, kStraightTiles, 1>(a, batch0, bt, ksplit, gpw,
                                                                     stream);
    }
  }
  return LaunchSized<BT, FUSED, VARIANT, GPT, 0, 0>(a, batch0, bt, ksplit, gpw, stream);
}

template <int BT, bool FUSED, int GPT>
hipError_t LaunchVariant(const Int4PackedArgs& a, int variant, int batch0, int bt,
                         hipStream_t stream) {
  if constexpr (!FUSED) {
    return LaunchOne<BT, false, LRTFC_QUANT_PORTABLE, GPT>(a, batch0, bt, stream);
  } else {
    switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      return LaunchOne<BT, FUSED, LRTFC_QUANT_NEON_V8, GPT>(a, batch0, bt, stream);
    case LRTFC_QUANT_NEON_LEGACY:
      return LaunchOne<BT, FUSED, LRTFC_QUANT_NEON_LEGACY, GPT>(a, batch0, bt, stream);
    default:
      return LaunchOne<BT, FUSED, LRTFC_QUANT_PORTABLE, GPT>(a, batch0, bt, stream);
  }
  }
}

// Depth up to 4096 keeps two groups per thread; up to 16384, eight. A fused launch holds
// the float rows (16 registers per group and row), so its deep form stops at two rows.
constexpr int kShallowDepth = 2 * kThreads * 8;
constexpr int kDeepDepth = 8 * kThreads * 8;

template <bool FUSED>
int MaxBatchTile(int depth) {
  return (FUSED && depth > kShallowDepth && depth <= kDeepDepth) ? 2 : 4;
}

// A workgroup may use 160 KB of LDS; the maps below keep 10 KB clear of that.
constexpr size_t kLdsBudget = 150 * 1024;

// Rows per launch: `want` (1, 2 or 4) cut down until the LDS map of that many rows fits.
int FitBatchTile(int want, int padded, int ksplit) {
  int bt = want > 2 ? 4 : want;
  while (bt > 1 && (bt > 2 ? Int4Shared<4>::Bytes(padded, ksplit)
                           : Int4Shared<2>::Bytes(padded, ksplit)) > kLdsBudget) {
    bt = bt > 2 ? 2 : 1;
  }
  return bt;
}

template <bool FUSED>
hipError_t LaunchTile(const Int4PackedArgs& a, int variant, int batch0, int bt,
                      hipStream_t stream) {
  if (a.depth > kShallowDepth && a.depth <= kDeepDepth) {
    if (bt <= 1) return LaunchVariant<1, FUSED, 8>(a, variant, batch0, bt, stream);
    if (bt <= 2) return LaunchVariant<2, FUSED, 8>(a, variant, batch0, bt, stream);
    if (!FUSED) return LaunchVariant<4, false, 8>(a, variant, batch0, bt, stream);
    return hipErrorInvalidValue;  // MaxBatchTile keeps fused deep launches at two rows
  }
  if (bt <= 1) return LaunchVariant<1, FUSED, 2>(a, variant, batch0, bt, stream);
  if (bt <= 2) return LaunchVariant<2, FUSED, 2>(a, variant, batch0, bt, stream);
  return LaunchVariant<4, FUSED, 2>(a, variant, batch0, bt, stream);
}

}  // namespace

size_t PackedInt4BlockwiseBytes(int out_depth, int depth) {
  const size_t groups = (static_cast<size_t>(out_depth) + kTileRows - 1) / kTileRows;
  const size_t chunks = (static_cast<size_t>(depth) / kBlock + kTileBlocks - 1) / kTileBlocks;
  return groups * chunks * kTileBytes;
}

hipError_t LaunchPackInt4Blockwise(const uint8_t* filter, const uint16_t* scales, int out_depth,
                                   int depth, uint8_t* packed, hipStream_t stream) {
  if (out_depth == 0 || depth == 0) return hipSuccess;
  const int chunks = (depth / kBlock + kTileBlocks - 1) / kTileBlocks;
  const int64_t total_vecs = static_cast<int64_t>(PackedInt4BlockwiseBytes(out_depth, depth) / 16);
  const unsigned grid = static_cast<unsigned>((total_vecs + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(PackInt4BlockwiseKernel, dim3(grid), dim3(kThreads), 0, stream, filter,
                     scales, out_depth, depth, chunks, total_vecs, packed);
  return hipGetLastError();
}

bool FcInt4PackedSupports(int depth, int blocksize) {
  if (blocksize != kBlock || depth <= 0 || depth % kBlock != 0) return false;
  const int chunks = (depth / kBlock + kTileBlocks - 1) / kTileBlocks;
  return Int4Shared<1>::Bytes(chunks * kTileBlocks * kBlock, kWaves) <= kLdsBudget;
}

hipError_t LaunchFcInt4Packed(const FcInt4Args& q, const uint8_t* packed, const float* input_f32,
                              int variant, hipStream_t stream) {
  if (q.batches == 0 || q.out_depth == 0) return hipSuccess;
  if (!FcInt4PackedSupports(q.depth, q.blocksize)) return hipErrorNotSupported;
  Int4PackedArgs a;
  a.packed = packed;
  a.input_f32 = input_f32;
  a.input_q = q.input;
  a.scaling_factors = q.scaling_factors;
  a.zero_points = q.zero_points;
  a.kfsum = q.kfsum;
  a.bias = q.bias;
  a.output = q.output;
  a.batches = q.batches;
  a.depth = q.depth;
  a.out_depth = q.out_depth;
  a.chunks = (q.depth / kBlock + kTileBlocks - 1) / kTileBlocks;
  const int padded = a.chunks * kTileBlocks * kBlock;
  const int tile = FitBatchTile(input_f32 ? MaxBatchTile<true>(q.depth) : MaxBatchTile<false>(q.depth),
                                padded, ChooseKsplit(q.out_depth, a.chunks));
  int batch0 = 0;
  while (batch0 < q.batches) {
    const int bt = min(tile, q.batches - batch0);
    const hipError_t err = input_f32 ? LaunchTile<true>(a, variant, batch0, bt, stream)
                                     : LaunchTile<false>(a, variant, batch0, bt, stream);
    if (err != hipSuccess) return err;
    batch0 += bt;
  }
  return hipSuccess;
}


hipError_t PrepareInt4Group(const lrtfc_int4_group_node* nodes, int count, int batches, int depth,
                            void* device_table, lrtfc_int4_group_launch* launch,
                            hipStream_t stream) {
  if (count < 1 || count > kMaxGroupNodes || !FcInt4PackedSupports(depth, kBlock)) {
    return hipErrorInvalidValue;
  }
  if (batches < 1) return hipErrorInvalidValue;
  {
    int total_tiles = 0;
    for (int i = 0; i < count; ++i) total_tiles += (nodes[i].out_depth + 15) / 16;
    bool nibbles = Int4NibbleGroupWins(batches, depth, total_tiles);
    bool decode = true;
    for (int i = 0; i < count; ++i) {
      nibbles = nibbles && nodes[i].nibble_filter != nullptr && nodes[i].workspace != nullptr;
      decode = decode && nodes[i].retiled_filter != nullptr;
    }
    if (nibbles) {
      return PrepareInt4NibbleGroup(nodes, count, batches, depth, device_table, launch, stream);
    }
    if (!decode) return hipErrorInvalidValue;
  }
  const int chunks = (depth / kBlock + kTileBlocks - 1) / kTileBlocks;
  int total_out = 0;
  for (int i = 0; i < count; ++i) total_out += nodes[i].out_depth;
  const int ksplit = ChooseKsplit(total_out, chunks);
  const int gpw = ChooseGroupsPerWave((total_out + kTileRows - 1) / kTileRows, chunks, ksplit);
  const int groups_per_wg = kWaves / ksplit * gpw;
  // Deep rows keep at most two in registers through the fused prologue; more rows are
  // quantized by a launch of their own when every node has a workspace to receive them.
  // Shallow rows do the same only in launches of many workgroups, where quantizing each row
  // once instead of once per workgroup outweighs the extra launch (config 5, B = 4: the 108
  // nodes of depth 2048 in 272 instead of 280 us per token; groups of one to three nodes lose).
  int total_blocks = 0;
  for (int i = 0; i < count; ++i) {
    const int groups = (nodes[i].out_depth + kTileRows - 1) / kTileRows;
    total_blocks += (groups + groups_per_wg - 1) / groups_per_wg;
  }
  bool split = batches > 2 && depth <= kDeepDepth &&
               (depth > kShallowDepth || total_blocks >= kSplitShallowMinBlocks);
  for (int i = 0; i < count; ++i) split = split && nodes[i].workspace != nullptr;
  // Three or four rows of a SMALL group (a stage of a decoder: one to three nodes that leave
  // most of the chip without a workgroup, their filters a few megabytes that the second reader
  // finds in the caches): the rows go as two pairs side by side in ONE launch, each workgroup
  // quantizing and multiplying two rows (2048 x 2048 at four rows: 6.3 us as one tile of four,
  // 4.7 us for two rows; 2048 x 16384: 16.5 us with the quantizer launch, 12.0 us for two fused
  // rows). Larger filters lose: the two 2048 -> 16384 projections of a decoder layer, 33.5 MB,
  // as pairs side by side take config 5's decoder-ordered token from 688 to 736 us.
  const int64_t filter_bytes = static_cast<int64_t>(total_out) * depth / 2;
  const bool side_by_side = (batches == 3 || batches == 4) && depth <= kDeepDepth &&
                            total_blocks <= kSideBySideMaxBlocks &&
                            filter_bytes <= kSideBySideMaxFilterBytes &&
                            FitBatchTile(2, chunks * kTileBlocks * kBlock, ksplit) == 2;
  if (side_by_side) split = false;
  Int4GroupTable host{};
  int next = 0;
  for (int i = 0; i < count; ++i) {
    host.first_block[i] = next;
    Int4PackedArgs& a = host.node[i];
    a.packed = nodes[i].retiled_filter;
    a.input_f32 = nodes[i].input;
    a.input_q = nullptr;
    a.scaling_factors = nullptr;
    a.zero_points = nullptr;
    if (split) {
      const ActivationWorkspace w = SplitActivationWorkspace(nodes[i].workspace, batches, depth);
      a.input_q = w.q;
      a.scaling_factors = w.sf;
      a.zero_points = w.zp;
    }
    a.kfsum = nodes[i].kfsum;
    a.bias = nodes[i].bias;
    a.output = nodes[i].output;
    a.batches = batches;
    a.depth = depth;
    a.out_depth = nodes[i].out_depth;
    a.chunks = chunks;
    const int groups = (nodes[i].out_depth + kTileRows - 1) / kTileRows;
    next += (groups + groups_per_wg - 1) / groups_per_wg;
  }
  host.first_block[count] = next;
  // Synchronous: the table is a stack object.
  hipError_t err = hipMemcpyAsync(device_table, &host, sizeof(host), hipMemcpyHostToDevice, stream);
  if (err == hipSuccess) err = hipStreamSynchronize(stream);
  if (err != hipSuccess) return err;
  launch->count = count;
  launch->grid_blocks = next;
  launch->ksplit = ksplit;
  launch->groups_per_wave = gpw;
  launch->batches = batches;
  launch->depth = depth;
  launch->split_quantize = side_by_side ? kRowPairsSideBySide : (split ? 1 : 0);
  launch->form = LRTFC_INT4_FORM_DECODE;
  return hipSuccess;
}

size_t Int4GroupTableBytes() {
  return sizeof(Int4GroupTable) > Int4NibbleGroupTableBytes() ? sizeof(Int4GroupTable)
                                                              : Int4NibbleGroupTableBytes();
}

namespace {
template <int BT, bool FUSED, int VARIANT, int GPT>
hipError_t LaunchGroupedOne(const void* table, const lrtfc_int4_group_launch& l, int batch0,
                            int bt, hipStream_t stream, int row_tiles = 1) {
  const int chunks = (l.depth / kBlock + kTileBlocks - 1) / kTileBlocks;
  const int padded = chunks * kTileBlocks * kBlock;
  const size_t lds = Int4Shared<BT>::Bytes(padded, l.ksplit);
  auto kernel = FcInt4PackedGroupedKernel<BT, FUSED, VARIANT, GPT>;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds)) return err;
  hipLaunchKernelGGL(kernel, dim3(l.grid_blocks, row_tiles), dim3(kThreads), lds, stream,
                     static_cast<const Int4GroupTable*>(table), l.count, batch0, bt, l.ksplit,
                     l.groups_per_wave);
  return hipGetLastError();
}

template <int BT, int GPT>
hipError_t LaunchGroupedVariant(const void* table, const lrtfc_int4_group_launch& l, int variant,
                                int batch0, int bt, hipStream_t stream, int row_tiles = 1) {
  switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      return LaunchGroupedOne<BT, true, LRTFC_QUANT_NEON_V8, GPT>(table, l, batch0, bt, stream,
                                                                  row_tiles);
    case LRTFC_QUANT_NEON_LEGACY:
      return LaunchGroupedOne<BT, true, LRTFC_QUANT_NEON_LEGACY, GPT>(table, l, batch0, bt, stream,
                                                                      row_tiles);
    default:
      return LaunchGroupedOne<BT, true, LRTFC_QUANT_PORTABLE, GPT>(table, l, batch0, bt, stream,
                                                                   row_tiles);
  }
}

hipError_t LaunchGroupQuantizer(const void* table, const lrtfc_int4_group_launch& l, int variant,
                                hipStream_t stream) {
  const auto* t = static_cast<const Int4GroupTable*>(table);
  const dim3 grid(static_cast<unsigned>(l.count) * l.batches);
  const bool deep = l.depth > kQuantizeDeepRow;
  auto launch = [&](auto narrow, auto wide) {
    if (deep) {
      hipLaunchKernelGGL(wide, grid, dim3(kQuantizeDeepThreads), 0, stream, t, l.batches);
    } else {
      hipLaunchKernelGGL(narrow, grid, dim3(kQuantizeThreads), 0, stream, t, l.batches);
    }
  };
  switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      launch(QuantizeGroupRowsKernel<LRTFC_QUANT_NEON_V8>,
             QuantizeGroupRowsKernel<LRTFC_QUANT_NEON_V8, kQuantizeDeepThreads>);
      break;
    case LRTFC_QUANT_NEON_LEGACY:
      launch(QuantizeGroupRowsKernel<LRTFC_QUANT_NEON_LEGACY>,
             QuantizeGroupRowsKernel<LRTFC_QUANT_NEON_LEGACY, kQuantizeDeepThreads>);
      break;
    default:
      launch(QuantizeGroupRowsKernel<LRTFC_QUANT_PORTABLE>,
             QuantizeGroupRowsKernel<LRTFC_QUANT_PORTABLE, kQuantizeDeepThreads>);
      break;
  }
  return hipGetLastError();
}
}  // namespace

hipError_t LaunchFcInt4PackedGrouped(const void* table, const lrtfc_int4_group_launch& l,
                                     int variant, hipStream_t stream) {
  if (l.count < 1 || l.grid_blocks < 1) return hipSuccess;
  if (l.form == LRTFC_INT4_FORM_GEMM_NIBBLES) {
    return LaunchFcInt4NibbleGrouped(table, l, variant, stream);
  }
  const int chunks = (l.depth / kBlock + kTileBlocks - 1) / kTileBlocks;
  const int padded = chunks * kTileBlocks * kBlock;
  if (l.split_quantize == 1) {
    if (hipError_t err = LaunchGroupQuantizer(table, l, variant, stream)) return err;
    const bool deep_rows = l.depth > kShallowDepth;
    const int tile = FitBatchTile(4, padded, l.ksplit);
    for (int batch0 = 0; batch0 < l.batches; batch0 += tile) {
      const int bt = min(tile, l.batches - batch0);
      hipError_t err;
      if (deep_rows) {
        err = bt <= 1   ? LaunchGroupedOne<1, false, LRTFC_QUANT_PORTABLE, 8>(table, l, batch0, bt, stream)
              : bt <= 2 ? LaunchGroupedOne<2, false, LRTFC_QUANT_PORTABLE, 8>(table, l, batch0, bt, stream)
                        : LaunchGroupedOne<4, false, LRTFC_QUANT_PORTABLE, 8>(table, l, batch0, bt, stream);
      } else {
        err = bt <= 1   ? LaunchGroupedOne<1, false, LRTFC_QUANT_PORTABLE, 2>(table, l, batch0, bt, stream)
              : bt <= 2 ? LaunchGroupedOne<2, false, LRTFC_QUANT_PORTABLE, 2>(table, l, batch0, bt, stream)
                        : LaunchGroupedOne<4, false, LRTFC_QUANT_PORTABLE, 2>(table, l, batch0, bt, stream);
      }
      if (err != hipSuccess) return err;
    }
    return hipSuccess;
  }
  const bool deep = l.depth > kShallowDepth && l.depth <= kDeepDepth;
  if (l.split_quantize == kRowPairsSideBySide) {
    // Three or four rows of a small group: two slices of the grid, two fused rows each.
    return deep ? LaunchGroupedVariant<2, 8>(table, l, variant, 0, 2, stream, 2)
                : LaunchGroupedVariant<2, 2>(table, l, variant, 0, 2, stream, 2);
  }
  const int tile = FitBatchTile(MaxBatchTile<true>(l.depth), padded, l.ksplit);
  for (int batch0 = 0; batch0 < l.batches; batch0 += tile) {  // more rows: one launch per tile
    const int bt = min(tile, l.batches - batch0);
    hipError_t err;
    if (deep) {
      err = bt <= 1 ? LaunchGroupedVariant<1, 8>(table, l, variant, batch0, bt, stream)
                    : LaunchGroupedVariant<2, 8>(table, l, variant, batch0, bt, stream);
    } else if (bt <= 1) {
      err = LaunchGroupedVariant<1, 2>(table, l, variant, batch0, bt, stream);
    } else if (bt <= 2) {
      err = LaunchGroupedVariant<2, 2>(table, l, variant, batch0, bt, stream);
    } else {
      err = LaunchGroupedVariant<4, 2>(table, l, variant, batch0, bt, stream);
    }
    if (err != hipSuccess) return err;
  }
  return hipSuccess;
}

}  // namespace lrtfc

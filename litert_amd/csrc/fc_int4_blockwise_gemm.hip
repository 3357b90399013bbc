// Blockwise-int4 FULLY_CONNECTED for prefill batches on gfx950: EvalBlockwise4Bit
// (tflite/kernels/fully_connected.cc:1014-1086) as a matrix-core GEMM.
//
// The decode kernel (fc_int4_packed.hip) streams the whole filter once per four batch rows,
// which is right for one to a few rows and hopeless for hundreds. Here every (row, channel)
// output keeps its float32 accumulator in a register and walks the blocks of 32 depth
// positions in order: one v_mfma_i32_16x16x32_i8 per block and 16 x 16 tile gives the exact
// int32 block sums (its K is exactly one block), and three vector operations per output add
// `float(sum) * scale[channel][block]` to the accumulator -- the reference's own order of
// float operations (:1069-1077), unfused, so the results are bit-identical to the decode
// kernel's and the oracle's. Those three operations per output and block, not the matrix
// cores, bound the kernel (the MFMA of a block takes 16 cycles, its 4 outputs per lane 48).
//
// Layouts, made once at prepare (filter) or per call (activations):
//   filter `tile16x32s`: for channel tile t (16 channels) and block b, 512 bytes: lane L's 8
//     bytes are channel 16 t + L % 16, depths 32 b + 8 (L / 16) ... + 8, sign-extended to
//     int8 -- the A operand of the MFMA as one 8-byte load per lane; after all tiles, the block
//     scales as float32, 16 per (t, b): a lane's 16-byte load is the scales of its four output
//     channels for one block, and a wavefront fetches those of 16 blocks in one instruction.
//   activations `tile16x64`: batch rows in place of channels (B operand), with the 8 bytes of
//     blocks 2 p and 2 p + 1 side by side in a lane's 16 bytes; written in that order by the
//     row quantizer itself.
// No LDS: a wavefront owns CT x RT tiles (16 to 32 channels x 16 to 64 rows, by batch size)
// and requests the operands of the next blocks while it works on the current ones (a ring of
// pairs of blocks in registers); both operands are re-read by other wavefronts from L2.
#include <mutex>

#include "kernels.h"
#include "quantize_device.h"

namespace lrtfc {
namespace {

#define LRTFC_GLOBAL __attribute__((address_space(1)))

constexpr int kThreads = 256;
constexpr int kBlock = 32;    // depth positions per quantization block
constexpr int kTile = 16;     // channels / rows per MFMA tile
// A wavefront owns CT x RT tiles of 16 channels x 16 rows (template parameters of the kernel);
// a workgroup is 2 x 2 wavefronts.

using i64 = long;
typedef long i64x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int SignedNibble(uint32_t byte, int high) {
  const int n = high ? (byte >> 4) : (byte & 0xF);
  return (n ^ 8) - 8;
}

// Model layout (rows of depth / 2 bytes, low nibble = even depth; fp16 scales [N, nb]) ->
// tile16x32s + float32 scales. One thread per 8-byte lane slot of the tile array.
__global__ __launch_bounds__(kThreads) void PackInt4BlockwiseGemmKernel(
    const uint8_t* __restrict__ filter, const uint16_t* __restrict__ scales_f16, int out_depth,
    int depth, int tiles, int nb, uint8_t* __restrict__ dst) {
  const int64_t slot = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t slots = static_cast<int64_t>(tiles) * nb * 64;
  if (slot < slots) {
    const int lane = static_cast<int>(slot & 63);
    const int64_t tb = slot >> 6;
    const int b = static_cast<int>(tb % nb);
    const int t = static_cast<int>(tb / nb);
    const int n = t * kTile + (lane & 15);
    const int k0 = b * kBlock + 8 * (lane >> 4);
    uint32_t lo = 0, hi = 0;
    if (n < out_depth) {
      const uint8_t* src = filter + static_cast<size_t>(n) * (depth / 2) + k0 / 2;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t byte = src[j];
        const uint32_t pair = (static_cast<uint32_t>(SignedNibble(byte, 0)) & 0xFF) |
                              (static_cast<uint32_t>(SignedNibble(byte, 1)) & 0xFF) << 8;
        if (j < 2) {
          lo |= pair << (16 * j);
        } else {
          hi |= pair << (16 * (j - 2));
        }
      }
    }
    reinterpret_cast<uint2*>(dst)[slot] = make_uint2(lo, hi);
  }
  // scales: one thread per (tile, block, channel)
  const int64_t scale_slots = static_cast<int64_t>(tiles) * nb * kTile;
  if (slot < scale_slots) {
    const int c = static_cast<int>(slot & 15);
    const int64_t tb = slot >> 4;
    const int b = static_cast<int>(tb % nb);
    const int t = static_cast<int>(tb / nb);
    const int n = t * kTile + c;
    float* out = reinterpret_cast<float*>(dst + slots * 8);
    out[slot] = n < out_depth ? HalfBitsToFloatFast(scales_f16[static_cast<size_t>(n) * nb + b]) : 0.0f;
  }
}

// Element k of batch row m within its row tile of the tile16x64 layout, as a byte offset
// from the tile row's base.
struct Tile16x64Placement {
  int row_in_tile;
  __device__ __forceinline__ size_t operator()(int k) const {
    const size_t lane_slot = static_cast<size_t>(k >> 6) * 64 + ((k & 31) >> 3) * 16 + row_in_tile;
    return (lane_slot * 2 + ((k >> 5) & 1)) * 8 + (k & 7);
  }
};

// BatchQuantizeFloats of float rows [batches, depth] straight into tile16x64: one workgroup
// per row of the padded batch (rows past the batch are zero). `tile_bytes`: one row tile.
template <int VARIANT>
__global__ __launch_bounds__(kQuantizeThreads) void QuantizeRowsTiledKernel(
    const float* __restrict__ input, int batches, int depth, size_t tile_bytes,
    int8_t* __restrict__ tiled, float* __restrict__ scaling_factors,
    int32_t* __restrict__ zero_points) {
  const int m = blockIdx.x;
  int8_t* tile_row = tiled + static_cast<size_t>(m / kTile) * tile_bytes;
  const Tile16x64Placement place{m % kTile};
  if (m < batches) {
    // EvalBlockwise4Bit always quantizes asymmetrically (fully_connected.cc:1044-1047).
    QuantizeRow<VARIANT>(input + static_cast<size_t>(m) * depth, depth, tile_row,
                         scaling_factors + m, zero_points + m, /*do_asymmetric=*/1, place);
  } else {
    for (int k = threadIdx.x * 8; k < depth; k += kQuantizeThreads * 8) {
      *reinterpret_cast<uint2*>(tile_row + place(k)) = make_uint2(0, 0);
    }
  }
}

struct GemmArgs {
  const i64* filter;        // tile16x32s
  const float4* scales;     // float32 [tiles][nb][16] viewed as float4
  const i64x2* activations;  // tile16x64
  const float* scaling_factors;  // [batches]
  const int32_t* zero_points;    // [batches]
  const float* kfsum;            // [out_depth]
  const float* bias;             // [out_depth] or nullptr
  float* output;                 // [batches, out_depth]
  int batches, out_depth, nb;
  int channel_tiles, row_tiles;  // of 16
  int vector_store;              // rows of the output start on 16-byte boundaries
};

// One pair of consecutive blocks of a wavefront's operands.
template <int CT, int RT>
struct Stage {
  i64 w[2][CT];  // channel tiles of the two blocks
  i64x2 x[RT];   // row tiles, both blocks
};

// Lane j of every 16 lanes to all 16 (row_newbcast:j).
template <int J>
__device__ __forceinline__ float RowBroadcast(float v) {
  // Every lane has a source lane, so no previous value is kept: the move can then merge into
  // the multiply that uses it.
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x150 + J, 0xF, 0xF, true));
}

// WROWS: wavefronts of a workgroup along the batch rows (1 or 2); the others along the channels.
// PAIRS: pairs of blocks in flight per wavefront. The count of outstanding vector loads a
//   wavefront can wait on selectively is 63, so depth comes from few, wide loads: a row tile's
//   two blocks in one 16-byte load, and the scales of 16 blocks in one load (lane = block
//   16 g + lane % 16, its float4 = channels 4 (lane / 16) ... + 4), handed to the lanes of a
//   block by a row broadcast.
template <int CT, int RT, int WROWS, int PAIRS>
__global__ __launch_bounds__(kThreads) void FcInt4BlockwiseGemmKernel(GemmArgs a) {
  constexpr int WCH = 4 / WROWS;
  const int lane = threadIdx.x & 63;
  // The wavefront index as a scalar: tile addresses then stay in scalar registers and every
  // load is "scalar base + lane offset".
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Workgroups walk the channel direction fastest: neighbours share activation tiles in L2.
  const int wg_c = blockIdx.x, wg_r = blockIdx.y;
  const int ct0 = (wg_c * WCH + wave % WCH) * CT;
  const int rt0 = (wg_r * WROWS + wave / WCH) * RT;
  if (ct0 >= a.channel_tiles || rt0 >= a.row_tiles) return;
  // Tiles past the edge re-read the last valid one; their outputs are never stored.
  int ct[CT], rt[RT];
#pragma unroll
  for (int j = 0; j < CT; ++j) ct[j] = min(ct0 + j, a.channel_tiles - 1);
#pragma unroll
  for (int j = 0; j < RT; ++j) rt[j] = min(rt0 + j, a.row_tiles - 1);
  const int nb = a.nb;
  const int pairs = (nb + 1) / 2;
  const i64* wp[CT];
  const float4* sp[CT];
  const i64x2* xp[RT];
#pragma unroll
  for (int j = 0; j < CT; ++j) {
    wp[j] = a.filter + static_cast<size_t>(ct[j]) * nb * 64 + lane;
    sp[j] = a.scales + static_cast<size_t>(ct[j]) * nb * 4 + (lane >> 4);
  }
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    xp[j] = a.activations + static_cast<size_t>(rt[j]) * pairs * 64 + lane;
  }
  auto fetch = [&](int p) {
    const int pp = min(p, pairs - 1);  // past the end: a hot line, result unused
    Stage<CT, RT> st;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int bb = min(2 * pp + h, nb - 1);
#pragma unroll
      for (int j = 0; j < CT; ++j) {
        st.w[h][j] = wp[j][static_cast<size_t>(bb) * 64];
      }
    }
#pragma unroll
    for (int j = 0; j < RT; ++j) st.x[j] = xp[j][static_cast<size_t>(pp) * 64];
    return st;
  };
  // Scale groups (16 blocks = 8 pairs) held per wavefront: the current one and as many ahead
  // as the ring of pairs reaches, so that a group is always requested before its blocks'
  // weights; a power of two, group g in slot g % kGroups.
  constexpr int kGroups = PAIRS > 8 ? 4 : 2;
  static_assert((kGroups - 1) * 8 >= PAIRS, "scale groups must lead the ring");
  float4 sg[kGroups][CT];
  auto fetch_scales = [&](int g, float4 (&dst)[CT]) {
    const int bb = min(16 * g + (lane & 15), nb - 1);
#pragma unroll
    for (int j = 0; j < CT; ++j) dst[j] = sp[j][static_cast<size_t>(bb) * 4];
  };
#pragma unroll
  for (int g = 0; g + 1 < kGroups; ++g) fetch_scales(g, sg[g]);
  Stage<CT, RT> ring[PAIRS];
#pragma unroll
  for (int s = 0; s < PAIRS; ++s) ring[s] = fetch(s);

  // out[cj][rj][i]: channel 16 ct[cj] + 4 (lane / 16) + i, batch row 16 rt[rj] + lane % 16.
  float out[CT][RT][4];
#pragma unroll
  for (int cj = 0; cj < CT; ++cj)
#pragma unroll
    for (int rj = 0; rj < RT; ++rj)
#pragma unroll
      for (int i = 0; i < 4; ++i) out[cj][rj][i] = 0.0f;

  const i32x4 zero = {0, 0, 0, 0};
  // One trip covers whole turns of the ring and of the scale slots, so that ring slots,
  // scale slots and broadcast lanes are compile-time constants.
  constexpr int kTrip = PAIRS > 8 * kGroups ? PAIRS : 8 * kGroups;
  static_assert(kTrip % PAIRS == 0 && kTrip % (8 * kGroups) == 0, "trip");
  for (int base = 0; base < pairs; base += kTrip) {
    StaticFor<kTrip>([&](auto u_const) {
      constexpr int u = decltype(u_const)::value;
      constexpr int s = u % PAIRS;
      constexpr int cur = (u / 8) % kGroups;  // slot of this pair's scale group
      if constexpr (u % 8 == 0) {
        // A new group of 16 blocks starts: the slot of the one before it takes the farthest.
        fetch_scales((base + u) / 8 + kGroups - 1, sg[(cur + kGroups - 1) % kGroups]);
      }
      const Stage<CT, RT> st = ring[s];
      ring[s] = fetch(base + u + PAIRS);
      StaticFor<2>([&](auto h_const) {
        constexpr int h = decltype(h_const)::value;
        if (2 * (base + u) + h < nb) {
#pragma unroll
          for (int cj = 0; cj < CT; ++cj) {
            constexpr int j = (2 * u + h) % 16;  // this block within its scale group
            const float sc[4] = {RowBroadcast<j>(sg[cur][cj].x), RowBroadcast<j>(sg[cur][cj].y),
                                 RowBroadcast<j>(sg[cur][cj].z), RowBroadcast<j>(sg[cur][cj].w)};
#pragma unroll
            for (int rj = 0; rj < RT; ++rj) {
              const i32x4 acc =
                  __builtin_amdgcn_mfma_i32_16x16x32_i8(st.w[h][cj], st.x[rj][h], zero, 0, 0, 0);
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                out[cj][rj][i] =
                    __fadd_rn(out[cj][rj][i], __fmul_rn(static_cast<float>(acc[i]), sc[i]));
              }
            }
          }
        }
      });
    });
  }

  // fully_connected.cc:1078-1082: zero-point term, row scale, bias.
#pragma unroll
  for (int rj = 0; rj < RT; ++rj) {
    if (rt0 + rj >= a.row_tiles) break;
    const int m = rt[rj] * kTile + (lane & 15);
    if (m >= a.batches) continue;
    const float zp = static_cast<float>(a.zero_points[m]);
    const float row_scale = a.scaling_factors[m];
#pragma unroll
    for (int cj = 0; cj < CT; ++cj) {
      if (ct0 + cj >= a.channel_tiles) break;
      const int n0 = ct[cj] * kTile + 4 * (lane >> 4);
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = min(n0 + i, a.out_depth - 1);
        float v = __fsub_rn(out[cj][rj][i], __fmul_rn(zp, a.kfsum[n]));
        v = __fmul_rn(v, row_scale);
        if (a.bias) v = __fadd_rn(v, a.bias[n]);
        o[i] = v;
      }
      float* dst = a.output + static_cast<size_t>(m) * a.out_depth + n0;
      if (n0 + 3 < a.out_depth && a.vector_store) {
        *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (n0 + i < a.out_depth) dst[i] = o[i];
        }
      }
    }
  }
}


// ---- the same product on a filter that stays 4 bits per weight --------------------------
//
// For batches between decode and prefill (5 to a few dozen rows) the filter stream bounds the
// kernel above, and sign-extending the nibbles to int8 at prepare doubles that stream. Here
// the filter stays packed (`tile16x128n`) and a wavefront expands a block's nibbles itself,
// three vector operations per block and 16 channels: for channel tile t and quad q of blocks
// (128 depth positions), 1 KiB: lane L's 16 bytes are four dwords, dword j for block 4 q + j,
// channel 16 t + L % 16, depths 8 (L / 16) ... + 8 of that block; byte k of a dword holds
// weight k of those eight in its low nibble and weight k + 4 in its high one (two's
// complement, as in the model). `(d << 4) & 0xF0F0F0F0` and `d & 0xF0F0F0F0` are then the
// eight weights as int8 values 16 w, in depth order: the A operand of v_mfma_i32_16x16x32_i8.
// Every block sum comes out multiplied by 16, hence every product and every partial sum of an
// output (scaling by a power of two commutes with each rounding; fp16 scales times integers
// stay far from the float32 range limits), and the finished sum is multiplied by 1/16 once.
// Behind the weight tiles lie the block scales as fp16: per channel tile and group of 16
// blocks, 512 bytes, lane L's 8 bytes = block 16 g + L % 16, channels 4 (L / 16) ... + 4.
// Activations: `tile16x64`, as above. One channel tile per wavefront (these batch sizes want
// the filter stream spread over as many wavefronts as possible).


__global__ __launch_bounds__(kThreads) void PackInt4BlockwiseNibblesKernel(
    const uint8_t* __restrict__ filter, const uint16_t* __restrict__ scales_f16, int out_depth,
    int depth, int tiles, int nb, int nq, int ng, uint8_t* __restrict__ dst) {
  const int64_t slot = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t slots = static_cast<int64_t>(tiles) * nq * 64;  // 16-byte lane slots
  if (slot < slots) {
    const int lane = static_cast<int>(slot & 63);
    const int64_t tq = slot >> 6;
    const int q = static_cast<int>(tq % nq);
    const int t = static_cast<int>(tq / nq);
    const int n = t * kTile + (lane & 15);
    uint32_t d[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int b = 4 * q + j;
      if (n < out_depth && b < nb) {
        // the slice's 8 weights lie in 4 consecutive bytes of the model's row: byte m holds
        // weights 2 m (low nibble) and 2 m + 1 (high nibble)
        const uint8_t* src = filter + static_cast<size_t>(n) * (depth / 2) + b * (kBlock / 2) +
                             4 * (lane >> 4);
        uint32_t w[8];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          w[2 * m] = src[m] & 0xFu;
          w[2 * m + 1] = src[m] >> 4;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) d[j] |= (w[k] | (w[k + 4] << 4)) << (8 * k);
      }
    }
    reinterpret_cast<uint4*>(dst)[slot] = make_uint4(d[0], d[1], d[2], d[3]);
  }
  // scales: one thread per (tile, group of 16 blocks, lane)
  const int64_t scale_slots = static_cast<int64_t>(tiles) * ng * 64;
  if (slot < scale_slots) {
    const int lane = static_cast<int>(slot & 63);
    const int64_t tg = slot >> 6;
    const int g = static_cast<int>(tg % ng);
    const int t = static_cast<int>(tg / ng);
    const int b = 16 * g + (lane & 15);
    uint16_t h[4] = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = t * kTile + 4 * (lane >> 4) + i;
      if (n < out_depth && b < nb) h[i] = scales_f16[static_cast<size_t>(n) * nb + b];
    }
    uint2* out = reinterpret_cast<uint2*>(dst + slots * 16);
    out[slot] = make_uint2(h[0] | (static_cast<uint32_t>(h[1]) << 16),
                           h[2] | (static_cast<uint32_t>(h[3]) << 16));
  }
}

struct NibbleGemmArgs {
  const i32x4* filter;      // tile16x128n
  const uint2* scales;      // fp16 [tiles][ng][64 lanes][4]
  const i64x2* activations;  // tile16x64
  const float* scaling_factors;
  const int32_t* zero_points;
  const float* kfsum;
  const float* bias;
  float* output;
  int batches, out_depth, nb;
  int channel_tiles, row_tiles;
  int vector_store;
};

// WQ: quads of weights in flight per wavefront; XQ: quads of activations in flight (they come
// from L2 and cost 8 registers per row tile and quad, so this ring is shorter). Measured at
// 14336 x 4096, 16 rows: 8 and 4 quads 16.9 us for quantizer + product; 16 weight quads 18.1 us
// -- a wavefront is alone on its SIMD here (896 wavefronts), and what bounds it is its own
// chain of about 15 vector operations per block, not the loads.
// The wavefronts of the 4-bit-resident kernels share nothing (no LDS image, no barrier), so each is
// a workgroup of its own: the dispatcher then spreads them one by one over the compute units.
// In workgroups of four, a launch of 2304 wavefronts leaves 64 compute units with three
// workgroups and the rest with two, and takes as long as three everywhere (36864 x 16384 at four
// rows: 84 us; as single wavefronts 71 us; 28672 x 16384: 59.6 -> 54.5 us).
constexpr int kLoneWave = 64;

template <int RT, int WQ, int XQ>
__global__ __launch_bounds__(kLoneWave) void FcInt4NibbleGemmKernel(NibbleGemmArgs a) {
  const int lane = threadIdx.x & 63;
  const int ct0 = blockIdx.x;
  const int rt0 = blockIdx.y * RT;
  if (ct0 >= a.channel_tiles || rt0 >= a.row_tiles) return;
  int rt[RT];
#pragma unroll
  for (int j = 0; j < RT; ++j) rt[j] = min(rt0 + j, a.row_tiles - 1);
  const int nb = a.nb;
  const int pairs = (nb + 1) / 2;
  const int nq = (nb + 3) / 4;
  const int ng = (nb + 15) / 16;
  const i32x4* wp = a.filter + static_cast<size_t>(ct0) * nq * 64 + lane;
  const uint2* sp = a.scales + static_cast<size_t>(ct0) * ng * 64 + lane;
  const i64x2* xp[RT];
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    xp[j] = a.activations + static_cast<size_t>(rt[j]) * pairs * 64 + lane;
  }
  // Past the end: a hot line, result unused.
  auto fetch_w = [&](int q) {
    return __builtin_nontemporal_load(wp + static_cast<size_t>(min(q, nq - 1)) * 64);
  };
  struct XStage {
    i64x2 x[RT][2];  // row tiles: blocks 0-1, blocks 2-3 of the quad
  };
  auto fetch_x = [&](int q) {
    const int qq = min(q, nq - 1);
    XStage st;
#pragma unroll
    for (int j = 0; j < RT; ++j) {
      st.x[j][0] = xp[j][static_cast<size_t>(min(2 * qq, pairs - 1)) * 64];
      st.x[j][1] = xp[j][static_cast<size_t>(min(2 * qq + 1, pairs - 1)) * 64];
    }
    return st;
  };
  // Scale groups (16 blocks = 4 quads): the current one and as many ahead as the weight ring
  // reaches, so that a group is requested before its blocks' weights.
  constexpr int kGroups = WQ / 4 + 1 <= 2 ? 2 : (WQ / 4 + 1 <= 4 ? 4 : 8);
  static_assert((kGroups - 1) * 4 >= WQ, "scale groups must lead the weight ring");
  uint2 sg[kGroups];
  auto fetch_scales = [&](int g) { return sp[static_cast<size_t>(min(g, ng - 1)) * 64]; };
#pragma unroll
  for (int g = 0; g + 1 < kGroups; ++g) sg[g] = fetch_scales(g);
  i32x4 wring[WQ];
  XStage xring[XQ];
#pragma unroll
  for (int s = 0; s < WQ; ++s) wring[s] = fetch_w(s);
#pragma unroll
  for (int s = 0; s < XQ; ++s) xring[s] = fetch_x(s);

  // out[rj][i]: channel 16 ct0 + 4 (lane / 16) + i, batch row 16 rt[rj] + lane % 16, times 16.
  float out[RT][4];
#pragma unroll
  for (int rj = 0; rj < RT; ++rj)
#pragma unroll
    for (int i = 0; i < 4; ++i) out[rj][i] = 0.0f;

  const i32x4 zero = {0, 0, 0, 0};
  constexpr int kTrip = WQ > 4 * kGroups ? WQ : 4 * kGroups;
  static_assert(kTrip % WQ == 0 && kTrip % XQ == 0 && kTrip % (4 * kGroups) == 0, "trip");
  float4 cur_scales = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  for (int base = 0; base < nq; base += kTrip) {
    StaticFor<kTrip>([&](auto u_const) {
      constexpr int u = decltype(u_const)::value;
      constexpr int cur = (u / 4) % kGroups;
      if constexpr (u % 4 == 0) {
        // A new group of 16 blocks starts: its scales become float32, and the slot of the group
        // before it takes the farthest one.
        const uint2 raw = sg[cur];
        cur_scales = make_float4(HalfBitsToFloatFast(static_cast<uint16_t>(raw.x & 0xFFFF)),
                                 HalfBitsToFloatFast(static_cast<uint16_t>(raw.x >> 16)),
                                 HalfBitsToFloatFast(static_cast<uint16_t>(raw.y & 0xFFFF)),
                                 HalfBitsToFloatFast(static_cast<uint16_t>(raw.y >> 16)));
        sg[(cur + kGroups - 1) % kGroups] = fetch_scales((base + u) / 4 + kGroups - 1);
      }
      const i32x4 w = wring[u % WQ];
      wring[u % WQ] = fetch_w(base + u + WQ);
      const XStage st = xring[u % XQ];
      xring[u % XQ] = fetch_x(base + u + XQ);
      StaticFor<4>([&](auto h_const) {
        constexpr int h = decltype(h_const)::value;
        if (4 * (base + u) + h < nb) {
          constexpr int j = (4 * u + h) % 16;  // this block within its scale group
          const float sc[4] = {RowBroadcast<j>(cur_scales.x), RowBroadcast<j>(cur_scales.y),
                               RowBroadcast<j>(cur_scales.z), RowBroadcast<j>(cur_scales.w)};
          const uint32_t d = static_cast<uint32_t>(w[h]);
          const uint32_t lo = (d << 4) & 0xF0F0F0F0u;
          const uint32_t hi = d & 0xF0F0F0F0u;
          const i64 wa = static_cast<i64>(static_cast<uint64_t>(lo) |
                                          (static_cast<uint64_t>(hi) << 32));
#pragma unroll
          for (int rj = 0; rj < RT; ++rj) {
            const i32x4 acc =
                __builtin_amdgcn_mfma_i32_16x16x32_i8(wa, st.x[rj][h >> 1][h & 1], zero, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              out[rj][i] = __fadd_rn(out[rj][i], __fmul_rn(static_cast<float>(acc[i]), sc[i]));
            }
          }
        }
      });
    });
  }

  // fully_connected.cc:1078-1082: zero-point term, row scale, bias -- after taking the factor
  // 16 back out (exact).
#pragma unroll
  for (int rj = 0; rj < RT; ++rj) {
    if (rt0 + rj >= a.row_tiles) break;
    const int m = rt[rj] * kTile + (lane & 15);
    if (m >= a.batches) continue;
    const float zp = static_cast<float>(a.zero_points[m]);
    const float row_scale = a.scaling_factors[m];
    const int n0 = ct0 * kTile + 4 * (lane >> 4);
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = min(n0 + i, a.out_depth - 1);
      float v = __fsub_rn(__fmul_rn(out[rj][i], 0.0625f), __fmul_rn(zp, a.kfsum[n]));
      v = __fmul_rn(v, row_scale);
      if (a.bias) v = __fadd_rn(v, a.bias[n]);
      o[i] = v;
    }
    float* dst = a.output + static_cast<size_t>(m) * a.out_depth + n0;
    if (n0 + 3 < a.out_depth && a.vector_store) {
      *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n0 + i < a.out_depth) dst[i] = o[i];
      }
    }
  }
}


// ---- the same filter for one to four rows: four blocks per matrix-core tile ----------------
//
// With at most four batch rows a 16 x 16 result tile per block is three quarters padding, and
// what bounds the kernel above is the vector work per tile (conversion, scale, add: per block
// whatever the row count). Here the sixteen columns of a result tile are (block j of the quad,
// row r), column 4 j + r: the quad's four MFMAs accumulate into ONE tile, MFMA j with a B operand
// that holds the rows' values of block j in columns 4 j .. 4 j + 3 and zeros elsewhere (a lane
// loads the eight activation bytes of its own column's block once per quad; a select under the
// mask "this lane's column belongs to block j" makes the four operands). One
// conversion and one scale per tile instead of four; the products of blocks 1..3 then reach the
// lanes of block 0 by row shifts and are added there in block order, which is the reference's
// order of float additions, so the results are bit-identical to every other form. Rows are read
// from the standard row quantizer's row-major output; there is no LDS image and no barrier.
struct NibbleQuadArgs {
  const i32x4* filter;   // tile16x128n
  const uint2* scales;   // fp16 [tiles][ng][64 lanes][4]
  const int8_t* rows;    // [batches][depth] int8
  const float* scaling_factors;
  const int32_t* zero_points;
  const float* kfsum;
  const float* bias;
  float* output;
  int batches, depth, out_depth, nb, channel_tiles, vector_store;
};

// The value of the lane N places up in the same row of 16 (row_shl:N); lanes past the row read 0.
template <int N>
__device__ __forceinline__ float FromLaneAbove(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x100 + N, 0xF, 0xF, true));
}

template <int WQ, int XQ>
__device__ __forceinline__ void FcInt4NibbleQuadBody(const NibbleQuadArgs& a, int ct0) {
  const int lane = threadIdx.x & 63;
  const int col = lane & 15;
  const int jl = col >> 2;                     // the block of a quad this lane's column belongs to
  const int r = min(col & 3, a.batches - 1);   // its batch row (clamped: the copy is not stored)
  const int nb = a.nb;
  const int nq = (nb + 3) / 4;
  const int ng = (nb + 15) / 16;
  // Every tensor is in global memory. The grouped kernel reads this struct from a table in
  // memory, and pointers that come from memory carry no address space: accesses through them
  // would go the flat path, whose waits also count LDS traffic (the scale broadcasts) and cannot
  // leave the rings of loads in flight. So the address space is stated here.
  const LRTFC_GLOBAL i32x4* wp =
      (const LRTFC_GLOBAL i32x4*)a.filter + static_cast<size_t>(ct0) * nq * 64 + lane;
  using U32x2 = unsigned __attribute__((ext_vector_type(2)));
  using F32x4 = float __attribute__((ext_vector_type(4)));
  const LRTFC_GLOBAL U32x2* sp =
      (const LRTFC_GLOBAL U32x2*)a.scales + static_cast<size_t>(ct0) * ng * 64 + lane;
  const LRTFC_GLOBAL int8_t* g_rows = (const LRTFC_GLOBAL int8_t*)a.rows;
  // This lane's eight activation bytes of quad q lie at rows + x_first + 128 q (clamped to the
  // row's last block: past the depth the weights are zeros).
  const uint32_t x_lane = static_cast<uint32_t>(r) * a.depth + 8 * (lane >> 4);
  const uint32_t x_first = x_lane + jl * kBlock;
  const uint32_t x_last = x_lane + (nb - 1) * kBlock;
  auto fetch_w = [&](int q) {
    return __builtin_nontemporal_load(wp + static_cast<size_t>(min(q, nq - 1)) * 64);
  };
  // Past the depth: the last block again (its weights there are zeros).
  auto fetch_x = [&](int q) {
    const uint32_t at = min(x_first + static_cast<uint32_t>(min(q, nq - 1)) * (4 * kBlock), x_last);
    return *reinterpret_cast<const LRTFC_GLOBAL i64*>(g_rows + at);
  };
  constexpr int kGroups = WQ / 4 + 1 <= 2 ? 2 : (WQ / 4 + 1 <= 4 ? 4 : 8);
  static_assert((kGroups - 1) * 4 >= WQ, "scale groups must lead the weight ring");
  uint2 sg[kGroups];
  auto fetch_scales = [&](int g) {
    const U32x2 raw = sp[static_cast<size_t>(min(g, ng - 1)) * 64];
    return make_uint2(raw.x, raw.y);
  };
#pragma unroll
  for (int g = 0; g + 1 < kGroups; ++g) sg[g] = fetch_scales(g);
  i32x4 wring[WQ];
  i64 xring[XQ];
#pragma unroll
  for (int s = 0; s < WQ; ++s) wring[s] = fetch_w(s);
#pragma unroll
  for (int s = 0; s < XQ; ++s) xring[s] = fetch_x(s);
  // Where quad t of a group of 16 blocks keeps this lane's scales: the lane of this row of 16
  // whose block is 4 t + jl (byte index for ds_bpermute).
  int from[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) from[t] = 4 * ((lane & 48) + 4 * t + jl);

  // out[i]: channel 16 ct0 + 4 (lane / 16) + i, batch row col (lanes with col < 4), times 16.
  float out[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  const i32x4 zero = {0, 0, 0, 0};
  constexpr int kTrip = WQ > 4 * kGroups ? WQ : 4 * kGroups;
  static_assert(kTrip % WQ == 0 && kTrip % XQ == 0 && kTrip % (4 * kGroups) == 0, "trip");
  float4 cur_scales = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  for (int base = 0; base < nq; base += kTrip) {
    StaticFor<kTrip>([&](auto u_const) {
      constexpr int u = decltype(u_const)::value;
      constexpr int cur = (u / 4) % kGroups;
      if constexpr (u % 4 == 0) {
        const uint2 raw = sg[cur];
        cur_scales = make_float4(HalfBitsToFloatFast(static_cast<uint16_t>(raw.x & 0xFFFF)),
                                 HalfBitsToFloatFast(static_cast<uint16_t>(raw.x >> 16)),
                                 HalfBitsToFloatFast(static_cast<uint16_t>(raw.y & 0xFFFF)),
                                 HalfBitsToFloatFast(static_cast<uint16_t>(raw.y >> 16)));
        sg[(cur + kGroups - 1) % kGroups] = fetch_scales((base + u) / 4 + kGroups - 1);
      }
      const i32x4 w = wring[u % WQ];
      wring[u % WQ] = fetch_w(base + u + WQ);
      const i64 x = xring[u % XQ];
      xring[u % XQ] = fetch_x(base + u + XQ);
      if (base + u < nq) {
        i32x4 acc;
        StaticFor<4>([&](auto h_const) {
          constexpr int h = decltype(h_const)::value;
          const uint32_t d = static_cast<uint32_t>(w[h]);
          const uint32_t lo = (d << 4) & 0xF0F0F0F0u;
          const uint32_t hi = d & 0xF0F0F0F0u;
          const i64 wa = static_cast<i64>(static_cast<uint64_t>(lo) |
                                          (static_cast<uint64_t>(hi) << 32));
          if constexpr (h == 0) {
            acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(wa, jl == h ? x : i64{0}, zero, 0, 0, 0);
          } else {
            acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(wa, jl == h ? x : i64{0}, acc, 0, 0, 0);
          }
        });
        constexpr int t = u % 4;
        const float sc[4] = {
            __int_as_float(__builtin_amdgcn_ds_bpermute(from[t], __float_as_int(cur_scales.x))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from[t], __float_as_int(cur_scales.y))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from[t], __float_as_int(cur_scales.z))),
            __int_as_float(__builtin_amdgcn_ds_bpermute(from[t], __float_as_int(cur_scales.w)))};
        // Blocks past the depth have zero weights and zero scales: they add +0.0f, which cannot
        // change a sum that has already taken its first block.
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __fmul_rn(static_cast<float>(acc[i]), sc[i]);
          float o = __fadd_rn(out[i], p);
          o = __fadd_rn(o, FromLaneAbove<4>(p));
          o = __fadd_rn(o, FromLaneAbove<8>(p));
          o = __fadd_rn(o, FromLaneAbove<12>(p));
          out[i] = o;
        }
      }
    });
  }

  // fully_connected.cc:1078-1082, after taking the factor 16 back out (exact).
  const int m = col;
  if (m >= a.batches || m >= 4) return;
  const float zp = static_cast<float>(((const LRTFC_GLOBAL int32_t*)a.zero_points)[m]);
  const float row_scale = ((const LRTFC_GLOBAL float*)a.scaling_factors)[m];
  const LRTFC_GLOBAL float* g_kfsum = (const LRTFC_GLOBAL float*)a.kfsum;
  const LRTFC_GLOBAL float* g_bias = (const LRTFC_GLOBAL float*)a.bias;
  const int n0 = ct0 * kTile + 4 * (lane >> 4);
  float o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = min(n0 + i, a.out_depth - 1);
    float v = __fsub_rn(__fmul_rn(out[i], 0.0625f), __fmul_rn(zp, g_kfsum[n]));
    v = __fmul_rn(v, row_scale);
    if (a.bias) v = __fadd_rn(v, g_bias[n]);
    o[i] = v;
  }
  LRTFC_GLOBAL float* dst = (LRTFC_GLOBAL float*)a.output + static_cast<size_t>(m) * a.out_depth + n0;
  if (n0 + 3 < a.out_depth && a.vector_store) {
    *reinterpret_cast<LRTFC_GLOBAL F32x4*>(dst) = F32x4{o[0], o[1], o[2], o[3]};
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (n0 + i < a.out_depth) dst[i] = o[i];
    }
  }
}

template <int WQ, int XQ>
__global__ __launch_bounds__(kLoneWave) void FcInt4NibbleQuadKernel(NibbleQuadArgs a) {
  const int ct0 = blockIdx.x;
  if (ct0 >= a.channel_tiles) return;
  FcInt4NibbleQuadBody<WQ, XQ>(a, ct0);
}


// Several filters of one depth in one launch (independent nodes of a graph, as in the decode
// kernel's grouped form): per node its arguments and the index of its first workgroup, in a
// table in device memory; every node's rows are quantized into its own workspace by one launch.
struct NibbleQuadGroupTable {
  int first_block[LRTFC_INT4_GROUP_MAX + 1];
  int reserved[3];
  NibbleQuadArgs node[LRTFC_INT4_GROUP_MAX];
  const float* input_f32[LRTFC_INT4_GROUP_MAX];
};

template <int WQ, int XQ>
__global__ __launch_bounds__(kLoneWave) void FcInt4NibbleQuadGroupedKernel(
    const NibbleQuadGroupTable* __restrict__ table, int count) {
  // The table counts in blocks of four channel tiles (first_block); a workgroup is one wavefront
  // with one tile. first_block is ascending: this block's node is the number of later nodes whose
  // first block is not beyond it (vector loads and ballots, 64 nodes per turn).
  const int lane = threadIdx.x & 63;
  const int block = static_cast<int>(blockIdx.x >> 2);
  int node = 0;
  for (int base = 0; base + 1 < count; base += 64) {
    const int probe = base + lane + 1;
    const bool not_beyond = probe < count && block >= table->first_block[min(probe, count)];
    node += __popcll(__ballot(not_beyond));
  }
  node = __builtin_amdgcn_readfirstlane(node);
  const NibbleQuadArgs a = table->node[node];
  const int ct0 = (block - table->first_block[node]) * 4 + static_cast<int>(blockIdx.x & 3);
  if (ct0 >= a.channel_tiles) return;
  FcInt4NibbleQuadBody<WQ, XQ>(a, ct0);
}

// Workgroup r quantizes row r % batches of node r / batches into that node's workspace
// (EvalBlockwise4Bit always quantizes asymmetrically, fully_connected.cc:1044-1047).
template <int VARIANT, int THREADS = kQuantizeThreads>
__global__ __launch_bounds__(THREADS) void QuantizeNibbleGroupRowsKernel(
    const NibbleQuadGroupTable* __restrict__ table, int batches) {
  const int node = blockIdx.x / batches;
  const int row = blockIdx.x - node * batches;
  const NibbleQuadArgs& a = table->node[node];
  QuantizeRow<VARIANT, RowMajorPlacement, THREADS>(
                       table->input_f32[node] + static_cast<size_t>(row) * a.depth, a.depth,
                       const_cast<int8_t*>(a.rows) + static_cast<size_t>(row) * a.depth,
                       const_cast<float*>(a.scaling_factors) + row,
                       const_cast<int32_t*>(a.zero_points) + row, /*do_asymmetric=*/1);
}

}  // namespace

size_t GemmInt4BlockwiseBytes(int out_depth, int depth) {
  const size_t tiles = (static_cast<size_t>(out_depth) + kTile - 1) / kTile;
  const size_t nb = static_cast<size_t>(depth) / kBlock;
  return tiles * nb * (512 + kTile * sizeof(float));
}

bool FcInt4BlockwiseGemmSupports(int depth, int blocksize) {
  return blocksize == kBlock && depth > 0 && depth % kBlock == 0;
}

hipError_t LaunchPackInt4BlockwiseGemm(const uint8_t* filter, const uint16_t* scales_f16,
                                       int out_depth, int depth, uint8_t* packed,
                                       hipStream_t stream) {
  if (out_depth == 0 || depth == 0) return hipSuccess;
  const int tiles = (out_depth + kTile - 1) / kTile;
  const int nb = depth / kBlock;
  const int64_t slots = static_cast<int64_t>(tiles) * nb * 64;
  const unsigned grid = static_cast<unsigned>((slots + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(PackInt4BlockwiseGemmKernel, dim3(grid), dim3(kThreads), 0, stream, filter,
                     scales_f16, out_depth, depth, tiles, nb, packed);
  return hipGetLastError();
}

// One row tile: 16 rows x the depth padded to whole pairs of blocks.
static size_t RowTileBytes(int depth) {
  return static_cast<size_t>(kTile) * ((static_cast<size_t>(depth) + 2 * kBlock - 1) /
                                       (2 * kBlock) * (2 * kBlock));
}

size_t TiledRowsBytes(int batches, int depth) {
  const size_t row_tiles = (static_cast<size_t>(batches) + kTile - 1) / kTile;
  return row_tiles * RowTileBytes(depth);
}

hipError_t LaunchFcInt4BlockwiseGemm(const float* input, int variant, float* scaling_factors,
                                     int32_t* zero_points, const uint8_t* gemm_filter,
                                     const float* kfsum, const float* bias, float* output,
                                     int batches, int depth, int out_depth, void* tiled_rows,
                                     hipStream_t stream) {
  if (batches == 0 || out_depth == 0) return hipSuccess;
  const int nb = depth / kBlock;
  const int row_tiles = (batches + kTile - 1) / kTile;
  const int channel_tiles = (out_depth + kTile - 1) / kTile;
  {
    const dim3 grid(row_tiles * kTile), block(kQuantizeThreads);
    int8_t* tiled = static_cast<int8_t*>(tiled_rows);
    const size_t tile_bytes = RowTileBytes(depth);
    switch (variant) {
      case LRTFC_QUANT_NEON_V8:
        hipLaunchKernelGGL(QuantizeRowsTiledKernel<LRTFC_QUANT_NEON_V8>, grid, block, 0, stream,
                           input, batches, depth, tile_bytes, tiled, scaling_factors, zero_points);
        break;
      case LRTFC_QUANT_NEON_LEGACY:
        hipLaunchKernelGGL(QuantizeRowsTiledKernel<LRTFC_QUANT_NEON_LEGACY>, grid, block, 0,
                           stream, input, batches, depth, tile_bytes, tiled, scaling_factors,
                           zero_points);
        break;
      default:
        hipLaunchKernelGGL(QuantizeRowsTiledKernel<LRTFC_QUANT_PORTABLE>, grid, block, 0, stream,
                           input, batches, depth, tile_bytes, tiled, scaling_factors, zero_points);
        break;
    }
    if (hipError_t err = hipGetLastError()) return err;
  }
  GemmArgs a;
  a.filter = reinterpret_cast<const i64*>(gemm_filter);
  a.scales = reinterpret_cast<const float4*>(gemm_filter +
                                             static_cast<size_t>(channel_tiles) * nb * 512);
  a.activations = static_cast<const i64x2*>(tiled_rows);
  a.scaling_factors = scaling_factors;
  a.zero_points = zero_points;
  a.kfsum = kfsum;
  a.bias = bias;
  a.output = output;
  a.batches = batches;
  a.out_depth = out_depth;
  a.nb = nb;
  a.channel_tiles = channel_tiles;
  a.row_tiles = row_tiles;
  a.vector_store = (out_depth % 4 == 0) && (reinterpret_cast<uintptr_t>(output) % 16 == 0);
  // Tiles per wavefront (channels x rows), the four wavefronts of a workgroup side by side
  // along the channels. Measured at 14336 x 4096: up to 128 rows one channel tile per
  // wavefront spreads the filter stream over the most wavefronts (128 rows: 42 us against 51 us
  // with two; 256 rows: level); beyond, 2 x 4 tiles re-read the least.
  const int CT = row_tiles <= 8 ? 1 : 2;
  const int RT = row_tiles <= 1 ? 1 : row_tiles <= 2 ? 2 : 4;
  const dim3 grid((channel_tiles + 4 * CT - 1) / (4 * CT), (row_tiles + RT - 1) / RT);
  if (grid.y > 65535) return hipErrorInvalidValue;
  // Pairs in flight: small tiles are bound by the filter stream and want many (16 rows: 19.5 us
  // with 16 blocks in flight, 17.1 us with 32); the 2 x 4 form is bound by its arithmetic and
  // runs best with one pair and 124 registers, four wavefronts per SIMD (2048 rows: 443 us
  // against 462 us with two pairs and two wavefronts per SIMD).
  if (CT == 2) {
    hipLaunchKernelGGL((FcInt4BlockwiseGemmKernel<2, 4, 1, 1>), grid, dim3(kThreads), 0,
                       stream, a);
  } else if (RT == 4) {
    hipLaunchKernelGGL((FcInt4BlockwiseGemmKernel<1, 4, 1, 4>), grid, dim3(kThreads), 0,
                       stream, a);
  } else if (RT == 2) {
    hipLaunchKernelGGL((FcInt4BlockwiseGemmKernel<1, 2, 1, 8>), grid, dim3(kThreads), 0,
                       stream, a);
  } else {
    hipLaunchKernelGGL((FcInt4BlockwiseGemmKernel<1, 1, 1, 16>), grid, dim3(kThreads), 0,
                       stream, a);
  }
  return hipGetLastError();
}

size_t GemmInt4BlockwiseNibbleBytes(int out_depth, int depth) {
  const size_t tiles = (static_cast<size_t>(out_depth) + kTile - 1) / kTile;
  const size_t nb = static_cast<size_t>(depth) / kBlock;
  return tiles * ((nb + 3) / 4 * 1024 + (nb + 15) / 16 * 512);
}

hipError_t LaunchPackInt4BlockwiseNibbles(const uint8_t* filter, const uint16_t* scales_f16,
                                          int out_depth, int depth, uint8_t* packed,
                                          hipStream_t stream) {
  if (out_depth == 0 || depth == 0) return hipSuccess;
  const int tiles = (out_depth + kTile - 1) / kTile;
  const int nb = depth / kBlock;
  const int nq = (nb + 3) / 4, ng = (nb + 15) / 16;
  const int64_t slots = static_cast<int64_t>(tiles) * nq * 64;
  const unsigned grid = static_cast<unsigned>((slots + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(PackInt4BlockwiseNibblesKernel, dim3(grid), dim3(kThreads), 0, stream,
                     filter, scales_f16, out_depth, depth, tiles, nb, nq, ng, packed);
  return hipGetLastError();
}

namespace {
template <int VARIANT>
void LaunchTiledQuantizer(const float* input, int batches, int depth, int row_tiles,
                          void* tiled_rows, float* scaling_factors, int32_t* zero_points,
                          hipStream_t stream) {
  const dim3 grid(row_tiles * kTile), block(kQuantizeThreads);
  hipLaunchKernelGGL(QuantizeRowsTiledKernel<VARIANT>, grid, block, 0, stream, input, batches,
                     depth, RowTileBytes(depth), static_cast<int8_t*>(tiled_rows),
                     scaling_factors, zero_points);
}
}  // namespace

hipError_t LaunchFcInt4BlockwiseNibbleGemm(const float* input, int variant,
                                           float* scaling_factors, int32_t* zero_points,
                                           const uint8_t* nibble_filter, const float* kfsum,
                                           const float* bias, float* output, int batches,
                                           int depth, int out_depth, void* tiled_rows,
                                           hipStream_t stream) {
  if (batches == 0 || out_depth == 0) return hipSuccess;
  const int nb = depth / kBlock;
  const int row_tiles = (batches + kTile - 1) / kTile;
  const int channel_tiles = (out_depth + kTile - 1) / kTile;
  if (batches <= 4) {
    // Row-major quantized rows (they fit where the tiled rows of a 16-row tile would lie).
    if (hipError_t err = LaunchBatchQuantize(input, batches, depth, static_cast<int8_t*>(tiled_rows),
                                             scaling_factors, zero_points, /*do_asymmetric=*/1,
                                             variant, stream)) {
      return err;
    }
    NibbleQuadArgs q;
    q.filter = reinterpret_cast<const i32x4*>(nibble_filter);
    q.scales = reinterpret_cast<const uint2*>(
        nibble_filter + static_cast<size_t>(channel_tiles) * ((nb + 3) / 4) * 1024);
    q.rows = static_cast<const int8_t*>(tiled_rows);
    q.scaling_factors = scaling_factors;
    q.zero_points = zero_points;
    q.kfsum = kfsum;
    q.bias = bias;
    q.output = output;
    q.batches = batches;
    q.depth = depth;
    q.out_depth = out_depth;
    q.nb = nb;
    q.channel_tiles = channel_tiles;
    q.vector_store = (out_depth % 4 == 0) && (reinterpret_cast<uintptr_t>(output) % 16 == 0);
    hipLaunchKernelGGL((FcInt4NibbleQuadKernel<8, 4>), dim3(channel_tiles), dim3(kLoneWave), 0,
                       stream, q);
    return hipGetLastError();
  }
  switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      LaunchTiledQuantizer<LRTFC_QUANT_NEON_V8>(input, batches, depth, row_tiles, tiled_rows,
                                                scaling_factors, zero_points, stream);
      break;
    case LRTFC_QUANT_NEON_LEGACY:
      LaunchTiledQuantizer<LRTFC_QUANT_NEON_LEGACY>(input, batches, depth, row_tiles, tiled_rows,
                                                    scaling_factors, zero_points, stream);
      break;
    default:
      LaunchTiledQuantizer<LRTFC_QUANT_PORTABLE>(input, batches, depth, row_tiles, tiled_rows,
                                                 scaling_factors, zero_points, stream);
      break;
  }
  if (hipError_t err = hipGetLastError()) return err;
  NibbleGemmArgs a;
  a.filter = reinterpret_cast<const i32x4*>(nibble_filter);
  a.scales = reinterpret_cast<const uint2*>(
      nibble_filter + static_cast<size_t>(channel_tiles) * ((nb + 3) / 4) * 1024);
  a.activations = static_cast<const i64x2*>(tiled_rows);
  a.scaling_factors = scaling_factors;
  a.zero_points = zero_points;
  a.kfsum = kfsum;
  a.bias = bias;
  a.output = output;
  a.batches = batches;
  a.out_depth = out_depth;
  a.nb = nb;
  a.channel_tiles = channel_tiles;
  a.row_tiles = row_tiles;
  a.vector_store = (out_depth % 4 == 0) && (reinterpret_cast<uintptr_t>(output) % 16 == 0);
  const int RT = row_tiles <= 1 ? 1 : 2;
  const dim3 grid(channel_tiles, (row_tiles + RT - 1) / RT);
  if (grid.y > 65535) return hipErrorInvalidValue;
  if (RT == 1) {
    hipLaunchKernelGGL((FcInt4NibbleGemmKernel<1, 8, 4>), grid, dim3(kLoneWave), 0, stream, a);
  } else {
    hipLaunchKernelGGL((FcInt4NibbleGemmKernel<2, 8, 2>), grid, dim3(kLoneWave), 0, stream, a);
  }
  return hipGetLastError();
}


size_t Int4NibbleGroupTableBytes() { return sizeof(NibbleQuadGroupTable); }

// With fewer than about one wavefront per SIMD the decode kernel, which splits a channel
// group's depth among wavefronts, is the faster one.
constexpr int kNibbleGroupMinTiles = 1024;

// The grouped launch takes the 4-bit-resident form where it is the faster one: three or four
// rows of filters deeper than 8192, whose rows the decode kernel parks in 64 KB of LDS per
// workgroup (28672 x 16384 at four rows: 64 us here against 82 us there).
bool Int4NibbleGroupWins(int batches, int depth, int total_channel_tiles) {
  return (batches == 3 || batches == 4) && depth > 8192 && depth % kBlock == 0 &&
         total_channel_tiles >= kNibbleGroupMinTiles;
}

hipError_t PrepareInt4NibbleGroup(const lrtfc_int4_group_node* nodes, int count, int batches,
                                  int depth, void* device_table, lrtfc_int4_group_launch* launch,
                                  hipStream_t stream) {
  if (count < 1 || count > LRTFC_INT4_GROUP_MAX || batches < 1 || batches > 4 ||
      depth % kBlock != 0) {
    return hipErrorInvalidValue;
  }
  static NibbleQuadGroupTable host;  // 20 KB: not on the stack
  static std::mutex host_mutex;
  std::lock_guard<std::mutex> lock(host_mutex);
  host = NibbleQuadGroupTable{};
  const int nb = depth / kBlock;
  int next = 0;
  for (int i = 0; i < count; ++i) {
    if (!nodes[i].nibble_filter || !nodes[i].workspace) return hipErrorInvalidValue;
    host.first_block[i] = next;
    NibbleQuadArgs& q = host.node[i];
    const int channel_tiles = (nodes[i].out_depth + kTile - 1) / kTile;
    const ActivationWorkspace w = SplitActivationWorkspace(nodes[i].workspace, batches, depth);
    q.filter = reinterpret_cast<const i32x4*>(nodes[i].nibble_filter);
    q.scales = reinterpret_cast<const uint2*>(
        nodes[i].nibble_filter + static_cast<size_t>(channel_tiles) * ((nb + 3) / 4) * 1024);
    q.rows = w.q;
    q.scaling_factors = w.sf;
    q.zero_points = w.zp;
    q.kfsum = nodes[i].kfsum;
    q.bias = nodes[i].bias;
    q.output = nodes[i].output;
    q.batches = batches;
    q.depth = depth;
    q.out_depth = nodes[i].out_depth;
    q.nb = nb;
    q.channel_tiles = channel_tiles;
    q.vector_store = (nodes[i].out_depth % 4 == 0) &&
                     (reinterpret_cast<uintptr_t>(nodes[i].output) % 16 == 0);
    host.input_f32[i] = nodes[i].input;
    next += (channel_tiles + 3) / 4;
  }
  host.first_block[count] = next;
  hipError_t err = hipMemcpyAsync(device_table, &host, sizeof(host), hipMemcpyHostToDevice, stream);
  if (err == hipSuccess) err = hipStreamSynchronize(stream);  // `host` is reused by the next call
  if (err != hipSuccess) return err;
  launch->count = count;
  launch->grid_blocks = next;
  launch->ksplit = 1;
  launch->groups_per_wave = 1;
  launch->batches = batches;
  launch->depth = depth;
  launch->split_quantize = 1;
  launch->form = LRTFC_INT4_FORM_GEMM_NIBBLES;
  return hipSuccess;
}

hipError_t LaunchFcInt4NibbleGrouped(const void* table, const lrtfc_int4_group_launch& l,
                                     int variant, hipStream_t stream) {
  if (l.count < 1 || l.grid_blocks < 1) return hipSuccess;
  const auto* t = static_cast<const NibbleQuadGroupTable*>(table);
  // This form serves groups deeper than 8192 only: the wide row quantizer.
  const dim3 qgrid(static_cast<unsigned>(l.count) * l.batches), qblock(kQuantizeDeepThreads);
  switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      hipLaunchKernelGGL((QuantizeNibbleGroupRowsKernel<LRTFC_QUANT_NEON_V8, kQuantizeDeepThreads>),
                         qgrid, qblock, 0, stream, t, l.batches);
      break;
    case LRTFC_QUANT_NEON_LEGACY:
      hipLaunchKernelGGL(
          (QuantizeNibbleGroupRowsKernel<LRTFC_QUANT_NEON_LEGACY, kQuantizeDeepThreads>), qgrid,
          qblock, 0, stream, t, l.batches);
      break;
    default:
      hipLaunchKernelGGL((QuantizeNibbleGroupRowsKernel<LRTFC_QUANT_PORTABLE, kQuantizeDeepThreads>),
                         qgrid, qblock, 0, stream, t, l.batches);
      break;
  }
  if (hipError_t err = hipGetLastError()) return err;
  // At most one wavefront per SIMD (narrow, deep filters): each keeps twice the loads in flight
  // (config 5's 18 down projections at four rows, 2304 wavefronts: 82.7 us on the small rings,
  // 90.0 us on the large ones).
  if (l.grid_blocks * 4 <= 1024) {
    hipLaunchKernelGGL((FcInt4NibbleQuadGroupedKernel<16, 8>), dim3(l.grid_blocks * 4),
                       dim3(kLoneWave), 0, stream, t, l.count);
  } else {
    hipLaunchKernelGGL((FcInt4NibbleQuadGroupedKernel<8, 4>), dim3(l.grid_blocks * 4),
                       dim3(kLoneWave), 0, stream, t, l.count);
  }
  return hipGetLastError();
}

}  // namespace lrtfc

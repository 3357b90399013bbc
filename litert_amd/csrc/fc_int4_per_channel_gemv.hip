// Decode-regime GEMV of the per-channel int4 hybrid path (EvalHybridDense4Bit,
// tflite/kernels/fully_connected.cc:1119-1187) on a filter that stays 4 bits per weight in
// HBM: half the bytes of the int8-expanded copy that the prefill GEMM runs on.
//
// Layout "tile16x128n": 1 KiB tiles of 16 channels x 128 depth. Lane L of a tile holds channel
// L % 16 and the 16 bytes = 32 nibbles of depth 32 * (L / 16) .. +32, low nibble first as in
// the model, each nibble stored as w + 8 (the model's byte XOR 0x88), so that two mask
// operations turn a dword into four unsigned bytes. Tiles of one 16-channel group are
// consecutive along the depth.
//
// A wavefront owns one group over the whole depth (or a share of it for small filters). Two
// forms: FcInt4PerChannelResidentKernel holds its whole share (at most 32 tiles) in registers,
// requested in straight-line code (rows up to 4096 deep); FcInt4PerChannelGemvKernel keeps a
// ring of 16 non-temporal 1 KiB loads in flight and refills it as it is consumed (any depth
// that fits LDS). Per
// tile: low nibbles (even depth positions) and high nibbles (odd positions) go to two
// v_mfma_i32_16x16x64_i8 against the activation rows, which the prologue parks in LDS
// de-interleaved to match. The matrix core therefore sums (w + 8) * q; the epilogue takes
// 8 * sum(q) back out -- sum(q) is known exactly from the row's input offset (-7 * sum(q),
// optimized/4bit/fully_connected_reference.cc:182-209) -- and then performs the reference's
// float steps (Hybrid4BitCore). Integer accumulation is exact, so the result is the one of
// the int8-expanded path bit for bit.
#include <type_traits>

#include "fc_epilogues.h"
#include "kernels.h"
#include "quantize_device.h"

namespace lrtfc {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWaveSize;
constexpr int kTileRows = 16;
constexpr int kSlabDepth = 128;  // depth per tile
constexpr int kQPad = 16;        // bytes of padding per staged activation row (bank spread)
constexpr int kRing = 16;        // weight tiles in flight per wavefront

__global__ __launch_bounds__(kThreads) void PackInt4PerChannelKernel(
    const uint8_t* __restrict__ src, int out_depth, int depth, int slabs, int64_t chunks,
    uint8_t* __restrict__ dst) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (c >= chunks) return;
  const int lane = static_cast<int>(c & 63);
  const int64_t tile_slab = c >> 6;
  const int slab = static_cast<int>(tile_slab % slabs);
  const int tile = static_cast<int>(tile_slab / slabs);
  const int row = tile * kTileRows + (lane & 15);
  const int k0 = slab * kSlabDepth + (lane >> 4) * 32;
  const int row_bytes = depth / 2;  // depth is even on this path
  uint8_t out[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    const int byte = k0 / 2 + t;
    const uint8_t v = (row < out_depth && byte < row_bytes)
                          ? src[static_cast<size_t>(row) * row_bytes + byte]
                          : static_cast<uint8_t>(0);
    out[t] = v ^ 0x88;
  }
  *reinterpret_cast<i32x4*>(dst + c * 16) = *reinterpret_cast<const i32x4*>(out);
}

struct NibbleArgs {
  const uint8_t* packed;        // tile16x128n
  const float* input_f32;       // fused form: float rows, quantized in the prologue
  const int8_t* input;          // [batches, depth] rows quantized by the 4-bit-path quantizer
  const float* scaling_factors; // [batches]
  const int32_t* input_offsets; // [batches]: -7 * sum(q) of the row
  const float* per_channel_scales;
  float filter_scale;
  const float* bias;
  float* output;
  int batches, depth, out_depth, activation;
  int slabs;                    // padded depth / 128
};

constexpr int kFusedRows = 4;                        // rows the fused prologue quantizes
constexpr int kFusedDepth = 4 * kThreads * 4;        // ... of at most this depth (in registers)
constexpr int kRowStateBytes = kFusedRows * (kWaves * 3 + 4) * 4;

size_t SharedBytes(int bt, int qstride) {
  return ((static_cast<size_t>(bt) * qstride + 15) & ~static_cast<size_t>(15)) +
         kWaves * 64 * sizeof(i32x4) + kRowStateBytes;
}

// Even-position and odd-position bytes of 16 consecutive int8.
__device__ __forceinline__ void Deinterleave16(const i32x4 v, i32x2* even, i32x2* odd) {
  (*even)[0] = static_cast<int>(__builtin_amdgcn_perm(v[1], v[0], 0x06040200u));
  (*even)[1] = static_cast<int>(__builtin_amdgcn_perm(v[3], v[2], 0x06040200u));
  (*odd)[0] = static_cast<int>(__builtin_amdgcn_perm(v[1], v[0], 0x07050301u));
  (*odd)[1] = static_cast<int>(__builtin_amdgcn_perm(v[3], v[2], 0x07050301u));
}

// FUSED: the rows arrive as floats and the 4-bit path's row quantizer
// (ReferenceBatchQuantizeFloats4Bit, optimized/4bit/fully_connected_reference.cc:121-180) runs
// in the prologue of every workgroup: at most kFusedRows rows of at most kFusedDepth values,
// depth a multiple of 4, 16-byte aligned.
template <bool FUSED>
__global__ __launch_bounds__(kThreads) void FcInt4PerChannelGemvKernel(NibbleArgs a, int batch0,
                                                                       int bt, int ksplit) {
  extern __shared__ __align__(16) int8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = tid / kWaveSize;
  const int col = lane & 15;     // batch column of this lane in the MFMA tiles
  const int kgroup = lane >> 4;  // which 32 of a tile's 128 depth positions this lane holds
  const int slabs = a.slabs;
  const int depth = a.depth;
  const int padded = slabs * kSlabDepth;
  const int qstride = padded + kQPad;
  int8_t* q = smem;
  i32x4* partial = reinterpret_cast<i32x4*>(
      smem + ((static_cast<size_t>(bt) * qstride + 15) & ~static_cast<size_t>(15)));
  // Row state of the fused form: per row and wavefront min, max and sum(q); then per row the
  // multiplier, the stored scale and the input offset.
  float* row_mm = reinterpret_cast<float*>(partial + kWaves * 64);  // [rows][waves][2]
  int32_t* row_sum = reinterpret_cast<int32_t*>(row_mm + kFusedRows * kWaves * 2);  // [rows][waves]
  float* row_mult = reinterpret_cast<float*>(row_sum + kFusedRows * kWaves);        // [rows]
  float* row_sf = row_mult + kFusedRows;
  int32_t* row_offset = reinterpret_cast<int32_t*>(row_sf + kFusedRows);
  const int tiles = (a.out_depth + kTileRows - 1) / kTileRows;
  const int tiles_per_wg = kWaves / ksplit;
  const int tile = blockIdx.x * tiles_per_wg + wave / ksplit;  // may run past the last group
  const int part = wave % ksplit;
  const int per_part = (slabs + ksplit - 1) / ksplit;
  const int s0 = part * per_part;
  const int s1 = min(slabs, s0 + per_part);
  const i32x4* wbase = reinterpret_cast<const i32x4*>(a.packed) +
                       (static_cast<size_t>(min(tile, tiles - 1)) * slabs) * 64 + lane;

  // Vector memory returns in issue order: the activation rows (small: up to kQRegs chunks per
  // thread in registers, else staged before anything else) go out ahead of the weights.
  constexpr int kQRegs = 4;
  const int chunks_per_row = padded / 16;
  const bool vec_ok = (depth % 16 == 0) && ((reinterpret_cast<uintptr_t>(a.input) & 15) == 0);
  const bool in_regs = vec_ok && bt * chunks_per_row <= kQRegs * kThreads;
  // Chunk c of a row (depth 16 c .. +16): its even bytes go to slab base + 8 * (c % 8), its odd
  // bytes 64 further on.
  auto park = [&](int b, int c, const i32x4 v) {
    i32x2 even, odd;
    Deinterleave16(v, &even, &odd);
    int8_t* base = q + b * qstride + (c >> 3) * kSlabDepth + (c & 7) * 8;
    *reinterpret_cast<i32x2*>(base) = even;
    *reinterpret_cast<i32x2*>(base + 64) = odd;
  };
  i32x4 qr[kQRegs];
  float4 xr[FUSED ? kFusedRows : 1][4];
  if (FUSED) {
#pragma unroll
    for (int b = 0; b < kFusedRows; ++b) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = (j * kThreads + tid) * 4;  // raw, clamped; consumed after the ring is out
        xr[b][j] = *reinterpret_cast<const float4*>(
            a.input_f32 + static_cast<size_t>(batch0 + min(b, bt - 1)) * depth + min(i, depth - 4));
      }
    }
  } else if (in_regs) {
#pragma unroll
    for (int j = 0; j < kQRegs; ++j) {
      const int c = j * kThreads + tid;
      const int b = c / chunks_per_row;
      const int i = (c - b * chunks_per_row) * 16;
      qr[j] = *reinterpret_cast<const i32x4*>(
          a.input + static_cast<size_t>(batch0 + min(b, bt - 1)) * depth + min(i, depth - 16));
    }
  } else {
    for (int b = 0; b < bt; ++b) {  // (never reached by the fused form)
      const int8_t* x = a.input + static_cast<size_t>(batch0 + b) * depth;
      for (int c = tid; c < chunks_per_row; c += kThreads) {
        i32x4 v = {0, 0, 0, 0};
        if (vec_ok) {
          if (c * 16 < depth) v = *reinterpret_cast<const i32x4*>(x + c * 16);
        } else {
          int8_t bytes[16];
          for (int t = 0; t < 16; ++t) bytes[t] = c * 16 + t < depth ? x[c * 16 + t] : 0;
          v = *reinterpret_cast<const i32x4*>(bytes);
        }
        park(b, c, v);
      }
    }
  }

  // Per-channel epilogue inputs of this lane's four channels: requested after the activation
  // rows and BEFORE the weights (behind the ring they would count as newer loads in the tile
  // loop's first round and make the first MFMA wait for the whole ring). Unconditional loads: an
  // absent array reads a valid dummy address and is ignored.
  float ep_scale[4], ep_bias[4];
  {
    const float* dummy = reinterpret_cast<const float*>(a.packed);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = min(min(tile, tiles - 1) * kTileRows + 4 * kgroup + i, a.out_depth - 1);
      ep_scale[i] = *(a.per_channel_scales ? a.per_channel_scales + n : dummy);
      ep_bias[i] = *(a.bias ? a.bias + n : dummy);
    }
  }
  i32x4 ring[kRing];
#pragma unroll
  for (int u = 0; u < kRing; ++u) {
    ring[u] = __builtin_nontemporal_load(wbase + static_cast<size_t>(min(s0 + u, slabs - 1)) * 64);
  }
  if (FUSED) {
#pragma unroll
    for (int b = 0; b < kFusedRows; ++b) {
      if (b < bt) {
        float mn = 0.0f, mx = 0.0f;  // clamped duplicates past the row are harmless here
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 t = xr[b][j];
          mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
          mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
        }
        mn = WaveMinF32(mn);
        mx = WaveMaxF32(mx);
        if (lane == 0) {
          row_mm[(b * kWaves + wave) * 2] = mn;
          row_mm[(b * kWaves + wave) * 2 + 1] = mx;
        }
      }
    }
    __syncthreads();
    if (tid < bt) {
      float mn = row_mm[tid * kWaves * 2], mx = row_mm[tid * kWaves * 2 + 1];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) {
        mn = fminf(mn, row_mm[(tid * kWaves + w) * 2]);
        mx = fmaxf(mx, row_mm[(tid * kWaves + w) * 2 + 1]);
      }
      float scale_denom = fmaxf(fabsf(mn), fabsf(mx));
      if (scale_denom == 0.0f) scale_denom = 127.0f;
      row_mult[tid] = static_cast<float>(127.0 / static_cast<double>(scale_denom));
      row_sf[tid] = static_cast<float>(static_cast<double>(scale_denom) / 127.0);
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < kFusedRows; ++b) {
      if (b < bt) {
        const float mult = row_mult[b];
        int32_t sum = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = (j * kThreads + tid) * 4;  // depth of the first of four values
          if (i < padded) {
            int32_t o[4] = {0, 0, 0, 0};
            if (i < depth) {
              const float4 t = xr[b][j];
              o[0] = static_cast<int8_t>(RoundHalfAway(__fmul_rn(t.x, mult)));
              o[1] = static_cast<int8_t>(RoundHalfAway(__fmul_rn(t.y, mult)));
              o[2] = static_cast<int8_t>(RoundHalfAway(__fmul_rn(t.z, mult)));
              o[3] = static_cast<int8_t>(RoundHalfAway(__fmul_rn(t.w, mult)));
              sum += (o[0] + o[1]) + (o[2] + o[3]);
            }
            // even depths to the first half of the slab's 128 bytes, odd depths to the second
            int8_t* base = q + b * qstride + (i >> 7) * kSlabDepth + ((i & 127) >> 1);
            *reinterpret_cast<int16_t*>(base) =
                static_cast<int16_t>((o[0] & 0xFF) | ((o[2] & 0xFF) << 8));
            *reinterpret_cast<int16_t*>(base + 64) =
                static_cast<int16_t>((o[1] & 0xFF) | ((o[3] & 0xFF) << 8));
          }
        }
        sum = WaveSumI32(sum);
        if (lane == 0) row_sum[b * kWaves + wave] = sum;
      }
    }
    __syncthreads();
    if (tid < bt) {
      int32_t total = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) total += row_sum[tid * kWaves + w];
      row_offset[tid] = total * -7;
    }
  } else if (in_regs) {
#pragma unroll
    for (int j = 0; j < kQRegs; ++j) {
      const int c = j * kThreads + tid;
      const int b = c / chunks_per_row;
      const int cc = c - b * chunks_per_row;
      if (b < bt) park(b, cc, cc * 16 < depth ? qr[j] : i32x4{0, 0, 0, 0});
    }
  }
  __syncthreads();

  // Matrix-core loop. Columns past the batch tile read row 0; their results are never stored.
  const int8_t* qbase = q + (col < bt ? col : 0) * qstride + kgroup * 16;
  constexpr int kAccs = 4;
  i32x4 acc4[kAccs];
#pragma unroll
  for (int i = 0; i < kAccs; ++i) acc4[i] = i32x4{0, 0, 0, 0};
  auto consume = [&](const i32x4 w, int slab, int slot) {
    const i32x4 qe = *reinterpret_cast<const i32x4*>(qbase + slab * kSlabDepth);
    const i32x4 qo = *reinterpret_cast<const i32x4*>(qbase + slab * kSlabDepth + 64);
    i32x4 lo, hi;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      lo[d] = w[d] & 0x0F0F0F0F;
      hi[d] = static_cast<int>((static_cast<uint32_t>(w[d]) >> 4) & 0x0F0F0F0Fu);
    }
    acc4[(2 * slot) % kAccs] =
        __builtin_amdgcn_mfma_i32_16x16x64_i8(lo, qe, acc4[(2 * slot) % kAccs], 0, 0, 0);
    acc4[(2 * slot + 1) % kAccs] =
        __builtin_amdgcn_mfma_i32_16x16x64_i8(hi, qo, acc4[(2 * slot + 1) % kAccs], 0, 0, 0);
  };
  int base = s0;
  for (; base + kRing < s1; base += kRing) {  // full rounds: consume a slot, refill it
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
      consume(ring[u], base + u, u);
      ring[u] = __builtin_nontemporal_load(
          wbase + static_cast<size_t>(min(base + kRing + u, slabs - 1)) * 64);
    }
  }
#pragma unroll
  for (int u = 0; u < kRing; ++u) {  // last turn of the ring
    if (base + u < s1) consume(ring[u], base + u, u);
  }
  i32x4 acc = (acc4[0] + acc4[1]) + (acc4[2] + acc4[3]);

  if (ksplit > 1) {  // depth shares of one channel group meet in LDS
    partial[wave * 64 + lane] = acc;
    __syncthreads();
    if (part != 0) return;
    for (int w = 1; w < ksplit; ++w) acc += partial[(wave + w) * 64 + lane];
  }

  // Epilogue. Accumulator register i holds channel 4 * (L / 16) + i, column L % 16.
  if (col >= bt || tile >= tiles) return;
  const int b = batch0 + col;
  const float batch_scale = FUSED ? row_sf[col] : a.scaling_factors[b];
  const int32_t input_offset = FUSED ? row_offset[col] : a.input_offsets[b];
  const int32_t sum_q = -(input_offset / 7);  // exact: the offset is -7 * sum(q)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = tile * kTileRows + 4 * kgroup + i;
    if (n >= a.out_depth) continue;
    const int32_t dot = acc[i] - 8 * sum_q;  // sum(w * q) from sum((w + 8) * q)
    a.output[static_cast<size_t>(b) * a.out_depth + n] = Hybrid4BitCore(
        dot, batch_scale, a.per_channel_scales ? ep_scale[i] : a.filter_scale, input_offset,
        a.bias ? ep_bias[i] : 0.0f, a.bias != nullptr, a.activation);
  }
}


// ---- the form for filters a launch can hold in its registers --------------------------------
//
// The same kernel built the way the int8 decode GEMV is (FcInt8ResidentGemvKernel): a launch of
// this size is a chain of latencies in front of a stream, and a ring that is refilled as it is
// consumed ties the stream to the consumer. Here every tile of a wavefront's share of the depth
// (at most TILES tiles of 1 KiB) has a variable of its own in straight-line code, so a request
// never waits for a product: kResidentAhead tiles go out before anything waits for anything,
// the kernel's one barrier (rows staged) follows, and from there requests and products
// alternate, the products kResidentLag tiles behind. The per-row work of the fused form belongs
// to single wavefronts (wavefront r reads, reduces, quantizes and stages row r on its own, at
// raised priority, while the others hold their first request back), the leading arguments
// arrive preloaded in registers and everything else is read from the argument segment where
// the code asks for it.

constexpr int kResidentLag = 12;
constexpr int kResidentAhead = 24;
constexpr int kResidentRowDepth = 8 * kWaveSize * 8;  // a wavefront's row: 8 x 8 floats per lane

// Where `NibbleArgs` lies in the argument segment: behind three pointers and seven ints.
constexpr size_t kResidentArgsOffset = 56;
static_assert(3 * sizeof(void*) + 7 * sizeof(int) <= kResidentArgsOffset &&
                  kResidentArgsOffset % alignof(NibbleArgs) == 0 &&
                  kResidentArgsOffset - (3 * sizeof(void*) + 7 * sizeof(int)) < alignof(NibbleArgs),
              "argument layout of FcInt4PerChannelResidentKernel");

size_t ResidentSharedBytes(int bt, int qstride) {
  return ((static_cast<size_t>(bt) * qstride + 15) & ~static_cast<size_t>(15)) + 128 +
         kWaves * 64 * sizeof(i32x4) + kFusedRows * 8;
}

// Four values of a row times its multiplier, rounded half away from zero, as four bytes (the
// saturation of v_cvt_pk_u8_f32 on value + 128 never binds: |v * mult| < 127.5).
__device__ __forceinline__ uint32_t QuantizeSymmetricPack4(float a, float b, float c, float d,
                                                           float mult) {
  uint32_t w = 0;
  w = __builtin_amdgcn_cvt_pk_u8_f32(__fadd_rn(RoundHalfAway(__fmul_rn(a, mult)), 128.0f), 0, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(__fadd_rn(RoundHalfAway(__fmul_rn(b, mult)), 128.0f), 1, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(__fadd_rn(RoundHalfAway(__fmul_rn(c, mult)), 128.0f), 2, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(__fadd_rn(RoundHalfAway(__fmul_rn(d, mult)), 128.0f), 3, w);
  return w ^ 0x80808080u;
}

template <bool FUSED, int TILES, int QREGS>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void FcInt4PerChannelResidentKernel(const uint8_t* early_packed, const float* early_input_f32,
                                    const int8_t* early_input, int early_depth, int early_slabs,
                                    int early_out_depth, int batch0, int bt, int ksplit_log2,
                                    int per_part, NibbleArgs unread) {
  // `unread` is never named again: its fields are fetched from the argument segment through
  // late_args() at the points where they are needed (naming it would let the compiler move all
  // of those loads to the kernel's entry, in front of the first weight request).
  extern __shared__ __align__(16) int8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWaveSize);
  const int ksplit = 1 << ksplit_log2;
  const int col = lane & 15;
  const int kgroup = lane >> 4;
  const int slabs = early_slabs;
  const int depth = early_depth;
  // A staged row is zero up to the end of the last share, so that a share that runs past the
  // depth multiplies its (clamped, re-read) tiles by zeros instead of branching.
  const int staged = ksplit * per_part * kSlabDepth;
  const int qstride = staged + kQPad;
  int8_t* q = smem;
  int8_t* zeros = smem + ((static_cast<size_t>(bt) * qstride + 15) & ~static_cast<size_t>(15));
  i32x4* partial = reinterpret_cast<i32x4*>(zeros + 128);
  float* row_sf = reinterpret_cast<float*>(partial + kWaves * 64);
  int32_t* row_offset = reinterpret_cast<int32_t*>(row_sf + kFusedRows);
  const int tiles = (early_out_depth + kTileRows - 1) / kTileRows;
  const int tile = ((blockIdx.x * kWaves) >> ksplit_log2) + (wave >> ksplit_log2);
  const int part = wave & (ksplit - 1);
  const int s0 = part * per_part;
  const uint8_t* group_base =
      early_packed + static_cast<size_t>(min(tile, tiles - 1)) * slabs * 1024;  // uniform

  using LateArgs = const __attribute__((address_space(4))) NibbleArgs;
  auto late_args = [&]() -> LateArgs* {
    auto* segment = (const __attribute__((address_space(4))) char*)
        __builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(segment));
    return (LateArgs*)(segment + kResidentArgsOffset);
  };
  i32x4 ring[TILES];
  auto request = [&](int u) {
    // Past the share or the depth: the share's last tile again (a hit in the nearest cache).
    const uint8_t* t =
        group_base + static_cast<size_t>(min(s0 + min(u, per_part - 1), slabs - 1)) * 1024;
    ring[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(t + lane * 16));
    __builtin_amdgcn_sched_barrier(0);
  };

  // Per-channel epilogue inputs of this lane's four channels and, for rows that arrive
  // quantized, the row's own parameters: requested behind the first tiles (a load issued at the
  // end of the kernel queues behind the whole chip's weight stream). Unconditional loads: an
  // absent array reads a valid dummy address and is ignored.
  float ep_scale[4], ep_bias[4];
  float ep_row_scale = 0.0f;
  int32_t ep_row_offset = 0;
  auto request_parameters = [&]() {
    const LateArgs* late = late_args();
    const float* dummy = reinterpret_cast<const float*>(early_packed);
    const float* scales = late->per_channel_scales;
    const float* bias = late->bias;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = min(min(tile, tiles - 1) * kTileRows + 4 * kgroup + i, early_out_depth - 1);
      ep_scale[i] = *(scales ? scales + n : dummy);
      ep_bias[i] = *(bias ? bias + n : dummy);
    }
    if (!FUSED) {
      const int row = batch0 + min(col, bt - 1);
      ep_row_scale = late->scaling_factors[row];
      ep_row_offset = late->input_offsets[row];
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  float* ep_out;
  int ep_activation, ep_flags;
  float ep_filter_scale;
  auto fetch_epilogue_scalars = [&]() {
    const LateArgs* late = late_args();
    ep_out = late->output;
    ep_activation = late->activation;
    ep_flags = (late->per_channel_scales ? 1 : 0) | (late->bias ? 2 : 0);
    ep_filter_scale = late->filter_scale;
  };

  const int8_t* qbase = q + (col < bt ? col : 0) * qstride + kgroup * 16 + s0 * kSlabDepth;
  const int8_t* zero_operand = zeros + kgroup * 16;
  constexpr int kAccs = 4;
  i32x4 acc4[kAccs];
#pragma unroll
  for (int i = 0; i < kAccs; ++i) acc4[i] = i32x4{0, 0, 0, 0};
  // Products of tiles g .. g + 3: their eight activation operands behind one LDS wait.
  auto multiply4 = [&](int g) {
    i32x4 qe[4], qo[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      // Past the share (TILES larger than the share): 16 bytes of zeros.
      const int8_t* at = g + u < per_part ? qbase + (g + u) * kSlabDepth : zero_operand;
      qe[u] = *reinterpret_cast<const i32x4*>(at);
      qo[u] = *reinterpret_cast<const i32x4*>(at + 64);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      i32x4 lo, hi;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        lo[d] = ring[g + u][d] & 0x0F0F0F0F;
        hi[d] = static_cast<int>((static_cast<uint32_t>(ring[g + u][d]) >> 4) & 0x0F0F0F0Fu);
      }
      acc4[u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(lo, qe[u], acc4[u], 0, 0, 0);
      acc4[u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(hi, qo[u], acc4[u], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto stream = [&](auto first_c, auto ahead_c) {
    constexpr int kFirst = decltype(first_c)::value;
    constexpr int kAhead = decltype(ahead_c)::value < TILES ? decltype(ahead_c)::value : TILES;
    constexpr int kLag = kResidentLag < kAhead ? kResidentLag : kAhead;
    static_assert(kFirst <= kAhead && kAhead % 4 == 0 && kLag % 4 == 0 && TILES % 4 == 0, "");
#pragma unroll
    for (int u = kFirst; u < kAhead; ++u) request(u);
    request_parameters();
    if (tid < 32) reinterpret_cast<int32_t*>(zeros)[tid] = 0;
    fetch_epilogue_scalars();
    __syncthreads();
#pragma unroll
    for (int g = 0; g < kAhead - kLag; g += 4) multiply4(g);
#pragma unroll
    for (int g = kAhead; g < TILES; g += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) request(g + u);
      multiply4(g - kLag);
    }
#pragma unroll
    for (int g = TILES - kLag; g < TILES; g += 4) multiply4(g);
  };
  using std::integral_constant;

  if (FUSED) {
    if (wave < bt) {
      __builtin_amdgcn_s_setprio(3);
      // This wavefront's row (ReferenceBatchQuantizeFloats4Bit,
      // optimized/4bit/fully_connected_reference.cc:121-180): 8 pieces of 8 floats per lane.
      constexpr int kPieces = 8;
      const float* x = early_input_f32 + static_cast<size_t>(batch0 + wave) * depth;
      float4 xr[kPieces][2];
#pragma unroll
      for (int j = 0; j < kPieces; ++j) {
        const int i = (j * kWaveSize + lane) * 8;
        xr[j][0] = *reinterpret_cast<const float4*>(x + min(i, depth - 4));
        xr[j][1] = *reinterpret_cast<const float4*>(x + min(i + 4, depth - 4));
      }
      __builtin_amdgcn_sched_barrier(0);
      // Every wavefront of a workgroup with four rows has one: some weights go out ahead of the
      // row's arithmetic, or nothing would be in flight meanwhile.
      constexpr int kEarly = TILES < 8 ? TILES : 8;
#pragma unroll
      for (int u = 0; u < kEarly; ++u) request(u);
      float mn = 0.0f, mx = 0.0f;  // clamped duplicates past the row are harmless here
#pragma unroll
      for (int j = 0; j < kPieces; ++j) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const float4 t = xr[j][h];
          mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
          mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
        }
      }
      mn = WaveMinF32(mn);
      mx = WaveMaxF32(mx);
      float scale_denom = fmaxf(fabsf(mn), fabsf(mx));
      if (scale_denom == 0.0f) scale_denom = 127.0f;
      const float mult = static_cast<float>(127.0 / static_cast<double>(scale_denom));
      const float sf = static_cast<float>(static_cast<double>(scale_denom) / 127.0);
      int8_t* qrow = q + wave * qstride;
      int32_t sum = 0;
#pragma unroll
      for (int j = 0; j < kPieces; ++j) {
        const int i = (j * kWaveSize + lane) * 8;  // depth of the first of eight values
        const float4 a = xr[j][0], b = xr[j][1];
        // Even depths to the first half of the slab's 128 bytes, odd depths to the second.
        uint32_t even = QuantizeSymmetricPack4(a.x, a.z, b.x, b.z, mult);
        uint32_t odd = QuantizeSymmetricPack4(a.y, a.w, b.y, b.w, mult);
        if (i + 4 >= depth) {  // the second four (or all eight) lie past the row
          even &= i < depth ? 0x0000FFFFu : 0u;
          odd &= i < depth ? 0x0000FFFFu : 0u;
        }
        sum = __builtin_amdgcn_sdot4(static_cast<int>(even), 0x01010101, sum, false);
        sum = __builtin_amdgcn_sdot4(static_cast<int>(odd), 0x01010101, sum, false);
        if (i < staged) {
          int8_t* base = qrow + (i >> 7) * kSlabDepth + ((i & 127) >> 1);
          *reinterpret_cast<uint32_t*>(base) = even;
          *reinterpret_cast<uint32_t*>(base + 64) = odd;
        }
      }
      sum = WaveSumI32(sum);
      if (lane == 0) {
        row_sf[wave] = sf;
        row_offset[wave] = sum * -7;
      }
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      stream(integral_constant<int, kEarly>{},
             integral_constant<int, (kEarly > kResidentLag ? kEarly : kResidentLag)>{});
    } else {
      __builtin_amdgcn_s_sleep(8);  // 512 cycles: the rows' requests go first
      stream(integral_constant<int, 0>{}, integral_constant<int, kResidentAhead>{});
    }
  } else {
    // Rows that arrive quantized: QREGS 16-byte chunks per thread (4: four rows of depth 4096;
    // 16: sixteen), requested ahead of the weights and parked de-interleaved when they are there.
    constexpr int kQRegs = QREGS;
    constexpr int kFirst = TILES < 8 ? TILES : 8;
    const int chunks_per_row = staged / 16;
    i32x4 qr[kQRegs];
#pragma unroll
    for (int j = 0; j < kQRegs; ++j) {
      const int c = j * kThreads + tid;
      const int b = c / chunks_per_row;
      const int i = (c - b * chunks_per_row) * 16;
      qr[j] = *reinterpret_cast<const i32x4*>(
          early_input + static_cast<size_t>(batch0 + min(b, bt - 1)) * depth + min(i, depth - 16));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kFirst; ++u) request(u);
#pragma unroll
    for (int j = 0; j < kQRegs; ++j) {
      const int c = j * kThreads + tid;
      const int b = c / chunks_per_row;
      const int cc = c - b * chunks_per_row;
      if (b < bt) {
        i32x2 even, odd;
        Deinterleave16(cc * 16 < depth ? qr[j] : i32x4{0, 0, 0, 0}, &even, &odd);
        int8_t* base = q + b * qstride + (cc >> 3) * kSlabDepth + (cc & 7) * 8;
        *reinterpret_cast<i32x2*>(base) = even;
        *reinterpret_cast<i32x2*>(base + 64) = odd;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    stream(integral_constant<int, kFirst>{}, integral_constant<int, kResidentAhead>{});
  }
  i32x4 acc = (acc4[0] + acc4[1]) + (acc4[2] + acc4[3]);

  if (ksplit > 1) {  // depth shares of one channel group meet in LDS (int32: exact)
    partial[wave * 64 + lane] = acc;
    __syncthreads();
    if (part != 0) return;
    for (int w = 1; w < ksplit; ++w) acc += partial[(wave + w) * 64 + lane];
  }

  // Epilogue. Accumulator register i holds channel 4 * (L / 16) + i, column L % 16.
  if (col >= bt || tile >= tiles) return;
  const int b = batch0 + col;
  const float batch_scale = FUSED ? row_sf[col] : ep_row_scale;
  const int32_t input_offset = FUSED ? row_offset[col] : ep_row_offset;
  const int32_t sum_q = -(input_offset / 7);  // exact: the offset is -7 * sum(q)
  float value[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int32_t dot = acc[i] - 8 * sum_q;  // sum(w * q) from sum((w + 8) * q)
    value[i] = Hybrid4BitCore(dot, batch_scale, (ep_flags & 1) ? ep_scale[i] : ep_filter_scale,
                              input_offset, (ep_flags & 2) ? ep_bias[i] : 0.0f,
                              (ep_flags & 2) != 0, ep_activation);
  }
  const int n0 = tile * kTileRows + 4 * kgroup;
  float* out = ep_out + static_cast<size_t>(b) * early_out_depth + n0;
  if (n0 + 4 <= early_out_depth && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    *reinterpret_cast<float4*>(out) = float4{value[0], value[1], value[2], value[3]};
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (n0 + i < early_out_depth) out[i] = value[i];
    }
  }
}

template <bool FUSED, int TILES, int QREGS>
hipError_t LaunchResident(const NibbleArgs& a, int batch0, int bt, int ksplit,
                          hipStream_t stream) {
  const int per_part = (a.slabs + ksplit - 1) / ksplit;
  const int qstride = ksplit * per_part * kSlabDepth + kQPad;
  const size_t lds = ResidentSharedBytes(bt, qstride);
  auto kernel = FcInt4PerChannelResidentKernel<FUSED, TILES, QREGS>;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds)) return err;
  const int tiles = (a.out_depth + kTileRows - 1) / kTileRows;
  const int tiles_per_wg = kWaves / ksplit;
  const int grid = (tiles + tiles_per_wg - 1) / tiles_per_wg;
  int ksplit_log2 = 0;
  while ((1 << ksplit_log2) < ksplit) ++ksplit_log2;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, a.packed, a.input_f32,
                     a.input, a.depth, a.slabs, a.out_depth, batch0, bt, ksplit_log2, per_part, a);
  return hipGetLastError();
}

// Whether the register-resident form takes a pass of bt rows; *launched tells. A wavefront's
// share of the depth has to fit its tile registers, a fused row the 64 floats per lane set aside
// for it, rows that arrive quantized the four chunks per thread.
template <bool FUSED>
hipError_t TryLaunchResident(const NibbleArgs& a, int batch0, int bt, hipStream_t stream,
                             bool* launched) {
  *launched = false;
  const int tiles = (a.out_depth + kTileRows - 1) / kTileRows;
  int ksplit = 1;
  while (ksplit < kWaves && (a.slabs + ksplit - 1) / ksplit > 32) ksplit *= 2;
  // Filters of few channel groups: smaller shares while half the chip's SIMDs have no wavefront
  // (14336 x 4096, one row: 7.3 us as 896 wavefronts with 32 tiles each, 7.4 us as 1792 with 16,
  // 10.8 us as 3584 with 8; two rows 7.3 / 8.2 us).
  while (ksplit < kWaves && tiles * ksplit < 512 && a.slabs / (ksplit * 2) >= 4) ksplit *= 2;
  const int per_part = (a.slabs + ksplit - 1) / ksplit;
  if (per_part > 32) return hipSuccess;
  const int staged = ksplit * per_part * kSlabDepth;
  if (FUSED) {
    if (bt > kFusedRows || a.depth > kResidentRowDepth || staged > kResidentRowDepth ||
        a.depth % 4 != 0 || a.depth < 4 || (reinterpret_cast<uintptr_t>(a.input_f32) & 15) != 0) {
      return hipSuccess;
    }
  } else {
    if (a.depth % 16 != 0 || a.depth < 16 || (reinterpret_cast<uintptr_t>(a.input) & 15) != 0 ||
        static_cast<int64_t>(bt) * (staged / 16) > 16 * kThreads) {
      return hipSuccess;
    }
  }
  if (ResidentSharedBytes(bt, staged + kQPad) > 150 * 1024) return hipSuccess;
  *launched = true;
  if (!FUSED && static_cast<int64_t>(bt) * (staged / 16) > 4 * kThreads) {
    if (per_part <= 8) return LaunchResident<false, 8, 16>(a, batch0, bt, ksplit, stream);
    if (per_part <= 16) return LaunchResident<false, 16, 16>(a, batch0, bt, ksplit, stream);
    return LaunchResident<false, 32, 16>(a, batch0, bt, ksplit, stream);
  }
  if (per_part <= 8) return LaunchResident<FUSED, 8, 4>(a, batch0, bt, ksplit, stream);
  if (per_part <= 16) return LaunchResident<FUSED, 16, 4>(a, batch0, bt, ksplit, stream);
  return LaunchResident<FUSED, 32, 4>(a, batch0, bt, ksplit, stream);
}

}  // namespace

size_t PackedInt4PerChannelBytes(int out_depth, int depth) {
  const size_t tiles = (static_cast<size_t>(out_depth) + kTileRows - 1) / kTileRows;
  const size_t slabs = (static_cast<size_t>(depth) + kSlabDepth - 1) / kSlabDepth;
  return tiles * slabs * 1024;
}

hipError_t LaunchPackInt4PerChannel(const uint8_t* filter, int out_depth, int depth,
                                    uint8_t* packed, hipStream_t stream) {
  if (out_depth == 0 || depth == 0) return hipSuccess;
  if (depth % 2 != 0) return hipErrorInvalidValue;
  const int slabs = (depth + kSlabDepth - 1) / kSlabDepth;
  const int64_t chunks = static_cast<int64_t>(PackedInt4PerChannelBytes(out_depth, depth) / 16);
  const unsigned grid = static_cast<unsigned>((chunks + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(PackInt4PerChannelKernel, dim3(grid), dim3(kThreads), 0, stream, filter,
                     out_depth, depth, slabs, chunks, packed);
  return hipGetLastError();
}

bool FcInt4PerChannelGemvSupports(int depth) {
  if (depth <= 0 || depth % 2 != 0) return false;
  const size_t qstride =
      (static_cast<size_t>(depth) + kSlabDepth - 1) / kSlabDepth * kSlabDepth + kQPad;
  return SharedBytes(1, static_cast<int>(qstride)) <= 150 * 1024;
}

hipError_t LaunchFcInt4PerChannelGemv(const uint8_t* packed, const float* input_f32,
                                      const int8_t* quantized_input,
                                      const float* scaling_factors, const int32_t* input_offsets,
                                      const float* per_channel_scales, float filter_scale,
                                      const float* bias, float* output, int batches, int depth,
                                      int out_depth, int activation, hipStream_t stream) {
  if (batches == 0 || out_depth == 0) return hipSuccess;
  if (!FcInt4PerChannelGemvSupports(depth)) return hipErrorNotSupported;
  NibbleArgs a;
  a.packed = packed;
  a.input_f32 = input_f32;
  a.input = quantized_input;
  a.scaling_factors = scaling_factors;
  a.input_offsets = input_offsets;
  a.per_channel_scales = per_channel_scales;
  a.filter_scale = filter_scale;
  a.bias = bias;
  a.output = output;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.activation = activation;
  a.slabs = (depth + kSlabDepth - 1) / kSlabDepth;
  const int qstride = a.slabs * kSlabDepth + kQPad;
  const int tiles = (out_depth + kTileRows - 1) / kTileRows;
  // One wavefront per channel group when that already gives the chip ~2 wavefronts per
  // SIMD-pair; otherwise split the depth so that short filters still spread out.
  int ksplit = 1;
  while (ksplit < kWaves && tiles * ksplit < 512 && a.slabs / (ksplit * 2) >= 4) ksplit *= 2;
  const int tiles_per_wg = kWaves / ksplit;
  const int grid = (tiles + tiles_per_wg - 1) / tiles_per_wg;
  const bool fused = input_f32 != nullptr;
  int batch0 = 0;
  while (batch0 < batches) {
    int bt = min(fused ? kFusedRows : 16, batches - batch0);
    while (bt > 1 && SharedBytes(bt, qstride) > 150 * 1024) --bt;
    bool launched = false;
    if (hipError_t err = fused ? TryLaunchResident<true>(a, batch0, bt, stream, &launched)
                               : TryLaunchResident<false>(a, batch0, bt, stream, &launched)) {
      return err;
    }
    if (launched) {
      batch0 += bt;
      continue;
    }
    const size_t lds = SharedBytes(bt, qstride);
    auto kernel = fused ? FcInt4PerChannelGemvKernel<true> : FcInt4PerChannelGemvKernel<false>;
    if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds)) return err;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, a, batch0, bt, ksplit);
    if (hipError_t err = hipGetLastError()) return err;
    batch0 += bt;
  }
  return hipSuccess;
}

bool FcInt4PerChannelGemvFuses(const float* input_f32, int batches, int depth) {
  return batches <= kFusedRows && depth <= kFusedDepth && depth % 4 == 0 &&
         (reinterpret_cast<uintptr_t>(input_f32) & 15) == 0;
}

}  // namespace lrtfc

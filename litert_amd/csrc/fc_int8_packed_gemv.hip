// Decode-regime FULLY_CONNECTED with int8 weights, batches 1..16, on pre-packed
// weights and the gfx950 matrix cores.
//
// Why matrix cores for a GEMV: with sdot4 every extra batch row costs a full set of
// VALU dot products and a cross-lane reduction, and the kernel turns ALU-bound at
// batch 8. v_mfma_i32_16x16x64_i8 multiplies a 16-row x 64-deep weight tile by up to 16
// activation columns in 16 cycles, far above the HBM rate, for any batch 1..16, and
// its accumulator layout needs no cross-lane reduction at all.
//
// HBM layout ("tile16x64", built once per constant filter by PackInt8FilterKernel):
// the filter is cut into tiles of 16 output channels x 64 depth = 1 KiB; inside a tile
// lane L's 16 bytes are channel (L % 16), depth 16 * (L / 16) .. +16, which is the MFMA
// A-operand register layout. Tiles of one 16-channel group are contiguous along the
// depth, so a wavefront's load instruction reads 1 KiB of consecutive bytes and a
// wavefront's whole share is one contiguous run.
//
// Two kernels run on this layout. FcInt8ResidentGemvKernel (further down, with its own
// account) takes the launches whose per-wavefront share of the depth fits the registers:
// depth up to 8192 at decode widths, i.e. the benchmark configurations. FcInt8PackedGemvKernel is the
// general form for everything else: a wavefront streams a contiguous run of one 16-channel
// group's tiles through a ring of 16 outstanding 1 KiB loads, refilling a slot as soon as the
// matrix core has consumed it; four wavefronts form a workgroup and share the staged
// activation rows. A group's depth is shared out over 1, 2 or 4 wavefronts of the workgroup
// (int32 partial tiles added through LDS: exact). The activation rows are requested before the
// first weight load and staged in LDS while the ring fills. In the hybrid form the staging
// step *is* the BatchQuantizeFloats of the op: the workgroup reduces min/max of each float
// row, derives scale and zero point, and writes the quantized row straight to LDS, so the op
// is a single kernel.
#include "fc_epilogues.h"
#include "kernels.h"
#include "quantize_device.h"

namespace lrtfc {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWaveSize;
constexpr int kTileRows = 16;
constexpr int kSlabDepth = 64;
constexpr int kQPad = 16;         // bytes of padding per staged activation row (bank spread)

__global__ __launch_bounds__(kThreads) void PackInt8FilterKernel(const int8_t* __restrict__ src,
                                                                 int out_depth, int depth,
                                                                 int slabs, int64_t chunks,
                                                                 int8_t* __restrict__ dst) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (c >= chunks) return;
  const int lane = static_cast<int>(c & 63);
  const int64_t tile_slab = c >> 6;
  const int slab = static_cast<int>(tile_slab % slabs);
  const int tile = static_cast<int>(tile_slab / slabs);
  const int row = tile * kTileRows + (lane & 15);
  const int k0 = slab * kSlabDepth + (lane >> 4) * 16;
  int8_t out[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    const int k = k0 + t;
    out[t] = (row < out_depth && k < depth) ? src[static_cast<size_t>(row) * depth + k] : 0;
  }
  *reinterpret_cast<i32x4*>(dst + c * 16) = *reinterpret_cast<const i32x4*>(out);
}

struct PackedArgs {
  FcInt8Args a;            // a.filter is the packed filter; a.input the int8 rows (unfused)
  const float* input_f32;  // fused form: float rows to quantize in the prologue
  int asymmetric;
  int slabs;               // padded depth / 64
};

// LDS map (dynamic): [bt rows x (slabs * 64 + kQPad)] int8 activations, then the
// cross-wave partial tiles, then per-row quantization state.
struct Shared {
  int8_t* q;
  i32x4* partial;  // [kWaves][64]
  float* sf;       // [16]
  float* inv;      // [16]
  int32_t* zp;     // [16]
  int32_t* zero;   // [16]
  float* mm;       // [16][kWaves][2]
};

__device__ __forceinline__ Shared CarveShared(int8_t* base, int bt, int qstride,
                                              int waves = kWaves) {
  Shared s;
  s.q = base;
  size_t off = (static_cast<size_t>(bt) * qstride + 15) & ~static_cast<size_t>(15);
  s.partial = reinterpret_cast<i32x4*>(base + off);
  off += waves * 64 * sizeof(i32x4);
  s.sf = reinterpret_cast<float*>(base + off);
  off += 16 * 4;
  s.inv = reinterpret_cast<float*>(base + off);
  off += 16 * 4;
  s.zp = reinterpret_cast<int32_t*>(base + off);
  off += 16 * 4;
  s.zero = reinterpret_cast<int32_t*>(base + off);
  off += 16 * 4;
  s.mm = reinterpret_cast<float*>(base + off);
  return s;
}

size_t SharedBytes(int bt, int qstride, int waves = kWaves) {
  return ((static_cast<size_t>(bt) * qstride + 15) & ~static_cast<size_t>(15)) +
         waves * 64 * sizeof(i32x4) + 4 * 16 * 4 + 16 * waves * 2 * 4;
}

constexpr int kRing = 16;  // weight tiles in flight per wavefront

// REG_ROWS: how many float rows the fused prologue may keep in registers (1, 2 or 4); a
// smaller value frees registers. Without the fused prologue it scales the registers that hold
// already quantized rows on their way to LDS (4 KiB of int8 per workgroup and unit). ksplit:
// wavefronts sharing one channel group (1, 2, 4).
//
// The leading scalar arguments repeat what the first loads need (filter and row addresses,
// shapes). The library is built with kernel-argument preloading, which hands the leading
// scalar arguments to a wavefront in registers when it starts; everything else is read from
// the argument segment as usual, ~0.5 us later, when the prologue has long begun (measured:
// 12.55 -> 12.28 us per launch at 14336 x 4096, B = 1).
// XREGS: 16-byte pieces of a float row a thread holds between the two passes of the fused
// prologue (4, 8 or 16: rows up to 4096, 8192, 16384 deep); REG_ROWS * XREGS stays at 16 or less.
template <Int8Epilogue EPI, bool FUSED, int VARIANT, int REG_ROWS, int XREGS>
__global__ __launch_bounds__(kThreads) void FcInt8PackedGemvKernel(
    const int8_t* early_filter, const float* early_input_f32, int early_depth, int early_slabs,
    int early_out_depth, int batch0, int bt, int ksplit, PackedArgs p) {
  extern __shared__ __align__(16) int8_t smem[];
  const FcInt8Args& a = p.a;
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = tid / kWaveSize;
  const int col = lane & 15;     // batch column of this lane in the MFMA tiles
  const int kgroup = lane >> 4;  // which 16 of a tile's 64 depth positions this lane holds
  const int slabs = early_slabs;
  const int depth = early_depth;
  const int qstride = slabs * kSlabDepth + kQPad;
  const Shared sh = CarveShared(smem, bt, qstride);
  const int tiles = (early_out_depth + kTileRows - 1) / kTileRows;
  const int tiles_per_wg = kWaves / ksplit;
  const int tile = blockIdx.x * tiles_per_wg + wave / ksplit;  // may run past the last group
  const int part = wave % ksplit;
  const int per_part = (slabs + ksplit - 1) / ksplit;
  const int s0 = part * per_part;
  const int s1 = min(slabs, s0 + per_part);
  const i32x4* wbase = reinterpret_cast<const i32x4*>(early_filter) +
                       (static_cast<size_t>(min(tile, tiles - 1)) * slabs) * 64 + lane;

  // Vector memory returns in issue order, so whatever the prologue needs must be requested
  // BEFORE the weight loads: then waiting for it leaves the weight loads in flight. Small
  // activation tiles are therefore fetched into registers first (kXRegs float4 per row per
  // thread for up to REG_ROWS rows, or kQRegs 16-byte chunks of int8), without branches;
  // larger ones are staged completely before the weights are requested.
  constexpr int kXRegs = XREGS, kQRegs = 4 * REG_ROWS;
  const int padded = slabs * kSlabDepth;
  const int vector_end = depth - (depth % 8);
  float4 xr[REG_ROWS][kXRegs];
  i32x4 qr[kQRegs];
  bool in_regs = false;
  if (FUSED) {
    const bool vec_ok =
        (depth % 4 == 0) && ((reinterpret_cast<uintptr_t>(early_input_f32) & 15) == 0);
    in_regs = vec_ok && bt <= REG_ROWS && depth <= kXRegs * kThreads * 4;
    if (in_regs) {
#pragma unroll
      for (int b = 0; b < REG_ROWS; ++b) {
#pragma unroll
        for (int j = 0; j < kXRegs; ++j) {
          const int i = (j * kThreads + tid) * 4;
          // Raw, clamped load; nothing may consume it before the weight loads are out.
          xr[b][j] = *reinterpret_cast<const float4*>(
              early_input_f32 + static_cast<size_t>(batch0 + min(b, bt - 1)) * depth +
              min(i, depth - 4));
        }
      }
    } else {
      // Slow form: the min/max pass reads memory before any weight load.
      for (int b = 0; b < bt; ++b) {
        const float* x = p.input_f32 + static_cast<size_t>(batch0 + b) * depth;
        float mn = 0.0f, mx = 0.0f;
        if (vec_ok) {
          for (int i = tid * 4; i < depth; i += kThreads * 4) {
            const float4 t = *reinterpret_cast<const float4*>(x + i);
            mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
            mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
          }
        } else {
          for (int i = tid; i < depth; i += kThreads) {
            mn = fminf(mn, x[i]);
            mx = fmaxf(mx, x[i]);
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
  } else {
    const bool vec_ok = (depth % 16 == 0) && ((reinterpret_cast<uintptr_t>(a.input) & 15) == 0);
    in_regs = vec_ok && bt * (padded / 16) <= kQRegs * kThreads;
    if (in_regs) {
      const int chunks_per_row = padded / 16;
#pragma unroll
      for (int j = 0; j < kQRegs; ++j) {
        const int c = j * kThreads + tid;
        const int b = c / chunks_per_row;
        const int i = (c - b * chunks_per_row) * 16;
        qr[j] = *reinterpret_cast<const i32x4*>(
            a.input + static_cast<size_t>(batch0 + min(b, bt - 1)) * depth + min(i, depth - 16));
      }
    } else {
      for (int b = 0; b < bt; ++b) {
        const int8_t* x = a.input + static_cast<size_t>(batch0 + b) * depth;
        int8_t* qrow = sh.q + b * qstride;
        if (vec_ok) {
          for (int i = tid * 16; i < padded; i += kThreads * 16) {
            i32x4 v = {0, 0, 0, 0};
            if (i < depth) v = *reinterpret_cast<const i32x4*>(x + i);
            *reinterpret_cast<i32x4*>(qrow + i) = v;
          }
        } else {
          for (int i = tid; i < padded; i += kThreads) qrow[i] = i < depth ? x[i] : 0;
        }
      }
    }
  }

  // Per-channel epilogue parameters of this lane's four channels, requested here: after the
  // activation rows (which the prologue waits for) and BEFORE the weights. Vector memory
  // returns in issue order and the tile loop waits with a fixed count of newer loads allowed
  // in flight; parameters requested behind the ring count as newer loads in the first round
  // and make the first MFMA wait for the whole ring instead of its first tile (measured:
  // 0.3-0.4 us per launch). Every load is unconditional -- an absent array reads a valid dummy
  // address and is ignored -- so that the number of loads in flight does not depend on the
  // path taken. (Scalar loads for these -- the 16 channels are uniform across the wavefront --
  // were measured slower: dozens of serialized scalar-cache round trips in the prologue.)
  // Loaded raw; combined in the epilogue.
  int32_t ep_i0[4], ep_i1[4], ep_i2[4], ep_i3[4];  // requantize: multiplier, shift, bias, row sum
  float ep_f0[4], ep_f1[4];                         // hybrid: channel scale, bias (+ ep_i0 row sum)
  {
    const int32_t* dummy_i = reinterpret_cast<const int32_t*>(a.filter);
    const float* dummy_f = reinterpret_cast<const float*>(a.filter);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = min(min(tile, tiles - 1) * kTileRows + 4 * kgroup + i, a.out_depth - 1);
      if (EPI == Int8Epilogue::kRequantize) {
        ep_i0[i] = a.multipliers[a.per_channel ? n : 0];
        ep_i1[i] = a.shifts[a.per_channel ? n : 0];
        ep_i2[i] = *(a.bias_i32 ? a.bias_i32 + n : dummy_i);
        ep_i3[i] = *(a.filter_row_sums ? a.filter_row_sums + n : dummy_i);
      } else {
        ep_i0[i] = *(a.filter_row_sums ? a.filter_row_sums + n : dummy_i);
        ep_f0[i] = *(a.per_channel_scales ? a.per_channel_scales + n : dummy_f);
        ep_f1[i] = *(a.bias_f32 ? a.bias_f32 + n : dummy_f);
      }
    }
  }

  // 1. Fill the first half of the ring (branch-free; a share shorter than the ring re-reads
  // its last tile). Issuing loads blocks while the memory pipeline is full -- which it is from
  // the first microsecond on -- so the second half is issued after the prologue's arithmetic
  // (step 2) rather than before it: the prologue then overlaps the wait for queue space.
  // (Three or four rows make the prologue long enough for three quarters of the ring to pay:
  // 14.5 -> 14.2 us at B = 4; at one or two rows the half ring is as good or better.)
  constexpr int kFirst = (FUSED && REG_ROWS >= 4) ? kRing * 3 / 4 : kRing / 2;
  i32x4 ring[kRing];
#pragma unroll
  for (int u = 0; u < kFirst; ++u) {
    ring[u] = __builtin_nontemporal_load(wbase + static_cast<size_t>(min(s0 + u, slabs - 1)) * 64);
  }

  // 2. Activation rows into LDS, zero-padded to the slab grid. In the fused form this is
  // the op's BatchQuantizeFloats.
  if (FUSED) {
    if (in_regs) {
#pragma unroll
      for (int b = 0; b < REG_ROWS; ++b) {
        if (b < bt) {
          float mn = 0.0f, mx = 0.0f;
#pragma unroll
          for (int j = 0; j < kXRegs; ++j) {
            // lanes past the row hold a clamped duplicate of real elements: harmless for min/max
            const float4 t = xr[b][j];
            mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
            mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
          }
          mn = WaveMinF32(mn);
          mx = WaveMaxF32(mx);
          if (lane == 0) {
            sh.mm[(b * kWaves + wave) * 2] = mn;
            sh.mm[(b * kWaves + wave) * 2 + 1] = mx;
          }
        }
      }
    }
    __syncthreads();
    if (tid < bt) {  // one lane per row derives that row's scale and zero point
      float mn = sh.mm[tid * kWaves * 2], mx = sh.mm[tid * kWaves * 2 + 1];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) {
        mn = fminf(mn, sh.mm[(tid * kWaves + w) * 2]);
        mx = fmaxf(mx, sh.mm[(tid * kWaves + w) * 2 + 1]);
      }
      const RowQuantParams qp =
          p.asymmetric ? AsymmetricRowParams<VARIANT>(mn, mx) : SymmetricRowParams(mn, mx);
      sh.sf[tid] = qp.scale;
      sh.inv[tid] = ElementwiseInv(qp);
      sh.zp[tid] = qp.zero_point;
      sh.zero[tid] = qp.all_zero ? 1 : 0;
    }
    __syncthreads();
    if (in_regs) {
#pragma unroll
      for (int b = 0; b < REG_ROWS; ++b) {
        if (b < bt) {
          RowQuantParams qp;
          qp.scale = sh.sf[b];
          qp.inv = sh.inv[b];
          qp.zero_point = sh.zp[b];
          qp.all_zero = sh.zero[b] != 0;
          int8_t* qrow = sh.q + b * qstride;
#pragma unroll
          for (int j = 0; j < kXRegs; ++j) {
            const int i = (j * kThreads + tid) * 4;
            if (i < padded) {
              int32_t packed = 0;
              if (i < depth) {
                const float4 t = xr[b][j];
                const bool tail = i >= vector_end;
                packed = QuantizePack4<VARIANT>(t.x, t.y, t.z, t.w, qp, tail);
              }
              *reinterpret_cast<int32_t*>(qrow + i) = packed;
            }
          }
        }
      }
    } else {
      const bool vec_ok =
          (depth % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.input_f32) & 15) == 0);
      for (int b = 0; b < bt; ++b) {
        const float* x = p.input_f32 + static_cast<size_t>(batch0 + b) * depth;
        RowQuantParams qp;
        qp.scale = sh.sf[b];
        qp.inv = sh.inv[b];
        qp.zero_point = sh.zp[b];
        qp.all_zero = sh.zero[b] != 0;
        int8_t* qrow = sh.q + b * qstride;
        if (vec_ok) {
          for (int i = tid * 4; i < padded; i += kThreads * 4) {
            int32_t packed = 0;
            if (i < depth) {
              const float4 t = *reinterpret_cast<const float4*>(x + i);
              const bool tail = i >= vector_end;
              packed = QuantizePack4<VARIANT>(t.x, t.y, t.z, t.w, qp, tail);
            }
            *reinterpret_cast<int32_t*>(qrow + i) = packed;
          }
        } else {
          for (int i = tid; i < padded; i += kThreads) {
            qrow[i] = i < depth ? static_cast<int8_t>(QuantizeElement<VARIANT>(
                                      x[i], qp, p.asymmetric, i >= vector_end))
                                : 0;
          }
        }
      }
    }
  } else if (in_regs) {
    const int chunks_per_row = padded / 16;
#pragma unroll
    for (int j = 0; j < kQRegs; ++j) {
      const int c = j * kThreads + tid;
      const int b = c / chunks_per_row;
      const int i = (c - b * chunks_per_row) * 16;
      if (b < bt) {
        *reinterpret_cast<i32x4*>(sh.q + b * qstride + i) = i < depth ? qr[j] : i32x4{0, 0, 0, 0};
      }
    }
  }
  __syncthreads();

  // The rest of the ring.
#pragma unroll
  for (int u = kFirst; u < kRing; ++u) {
    ring[u] = __builtin_nontemporal_load(wbase + static_cast<size_t>(min(s0 + u, slabs - 1)) * 64);
  }

  // 3. Matrix-core loop. B operand: lane L supplies batch column (L % 16), the same 16
  // depth positions as its weight bytes. Columns past the tile read row 0; their
  // results are never stored. Four accumulators break the MFMA dependency chain.
  const int8_t* qbase = sh.q + (col < bt ? col : 0) * qstride + kgroup * 16;
  constexpr int kAccs = 4;  // independent accumulators (eight measured slower: 15.9 vs 13.2 us)
  i32x4 acc4[kAccs];
#pragma unroll
  for (int i = 0; i < kAccs; ++i) acc4[i] = i32x4{0, 0, 0, 0};
  int base = s0;
  for (; base + kRing < s1; base += kRing) {  // full rounds: consume a slot, refill it
#pragma unroll
    for (int g = 0; g < kRing; g += 4) {
      i32x4 bq[4];  // four activation operands per LDS wait
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        bq[u] = *reinterpret_cast<const i32x4*>(qbase + (base + g + u) * kSlabDepth);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc4[(g + u) % kAccs] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
            ring[g + u], bq[u], acc4[(g + u) % kAccs], 0, 0, 0);
        ring[g + u] = __builtin_nontemporal_load(
            wbase + static_cast<size_t>(min(base + kRing + g + u, slabs - 1)) * 64);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kRing; ++u) {  // last turn of the ring
    if (base + u < s1) {
      const i32x4 bq = *reinterpret_cast<const i32x4*>(qbase + (base + u) * kSlabDepth);
      acc4[u % kAccs] =
          __builtin_amdgcn_mfma_i32_16x16x64_i8(ring[u], bq, acc4[u % kAccs], 0, 0, 0);
    }
  }
  i32x4 acc = (acc4[0] + acc4[1]) + (acc4[2] + acc4[3]);

  // 4. Depth shares of one channel group meet in LDS.
  if (ksplit > 1) {
    sh.partial[wave * 64 + lane] = acc;
    __syncthreads();
    if (part != 0) return;
    for (int w = 1; w < ksplit; ++w) acc += sh.partial[(wave + w) * 64 + lane];
  }

  // 5. Epilogue. Accumulator register i holds channel 4 * (L / 16) + i, column L % 16.
  if (col >= bt || tile >= tiles) return;
  const int b = batch0 + col;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = tile * kTileRows + 4 * kgroup + i;
    if (n >= a.out_depth) continue;
    if (EPI == Int8Epilogue::kRequantize) {
      const int32_t bias = a.bias_i32 ? ep_i2[i] : 0;
      const int32_t row_sum = a.filter_row_sums ? ep_i3[i] : 0;  // input_offset != 0 needs them
      a.output_i8[static_cast<size_t>(b) * a.out_depth + n] =
          RequantizeCore(acc[i] + bias + a.input_offset * row_sum, ep_i0[i], ep_i1[i],
                         a.output_offset, a.act_min, a.act_max);
    } else {
      const float batch_scale = FUSED ? sh.sf[col] : a.scaling_factors[b];
      const int32_t batch_zp = FUSED ? sh.zp[col] : (a.zero_points ? a.zero_points[b] : 0);
      const float channel_scale = a.per_channel_scales ? ep_f0[i] : a.filter_scale;
      const float bias = a.bias_f32 ? ep_f1[i] : 0.0f;
      const int32_t row_sum = a.filter_row_sums ? ep_i0[i] : 0;
      float value;
      if (EPI == Int8Epilogue::kHybrid4Bit) {
        value = Hybrid4BitCore(acc[i], batch_scale, channel_scale, batch_zp, bias,
                               a.bias_f32 != nullptr, a.activation);
      } else if (FUSED) {
        // Whole-zero input (fully_connected.cc:789-795): this launch knows its own rows from
        // the prologue; rows of other launches of the same call are scanned, lazily.
        bool zero_input = false;
        if (sh.zero[col] != 0 && IsNegativeZero(bias)) {
          zero_input = true;
          for (int r = 0; r < bt; ++r) zero_input = zero_input && sh.zero[r] != 0;
          if (zero_input && a.batches > bt) {
            zero_input = AllZeroF32(p.input_f32, static_cast<size_t>(a.batches) * depth);
          }
        }
        value = zero_input ? ApplyFloatActivation(bias, a.activation)
                           : HybridCore(acc[i], batch_scale, channel_scale, batch_zp, row_sum,
                                        bias, a.activation);
      } else {
        value = HybridCoreZeroAware(a, acc[i], batch_scale, channel_scale, batch_zp, row_sum,
                                    bias);
      }
      a.output_f32[static_cast<size_t>(b) * a.out_depth + n] = value;
    }
  }
}

// ---- the form for filters a launch can hold in its registers --------------------------------
//
// A decode launch of this size is a chain of latencies in front of a stream: the memory system
// needs about 8 us for 58 MB however the loads are arranged, and every microsecond in which
// loads that could have been in flight were not is added to that. A ring that is refilled as
// it is consumed ties the stream to the consumer: a slot is requested again only after the
// product that empties it, and nothing beyond the ring is requested until the activation rows
// are quantized and staged. This form unties them. Every tile of a wavefront's share of the
// depth (at most TILES tiles of 1 KiB) has a variable of its own in straight-line code, so in
// program order a request never waits for a product (the tiles between request and product
// are what stays live in registers: kStreamAhead at the barrier, about kStreamLag afterwards):
//   * kAhead tiles are requested before anything waits for anything; the one barrier of the
//     kernel (rows staged) follows, and from there on the wavefront alternates "request tile
//     u" with "multiply tile u - kLag", in straight-line code whose waits the compiler counts
//     exactly. A compute unit accepts only some tens of KiB of outstanding loads, so a
//     wavefront spends most of its time blocked in load issue: whatever it has to compute
//     must sit between two requests, not behind the last one.
//   * The per-row work is given to single wavefronts: wavefront r of a workgroup (r < rows)
//     reads row r into its registers, reduces it, derives the row's parameters and writes the
//     quantized row to LDS on its own, with no workgroup-wide step. Its row loads must not
//     queue behind the other wavefronts' weight requests (the vector memory path of a compute
//     unit serves requests in order): it runs at raised priority until the row is requested,
//     and the others hold their first request back for some hundred cycles.

constexpr int kFusedRowMaxDepth = 4096;  // a wavefront holds its row in 16 x 16 bytes per lane
constexpr int kFusedMaxRows = 8;          // one wavefront of eight per row
constexpr int kStreamLag = 12;    // products trail the requests by this many tiles
constexpr int kStreamAhead = 24;  // tiles requested before the barrier (wavefronts without a row)

// Where `PackedArgs p` lies in the kernel's argument segment: behind three pointers and seven
// ints, at its own alignment.
struct ResidentLeadingArgs {
  const void* pointers[3];
  int ints[7];
};
constexpr size_t kResidentPackedArgsOffset =
    (sizeof(ResidentLeadingArgs) + alignof(PackedArgs) - 1) / alignof(PackedArgs) * alignof(PackedArgs);
static_assert(kResidentPackedArgsOffset == 56, "argument layout of FcInt8ResidentGemvKernel");

template <Int8Epilogue EPI, bool FUSED, int VARIANT, int TILES, bool EARLY, int WAVES, int RT = 1>
__global__ __launch_bounds__(WAVES * kWaveSize)
__attribute__((amdgpu_waves_per_eu(WAVES / 2 / RT, WAVES / 2 / RT)))
void FcInt8ResidentGemvKernel(
    const int8_t* early_filter, const float* early_input_f32, const int8_t* early_input_i8,
    int early_depth, int early_slabs, int early_out_depth, int batch0, int bt, int ksplit_log2,
    int per_part, PackedArgs p) {
  extern __shared__ __align__(16) int8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int ksplit = 1 << ksplit_log2;
  // The wavefront's index as a scalar: everything derived from it (its channel group, its
  // share of the depth, whether it has a row to quantize) is then uniform to the compiler,
  // which keeps the branches scalar and the tile addresses in scalar registers.
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWaveSize);
  const int col = lane & 15;
  const int kgroup = lane >> 4;
  const int slabs = early_slabs;
  const int depth = early_depth;
  // per_part = ceil(slabs / ksplit) <= TILES (the launcher's choice). A staged row is
  // zero-filled up to the end of the last share, so that a share that runs past the depth
  // multiplies its (clamped, re-read) tiles by zeros instead of branching.
  const int staged = ksplit * per_part * kSlabDepth;
  const int qstride = staged + kQPad;
  // RT: tiles of 16 batch rows a wavefront multiplies each weight tile with (2: 17 to 32 rows
  // that arrive quantized; every row of a workgroup's LDS image is then read by eight
  // wavefronts instead of four, and the workgroup has its compute unit to itself).
  static_assert(RT == 1 || (RT == 2 && !FUSED), "two row tiles: rows that arrive quantized");
  const Shared sh = CarveShared(smem, bt, qstride, WAVES * RT);
  const int tiles = (early_out_depth + kTileRows - 1) / kTileRows;
  const int tile = ((blockIdx.x * WAVES) >> ksplit_log2) + (wave >> ksplit_log2);
  const int part = wave & (ksplit - 1);
  const int s0 = part * per_part;
  const int8_t* group_base =
      early_filter + static_cast<size_t>(min(tile, tiles - 1)) * slabs * 1024;  // uniform
  // The argument segment beyond the leading (preloaded) arguments, as a pointer the compiler
  // cannot see through: scalar loads through it stay where the code asks for them. Read in the
  // ordinary way, the compiler moves every argument load to the kernel's entry, and the first
  // weight request -- which needs the preloaded arguments only -- waits behind a fetch of the
  // argument segment from memory.
  using LateArgs = const __attribute__((address_space(4))) PackedArgs;
  auto late_args = [&]() -> LateArgs* {
    auto* segment = (const __attribute__((address_space(4))) char*)
        __builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(segment));
    return (LateArgs*)(segment + kResidentPackedArgsOffset);
  };
  i32x4 ring[TILES];
  auto request = [&](int u) {
    // Past the share or the depth: the share's last tile again (a hit in the nearest cache).
    const int8_t* t =
        group_base + static_cast<size_t>(min(s0 + min(u, per_part - 1), slabs - 1)) * 1024;
    ring[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(t + lane * 16));
    __builtin_amdgcn_sched_barrier(0);  // issue order = the order the products take them in
  };

  // The row parameters of this lane's batch column: read from LDS behind the barrier (fused) or
  // requested with the per-channel parameters (rows that arrive quantized).
  float lds_scale[RT] = {};
  int32_t lds_zp[RT] = {};
  int32_t lds_zero = 0;
  bool ep_has_row_zero_points = false;
  // Per-channel epilogue parameters, requested behind the first tiles (they are needed last).
  // Unconditional loads: an absent array reads a valid dummy address.
  int32_t ep_i0[4], ep_i1[4], ep_i2[4], ep_i3[4];
  float ep_f0[4], ep_f1[4];
  auto request_parameters = [&]() {
    // Pointers from the argument segment, read HERE (see late_args).
    const LateArgs* late = late_args();
    const int out_depth = early_out_depth;
    const int32_t* dummy_i = reinterpret_cast<const int32_t*>(early_filter);
    const float* dummy_f = reinterpret_cast<const float*>(early_filter);
    if (EPI == Int8Epilogue::kRequantize) {
      const int32_t* multipliers = late->a.multipliers;
      const int32_t* shifts = late->a.shifts;
      const int32_t* bias = late->a.bias_i32;
      const int32_t* row_sums = late->a.filter_row_sums;
      const int per_channel = late->a.per_channel;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = min(min(tile, tiles - 1) * kTileRows + 4 * kgroup + i, out_depth - 1);
        ep_i0[i] = multipliers[per_channel ? n : 0];
        ep_i1[i] = shifts[per_channel ? n : 0];
        ep_i2[i] = *(bias ? bias + n : dummy_i);
        ep_i3[i] = *(row_sums ? row_sums + n : dummy_i);
      }
    } else {
      const int32_t* row_sums = late->a.filter_row_sums;
      const float* scales = late->a.per_channel_scales;
      const float* bias = late->a.bias_f32;
      if (!FUSED) {
        // The rows' own parameters: a global load in the epilogue would queue behind the
        // whole weight stream.
        const float* row_scales = late->a.scaling_factors;
        const int32_t* row_zero_points = late->a.zero_points;
#pragma unroll
        for (int r = 0; r < RT; ++r) {
          const int row = batch0 + min(col + 16 * r, bt - 1);
          lds_scale[r] = row_scales[row];
          lds_zp[r] = *(row_zero_points ? row_zero_points + row : dummy_i);
        }
        ep_has_row_zero_points = row_zero_points != nullptr;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = min(min(tile, tiles - 1) * kTileRows + 4 * kgroup + i, out_depth - 1);
        ep_i0[i] = *(row_sums ? row_sums + n : dummy_i);
        ep_f0[i] = *(scales ? scales + n : dummy_f);
        ep_f1[i] = *(bias ? bias + n : dummy_f);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // The epilogue's scalar inputs, read from the argument segment where `stream` says (while the
  // wavefront waits at the barrier anyway: a scalar load issued at the end of the kernel queues
  // behind the whole chip's weight stream).
  void* ep_out;
  int ep_activation, ep_flags, ep_batches;
  float ep_filter_scale;
  int32_t ep_offsets0, ep_offsets1, ep_offsets2, ep_offsets3;
  auto fetch_epilogue_scalars = [&]() {
    const LateArgs* late = late_args();
    ep_out = EPI == Int8Epilogue::kRequantize ? static_cast<void*>(late->a.output_i8)
                                              : static_cast<void*>(late->a.output_f32);
    ep_activation = late->a.activation;
    ep_flags = (late->a.bias_i32 ? 1 : 0) | (late->a.filter_row_sums ? 2 : 0) |
               (late->a.per_channel_scales ? 4 : 0) | (late->a.bias_f32 ? 8 : 0) |
               (late->a.zero_input_exit ? 32 : 0) | (late->a.batch_matmul ? 64 : 0);
    ep_filter_scale = late->a.filter_scale;
    ep_offsets0 = late->a.input_offset;
    ep_offsets1 = late->a.output_offset;
    ep_offsets2 = late->a.act_min;
    ep_offsets3 = late->a.act_max;
    ep_batches = late->a.batches;
  };
  const int8_t* qbase[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    qbase[r] = sh.q + (col + 16 * r < bt ? col + 16 * r : 0) * qstride + kgroup * 16 +
               s0 * kSlabDepth;
  }
  const int8_t* pad_zero = sh.q + staged;  // the kQPad bytes behind row 0, cleared below
  constexpr int kAccs = 4;
  i32x4 acc4[RT][kAccs];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int i = 0; i < kAccs; ++i) acc4[r][i] = i32x4{0, 0, 0, 0};
  // Products of tiles g .. g + 3: four activation operands (per row tile) per LDS wait.
  auto multiply4 = [&](int g) {
    i32x4 bq[RT][4];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        // Past the share (which only happens when TILES is larger than the share) the operand
        // is the 16 bytes of zeros behind row 0.
        const int8_t* at = g + u < per_part ? qbase[r] + (g + u) * kSlabDepth : pad_zero;
        bq[r][u] = *reinterpret_cast<const i32x4*>(at);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        acc4[r][u] =
            __builtin_amdgcn_mfma_i32_16x16x64_i8(ring[g + u], bq[r][u], acc4[r][u], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // Tiles [0, first) are requested; requests up to `ahead`, the barrier, then requests and
  // products in alternation, the products kLag tiles behind.
  auto stream = [&](auto first_c, auto ahead_c) {
    constexpr int kFirst = decltype(first_c)::value;
    constexpr int kAhead = decltype(ahead_c)::value < TILES ? decltype(ahead_c)::value : TILES;
    constexpr int kLag = kStreamLag < kAhead ? kStreamLag : kAhead;
    static_assert(kFirst <= kAhead && kAhead % 4 == 0 && kLag % 4 == 0 && TILES % 4 == 0, "");
#pragma unroll
    for (int u = kFirst; u < kAhead; ++u) request(u);
    request_parameters();
    if (tid < 4) *reinterpret_cast<int32_t*>(sh.q + staged + tid * 4) = 0;  // pad_zero
    // What the epilogue reads from the argument segment is fetched here, while the wavefront
    // waits at the barrier anyway: a scalar load issued at the end of the kernel queues behind
    // the whole chip's weight stream and costs some hundred nanoseconds of every launch.
    fetch_epilogue_scalars();
    __syncthreads();
    if (FUSED) {  // the row's parameters for the epilogue, while nothing waits for them
      lds_scale[0] = sh.sf[col < bt ? col : 0];
      lds_zp[0] = sh.zp[col < bt ? col : 0];
      lds_zero = sh.zero[col < bt ? col : 0];
    }
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
      // This wavefront's row: 16 pieces of 16 bytes per lane (depth <= 4096).
      constexpr int kPieces = 16;
      constexpr int kEarly = EARLY ? (WAVES > 4 ? 4 : (TILES < 8 ? TILES : 8)) : 0;
      const float* x = early_input_f32 + static_cast<size_t>(batch0 + wave) * depth;
      float4 xr[kPieces];
#pragma unroll
      for (int j = 0; j < kPieces; ++j) {
        const int i = (j * kWaveSize + lane) * 4;
        xr[j] = *reinterpret_cast<const float4*>(x + min(i, depth - 4));
      }
      __builtin_amdgcn_sched_barrier(0);
      if (EARLY) {
        // Every wavefront of the workgroup has a row: some weights go out ahead of the row's
        // arithmetic, or nothing would be in flight meanwhile.
#pragma unroll
        for (int u = 0; u < kEarly; ++u) request(u);
      }
      float mn = 0.0f, mx = 0.0f;
#pragma unroll
      for (int j = 0; j < kPieces; ++j) {
        const float4 t = xr[j];  // past the row: a clamped duplicate, harmless for min/max
        mn = fminf(fminf(mn, t.x), fminf(fminf(t.y, t.z), t.w));
        mx = fmaxf(fmaxf(mx, t.x), fmaxf(fmaxf(t.y, t.z), t.w));
      }
      mn = WaveMinF32(mn);
      mx = WaveMaxF32(mx);
      const int asymmetric = late_args()->asymmetric;
      RowQuantParams qp =
          asymmetric ? AsymmetricRowParams<VARIANT>(mn, mx) : SymmetricRowParams(mn, mx);
      if (lane == 0) {
        sh.sf[wave] = qp.scale;
        sh.zp[wave] = qp.zero_point;
        sh.zero[wave] = qp.all_zero ? 1 : 0;
      }
      qp.inv = ElementwiseInv(qp);
      const int vector_end = depth - (depth % 8);
      int8_t* qrow = sh.q + wave * qstride;
      // A row of exactly 16 pieces per lane needs no test per piece (each test is a basic block
      // of its own and keeps the pieces' arithmetic from overlapping).
      auto quantize_pieces = [&](auto whole_c) {
        constexpr bool kWhole = decltype(whole_c)::value;
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
          const int i = (j * kWaveSize + lane) * 4;
          const float4 t = xr[j];
          int32_t packed =
              QuantizePack4<VARIANT>(t.x, t.y, t.z, t.w, qp, kWhole ? false : i >= vector_end);
          if (!kWhole) packed = i < depth ? packed : 0;
          if (kWhole || i < staged) *reinterpret_cast<int32_t*>(qrow + i) = packed;
        }
      };
      if (depth == kPieces * kWaveSize * 4) {
        quantize_pieces(std::true_type{});
      } else {
        quantize_pieces(std::false_type{});
      }
      // Zeros between 16 pieces' worth and the end of the last share (a few slabs at most).
      for (int i = kPieces * kWaveSize * 4 + lane * 4; i < staged; i += kWaveSize * 4) {
        *reinterpret_cast<int32_t*>(qrow + i) = 0;
      }
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      stream(integral_constant<int, kEarly>{}, integral_constant<int, (kEarly > kStreamLag ? kEarly : kStreamLag)>{});
    } else {
      __builtin_amdgcn_s_sleep(8);  // 512 cycles: the rows' requests go first
      stream(integral_constant<int, 0>{}, integral_constant<int, kStreamAhead>{});
    }
  } else {
    // Rows that arrive quantized: up to 16 rows of depth 4096, 16 bytes per thread and piece,
    // requested ahead of the weights and written to LDS when they are there.
    // 16-byte pieces of quantized rows per thread: 4 rows of depth 4096, or 16 (EARLY, which
    // has no other meaning for rows that arrive quantized).
    constexpr int kQRegs = (EARLY ? 64 : 16) * RT / WAVES;
    constexpr int kFirst = TILES < 8 ? TILES : 8;
    i32x4 qr[kQRegs];
    const int chunks_per_row = staged / 16;
#pragma unroll
    for (int j = 0; j < kQRegs; ++j) {
      const int c = j * (WAVES * kWaveSize) + tid;
      const int b = min(c / chunks_per_row, bt - 1);
      const int i = (c % chunks_per_row) * 16;
      qr[j] = *reinterpret_cast<const i32x4*>(
          early_input_i8 + static_cast<size_t>(batch0 + b) * depth + min(i, depth - 16));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kFirst; ++u) request(u);
#pragma unroll
    for (int j = 0; j < kQRegs; ++j) {
      const int c = j * (WAVES * kWaveSize) + tid;
      const int b = c / chunks_per_row;
      const int i = (c % chunks_per_row) * 16;
      if (b < bt) {
        *reinterpret_cast<i32x4*>(sh.q + b * qstride + i) = i < depth ? qr[j] : i32x4{0, 0, 0, 0};
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    stream(integral_constant<int, kFirst>{}, integral_constant<int, kStreamAhead>{});
  }
  i32x4 acc_of[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc_of[r] = (acc4[r][0] + acc4[r][1]) + (acc4[r][2] + acc4[r][3]);

  if (ksplit > 1) {
#pragma unroll
    for (int r = 0; r < RT; ++r) sh.partial[(r * WAVES + wave) * 64 + lane] = acc_of[r];
    __syncthreads();
    if (part != 0) return;
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      for (int w = 1; w < ksplit; ++w) acc_of[r] += sh.partial[(r * WAVES + wave + w) * 64 + lane];
    }
  }

  if (tile >= tiles) return;
  // The epilogue of one row tile: this lane's row is col + 16 * r.
  auto finish = [&](int r, const i32x4 acc) {
  if (col + 16 * r >= bt) return;
  const int b = batch0 + col + 16 * r;
  const int out_depth = early_out_depth;
  const int n0 = tile * kTileRows + 4 * kgroup;  // this lane's four channels: n0 .. n0 + 3
  if (EPI == Int8Epilogue::kRequantize) {
    int32_t q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int32_t bias = (ep_flags & 1) ? ep_i2[i] : 0;
      const int32_t row_sum = (ep_flags & 2) ? ep_i3[i] : 0;
      q[i] = RequantizeCore(acc[i] + bias + ep_offsets0 * row_sum, ep_i0[i], ep_i1[i],
                            ep_offsets1, ep_offsets2, ep_offsets3);
    }
    int8_t* out = static_cast<int8_t*>(ep_out) + static_cast<size_t>(b) * out_depth + n0;
    if (n0 + 4 <= out_depth && (reinterpret_cast<uintptr_t>(out) & 3) == 0) {
      *reinterpret_cast<int32_t*>(out) = PackLowBytes(q[0], q[1], q[2], q[3]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n0 + i < out_depth) out[i] = static_cast<int8_t>(q[i]);
      }
    }
    return;
  }
  // Float epilogues. The four values of a lane are computed side by side without branches (the
  // tail of the slowest wavefront is the tail of the launch); the one rare case that needs a
  // scan of the input, a whole-zero input meeting a -0.0f bias, takes a branch of its own.
  const float batch_scale = lds_scale[r];
  const int32_t batch_zp = (FUSED || ep_has_row_zero_points) ? lds_zp[r] : 0;
  const bool row_zero = FUSED ? lds_zero != 0 : true;
  float value[4];
  bool rare = false;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float channel_scale = (ep_flags & 4) ? ep_f0[i] : ep_filter_scale;
    const float bias = (ep_flags & 8) ? ep_f1[i] : 0.0f;
    const int32_t row_sum = (ep_flags & 2) ? ep_i0[i] : 0;
    if (EPI == Int8Epilogue::kHybrid4Bit) {
      // Hybrid4BitCore with the activation as selects.
      const float val = __fmul_rn(static_cast<float>(batch_zp), batch_scale);
      float out = __fmul_rn(val, channel_scale);
      if (ep_flags & 8) out = __fadd_rn(out, bias);
      const float term = __fmul_rn(static_cast<float>(acc[i] - batch_zp), batch_scale);
      out = __fadd_rn(out, __fmul_rn(term, channel_scale));
      value[i] = ApplyFloatActivationSelect(out, ep_activation);
    } else {
      const float scale = __fmul_rn(batch_scale, channel_scale);
      const float as_bmm =
          HybridBatchMatMulCore(acc[i], batch_scale, channel_scale, batch_zp, row_sum);
      const int32_t corrected = acc[i] - row_sum * batch_zp;
      const float as_fc = ApplyFloatActivationSelect(
          __fadd_rn(bias, __fmul_rn(static_cast<float>(corrected), scale)), ep_activation);
      value[i] = (!FUSED && (ep_flags & 64)) ? as_bmm : as_fc;
      // Whole-zero input (fully_connected.cc:789-795): possible only where the dot product is
      // zero under a -0.0f bias (fused: and this row quantized to zeros).
      rare = rare || (IsNegativeZero(bias) && acc[i] == 0 && row_zero);
    }
  }
  if (EPI != Int8Epilogue::kHybrid4Bit && rare && (FUSED || (ep_flags & 32)) &&
      !(ep_flags & 64)) {
    bool zero_input;
    if (FUSED) {
      // This launch knows its own rows from the prologue; rows of other launches of the same
      // call are scanned.
      zero_input = true;
      for (int r = 0; r < bt; ++r) zero_input = zero_input && sh.zero[r] != 0;
      if (zero_input && ep_batches > bt) {
        zero_input = AllZeroF32(early_input_f32, static_cast<size_t>(ep_batches) * depth);
      }
    } else {
      zero_input = AllZeroInt8(early_input_i8, static_cast<size_t>(ep_batches) * depth);
    }
    if (zero_input) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float bias = (ep_flags & 8) ? ep_f1[i] : 0.0f;
        if (IsNegativeZero(bias) && acc[i] == 0) {
          value[i] = ApplyFloatActivation(bias, ep_activation);
        }
      }
    }
  }
  float* out = static_cast<float*>(ep_out) + static_cast<size_t>(b) * out_depth + n0;
  if (n0 + 4 <= out_depth && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    *reinterpret_cast<float4*>(out) = make_float4(value[0], value[1], value[2], value[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (n0 + i < out_depth) out[i] = value[i];
    }
  }
  };
#pragma unroll
  for (int r = 0; r < RT; ++r) finish(r, acc_of[r]);
}

// How many wavefronts share one channel group's depth (see LaunchSized below).
int ChooseKsplit(int slabs, int tiles, int waves = kWaves) {
  int ksplit = 1;
  while (ksplit < waves && slabs / (ksplit * 2) >= 2 * kRing) ksplit *= 2;
  while (ksplit < waves && tiles * ksplit < 1024 && slabs / (ksplit * 2) >= 4) ksplit *= 2;
  return ksplit;
}

template <Int8Epilogue EPI, bool FUSED, int VARIANT, int TILES, bool EARLY, int WAVES = kWaves,
          int RT = 1>
hipError_t LaunchResidentSized(const PackedArgs& p, int batch0, int bt, int ksplit,
                              hipStream_t stream) {
  const int per_part = (p.slabs + ksplit - 1) / ksplit;
  const int qstride = ksplit * per_part * kSlabDepth + kQPad;
  const size_t lds = SharedBytes(bt, qstride, WAVES * RT);
  auto kernel = FcInt8ResidentGemvKernel<EPI, FUSED, VARIANT, TILES, EARLY, WAVES, RT>;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds)) return err;
  const int tiles = (p.a.out_depth + kTileRows - 1) / kTileRows;
  const int tiles_per_wg = WAVES / ksplit;
  const int grid = (tiles + tiles_per_wg - 1) / tiles_per_wg;
  int ksplit_log2 = 0;
  while ((1 << ksplit_log2) < ksplit) ++ksplit_log2;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(WAVES * kWaveSize), lds, stream, p.a.filter, p.input_f32,
                     p.a.input, p.a.depth, p.slabs, p.a.out_depth, batch0, bt, ksplit_log2,
                     per_part, p);
  return hipGetLastError();
}

// Whether the register-resident form takes this launch; *launched tells. It needs a wavefront's
// share of the depth to fit its tile registers, and rows that fit the registers set aside for
// them. Workgroups of four wavefronts with up to 32 tiles each serve one fused row and rows that
// arrive quantized; two to eight fused rows take workgroups of eight wavefronts with up to 16
// tiles each, so that the wavefronts that quantize (one per row) leave as many that only
// stream (measured at 14336 x 4096, one launch, cold: 1 row 11.0 us narrow / 11.4 wide; 2 rows
// 11.4 / 11.3; 4 rows 12.6 / 12.0; 8 rows 13.1 wide against 14.7 as row quantizer + product).
// 17 to 32 rows that arrive quantized: one pass over the filter with two row tiles per weight
// tile, on workgroups of eight wavefronts with at most 32 tiles each, as long as the rows' LDS
// image (32 x depth) fits one compute unit. *ksplit receives the depth split.
bool ResidentTwoRowTilesFit(const PackedArgs& p, int bt, int* ksplit_out) {
  if (bt <= 16 || bt > 32) return false;
  if (p.a.depth % 16 != 0 || (reinterpret_cast<uintptr_t>(p.a.input) & 15) != 0) return false;
  // The rows' image leaves room for one workgroup per compute unit, and every workgroup stages
  // the whole image: the fewest workgroups that still cover the chip in one round win (measured
  // at 14336 x 4096, 32 rows: shares of 32 tiles, 224 workgroups, 17.6 us for quantizer +
  // product; shares of 16 tiles, 448 workgroups in two rounds, 21.5 us). So: the largest share
  // (at most 32 tiles) that still gives about one workgroup per compute unit, else the split
  // with the most workgroups.
  const int tiles = (p.a.out_depth + kTileRows - 1) / kTileRows;
  int ksplit = 0;
  for (int k = 1; k <= 8; k *= 2) {
    if ((p.slabs + k - 1) / k > 32) continue;
    ksplit = k;  // candidates come with growing workgroup counts
    const int tiles_per_wg = 8 / k;
    if ((tiles + tiles_per_wg - 1) / tiles_per_wg >= 192) break;
  }
  if (ksplit == 0) return false;
  const int per_part = (p.slabs + ksplit - 1) / ksplit;
  const int staged = ksplit * per_part * kSlabDepth;
  if (static_cast<int64_t>(bt) * (staged / 16) > 16 * 8 * kWaveSize) return false;
  if (SharedBytes(bt, staged + kQPad, 16) > 150 * 1024) return false;
  if (ksplit_out) *ksplit_out = ksplit;
  return true;
}

template <Int8Epilogue EPI, bool FUSED, int VARIANT>
hipError_t TryLaunchResident(const PackedArgs& p, int batch0, int bt, hipStream_t stream,
                            bool* launched) {
  *launched = false;
  const int tiles = (p.a.out_depth + kTileRows - 1) / kTileRows;
  const int depth = p.a.depth;
  if constexpr (!FUSED) {
    if (bt > 16) {
      int ksplit = 1;
      if (!ResidentTwoRowTilesFit(p, bt, &ksplit)) return hipSuccess;
      *launched = true;
      if ((p.slabs + ksplit - 1) / ksplit <= 8) {
        return LaunchResidentSized<EPI, false, VARIANT, 8, true, 8, 2>(p, batch0, bt, ksplit, stream);
      }
      if ((p.slabs + ksplit - 1) / ksplit > 16) {
        return LaunchResidentSized<EPI, false, VARIANT, 32, true, 8, 2>(p, batch0, bt, ksplit, stream);
      }
      return LaunchResidentSized<EPI, false, VARIANT, 16, true, 8, 2>(p, batch0, bt, ksplit, stream);
    }
  }
  if (FUSED) {
    const bool vec_ok =
        (depth % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.input_f32) & 15) == 0);
    if (!vec_ok || depth > kFusedRowMaxDepth || depth < 4 || bt > kFusedMaxRows) return hipSuccess;
    if (bt > 1) {
      int ksplit = 1;
      while ((p.slabs + ksplit - 1) / ksplit > 16) ksplit *= 2;  // depth <= 4096: at most 4
      const int per_part = (p.slabs + ksplit - 1) / ksplit;
      *launched = true;
      if (per_part <= 8) {
        return bt > 4 ? LaunchResidentSized<EPI, FUSED, VARIANT, 8, true, 8>(p, batch0, bt, ksplit, stream)
                      : LaunchResidentSized<EPI, FUSED, VARIANT, 8, false, 8>(p, batch0, bt, ksplit, stream);
      }
      // Shares of 9 to 16 tiles: the quantizing wavefronts request four tiles ahead of their row's
      // arithmetic at any row count (14336 x 4096 at 2 / 3 / 4 rows: 11.2 / 11.5 / 11.9 us against
      // 11.3 / 11.6 / 12.0 us without).
      return LaunchResidentSized<EPI, FUSED, VARIANT, 16, true, 8>(p, batch0, bt, ksplit, stream);
    }
  }
  int ksplit = ChooseKsplit(p.slabs, tiles);
  while (ksplit < kWaves && (p.slabs + ksplit - 1) / ksplit > 32) ksplit *= 2;
  const int per_part = (p.slabs + ksplit - 1) / ksplit;
  if (per_part > 32) return hipSuccess;
  bool many_rows = false;
  if (!FUSED) {
    const bool vec_ok = (depth % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.a.input) & 15) == 0);
    const int64_t chunks = static_cast<int64_t>(bt) * (ksplit * per_part * kSlabDepth / 16);
    if (!vec_ok || chunks > 16 * kThreads) return hipSuccess;
    many_rows = chunks > 4 * kThreads;
  }
  *launched = true;
  if (per_part <= 8) {
    return many_rows ? LaunchResidentSized<EPI, FUSED, VARIANT, 8, !FUSED>(p, batch0, bt, ksplit, stream)
                     : LaunchResidentSized<EPI, FUSED, VARIANT, 8, false>(p, batch0, bt, ksplit, stream);
  }
  if (per_part <= 16) {
    return many_rows ? LaunchResidentSized<EPI, FUSED, VARIANT, 16, !FUSED>(p, batch0, bt, ksplit, stream)
                     : LaunchResidentSized<EPI, FUSED, VARIANT, 16, false>(p, batch0, bt, ksplit, stream);
  }
  return many_rows ? LaunchResidentSized<EPI, FUSED, VARIANT, 32, !FUSED>(p, batch0, bt, ksplit, stream)
                   : LaunchResidentSized<EPI, FUSED, VARIANT, 32, false>(p, batch0, bt, ksplit, stream);
}

template <Int8Epilogue EPI, bool FUSED, int VARIANT, int REG_ROWS, int XREGS = 4>
hipError_t LaunchSized(const PackedArgs& p, int batch0, int bt, hipStream_t stream) {
  const int qstride = p.slabs * kSlabDepth + kQPad;
  const size_t lds = SharedBytes(bt, qstride);
  auto kernel = FcInt8PackedGemvKernel<EPI, FUSED, VARIANT, REG_ROWS, XREGS>;
  if (hipError_t err = EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds)) return err;
  const int tiles = (p.a.out_depth + kTileRows - 1) / kTileRows;
  // How many wavefronts share one channel group's depth. What the memory system rewards is
  // bytes in flight: a wavefront keeps kRing tiles outstanding whatever its share, so shares
  // of about two rings (32 tiles) put twice the wavefronts -- and twice the outstanding
  // loads -- on each CU compared with one wavefront per group at depth 4096 (measured at
  // 14336 x 4096, B = 1: 13.5 -> 12.7 us; 8192 x 8192: 19.6 -> 17.2 us; shares of 16 tiles are
  // slower again). Short filters split further until the chip has a wavefront per SIMD.
  int ksplit = 1;
  while (ksplit < kWaves && p.slabs / (ksplit * 2) >= 2 * kRing) ksplit *= 2;
  while (ksplit < kWaves && tiles * ksplit < 1024 && p.slabs / (ksplit * 2) >= 4) ksplit *= 2;
  const int tiles_per_wg = kWaves / ksplit;
  const int grid = (tiles + tiles_per_wg - 1) / tiles_per_wg;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, p.a.filter, p.input_f32,
                     p.a.depth, p.slabs, p.a.out_depth, batch0, bt, ksplit, p);
  return hipGetLastError();
}

template <Int8Epilogue EPI, bool FUSED, int VARIANT>
hipError_t LaunchOne(const PackedArgs& p, int batch0, int bt, hipStream_t stream) {
  {
    bool launched = false;
    hipError_t err = TryLaunchResident<EPI, FUSED, VARIANT>(p, batch0, bt, stream, &launched);
    if (launched || err != hipSuccess) return err;
  }
  if (!FUSED) {
    // Quantized rows that fit the registers are requested before the weights and need no
    // wait of their own: up to 16 rows of depth 4096.
    const int64_t row_bytes = static_cast<int64_t>(bt) * p.slabs * kSlabDepth;
    if (row_bytes <= 16 * kThreads * 4) return LaunchSized<EPI, false, VARIANT, 1>(p, batch0, bt, stream);
    if (row_bytes <= 16 * kThreads * 8) return LaunchSized<EPI, false, VARIANT, 2>(p, batch0, bt, stream);
    return LaunchSized<EPI, false, VARIANT, 4>(p, batch0, bt, stream);
  }
  // Deep rows stay in registers through the prologue too, as long as rows x depth fits 16
  // pieces per thread: a row that does not is read twice, with the weight loads behind the
  // first pass instead of under it (2048 x 16384, B = 1: 15.6 us that way, 11.8 us from
  // registers).
  const int depth = p.a.depth;
  if (bt <= 1) {
    if (depth > 8192 && depth <= 16384) return LaunchSized<EPI, FUSED, VARIANT, 1, 16>(p, batch0, bt, stream);
    if (depth > 4096 && depth <= 8192) return LaunchSized<EPI, FUSED, VARIANT, 1, 8>(p, batch0, bt, stream);
    return LaunchSized<EPI, FUSED, VARIANT, 1>(p, batch0, bt, stream);
  }
  if (bt <= 2) {
    if (depth > 4096 && depth <= 8192) return LaunchSized<EPI, FUSED, VARIANT, 2, 8>(p, batch0, bt, stream);
    return LaunchSized<EPI, FUSED, VARIANT, 2>(p, batch0, bt, stream);
  }
  return LaunchSized<EPI, FUSED, VARIANT, 4>(p, batch0, bt, stream);
}

template <Int8Epilogue EPI, bool FUSED>
hipError_t LaunchVariant(const PackedArgs& p, int variant, int batch0, int bt,
                         hipStream_t stream) {
  if (!FUSED) return LaunchOne<EPI, false, LRTFC_QUANT_PORTABLE>(p, batch0, bt, stream);
  switch (variant) {
    case LRTFC_QUANT_NEON_V8:
      return LaunchOne<EPI, FUSED, LRTFC_QUANT_NEON_V8>(p, batch0, bt, stream);
    case LRTFC_QUANT_NEON_LEGACY:
      return LaunchOne<EPI, FUSED, LRTFC_QUANT_NEON_LEGACY>(p, batch0, bt, stream);
    default:
      return LaunchOne<EPI, FUSED, LRTFC_QUANT_PORTABLE>(p, batch0, bt, stream);
  }
}

}  // namespace

size_t PackedInt8FilterBytes(int out_depth, int depth) {
  const size_t tiles = (static_cast<size_t>(out_depth) + kTileRows - 1) / kTileRows;
  const size_t slabs = (static_cast<size_t>(depth) + kSlabDepth - 1) / kSlabDepth;
  return tiles * slabs * 1024;
}

hipError_t LaunchPackInt8Filter(const int8_t* filter, int out_depth, int depth, int8_t* packed,
                                hipStream_t stream) {
  if (out_depth == 0 || depth == 0) return hipSuccess;
  const int slabs = (depth + kSlabDepth - 1) / kSlabDepth;
  const int64_t chunks = static_cast<int64_t>(PackedInt8FilterBytes(out_depth, depth) / 16);
  const unsigned grid = static_cast<unsigned>((chunks + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(PackInt8FilterKernel, dim3(grid), dim3(kThreads), 0, stream, filter,
                     out_depth, depth, slabs, chunks, packed);
  return hipGetLastError();
}

int FcInt8PackedGemvFusedMaxRows(int depth) {
  // Eight rows where a wavefront can hold a whole row (the register-resident form: one wavefront
  // of eight per row); four on deeper rows, which every wavefront of a workgroup quantizes.
  return (depth % 4 == 0 && depth <= kFusedRowMaxDepth) ? kFusedMaxRows : 4;
}

bool FcInt8PackedGemvTakesRowsInOnePass(const FcInt8Args& a) {
  if (a.batches <= 16) return FcInt8PackedGemvSupports(a);
  if (!FcInt8PackedGemvSupports(a)) return false;
  if (a.batches > 32) return FcInt8RowsGemvTakes(a);
  PackedArgs p;
  p.a = a;
  p.slabs = (a.depth + kSlabDepth - 1) / kSlabDepth;
  return ResidentTwoRowTilesFit(p, a.batches, nullptr);
}

bool FcInt8PackedGemvSupports(const FcInt8Args& a) {
  // The per-tensor form with a non-zero filter zero point needs sum(x), which this
  // kernel does not carry; the row-major GEMV handles it.
  const size_t qstride = (static_cast<size_t>(a.depth) + kSlabDepth - 1) / kSlabDepth * kSlabDepth +
                         kQPad;
  return a.filter_offset == 0 && a.depth > 0 && SharedBytes(1, static_cast<int>(qstride)) <= 150 * 1024;
}

hipError_t LaunchFcInt8PackedGemv(const FcInt8Args& a, Int8Epilogue epilogue,
                                  const float* input_f32, int asymmetric, int variant,
                                  hipStream_t stream) {
  if (a.batches == 0 || a.out_depth == 0) return hipSuccess;
  if (!FcInt8PackedGemvSupports(a)) return hipErrorNotSupported;
  if (!input_f32 && a.batches > 32 && FcInt8RowsGemvTakes(a)) {
    return LaunchFcInt8RowsGemv(a, epilogue, stream);
  }
  PackedArgs p;
  p.a = a;
  p.input_f32 = input_f32;
  p.asymmetric = asymmetric;
  p.slabs = (a.depth + kSlabDepth - 1) / kSlabDepth;
  const int qstride = p.slabs * kSlabDepth + kQPad;
  int batch0 = 0;
  while (batch0 < a.batches) {
    int bt = min(16, a.batches - batch0);
    if (!input_f32 && ResidentTwoRowTilesFit(p, a.batches - batch0, nullptr)) {
      bt = a.batches - batch0;  // 17 to 32 rows in one pass
    }
    while (bt > 1 && bt <= 16 && SharedBytes(bt, qstride) > 150 * 1024) --bt;
    hipError_t err;
    if (epilogue == Int8Epilogue::kRequantize) {
      err = LaunchVariant<Int8Epilogue::kRequantize, false>(p, variant, batch0, bt, stream);
    } else if (epilogue == Int8Epilogue::kHybrid4Bit) {
      err = LaunchVariant<Int8Epilogue::kHybrid4Bit, false>(p, variant, batch0, bt, stream);
    } else if (input_f32) {
      err = LaunchVariant<Int8Epilogue::kHybrid, true>(p, variant, batch0, bt, stream);
    } else {
      err = LaunchVariant<Int8Epilogue::kHybrid, false>(p, variant, batch0, bt, stream);
    }
    if (err != hipSuccess) return err;
    batch0 += bt;
  }
  return hipSuccess;
}

}  // namespace lrtfc

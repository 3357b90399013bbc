// EMBEDDING_LOOKUP from quantized tables to floats on gfx950: the op that produces the first
// activation row of a decoder from a token id. Replaces EvalBlockwise (Int4 table with fp16
// block scales, tflite/kernels/embedding_lookup.cc:194-307) and EvalHybrid (Int8 / Int4 table
// with one scale or one per row, :309-395).
//
// The work is a gather: each looked-up row is read once (cols / 2 or cols bytes plus its
// scales) and written once as floats, so the kernel is bound by the output stream in HBM. A
// thread converts 8 consecutive columns: one 4-byte (Int4) or 8-byte (Int8) load, 8 products,
// one or two 16-byte stores; a wavefront covers 512 consecutive columns of one row, so loads
// and stores are contiguous per wavefront. Shapes whose rows or blocks are not multiples of 8
// columns take a narrow form (2 columns per thread for Int4, 1 for Int8).
//
// Arithmetic, as Unpack4Bit (:140-159) and the Int8 loop (:337-347) do it: an Int4 value is moved
// to the top of an int8 (16 x its signed value) and multiplied by scale / 16, an Int8 value
// is multiplied by the scale; one float32 product per element, converted to binary16 (round to
// nearest even, as tflite::half does) for a Float16 output. scale / 16 is computed as
// scale * 0.0625f, which is the same correctly rounded value because 1/16 is a power of two.
//
// Indices outside [0, rows) make the reference fail at the first such lookup (:280-286,
// :365-371). Here the first workgroup scans the lookup vector and records the first offending
// position in `status` (three device int32: {0 or 1, position or -1, the index found there or
// 0}), rewritten in full by every launch; rows with such an index are not written.
#include "kernels.h"

namespace lrtfc {
namespace {

constexpr int kThreads = 256;
// From this many looked-up rows on, float32 rows leave in contiguous kilobytes per store
// instruction (256000 x 2048 Int4 table: 2048 rows 6.7 -> 5.9 us; one row 2.2 us on the short
// kernel, 2.5 us on this one).
constexpr int kRunsMinRows = 32;

struct LookupArgs {
  const int32_t* lookup;
  const uint8_t* table;
  const uint16_t* block_scales;  // blockwise: [rows, cols / blocksize] binary16; else nullptr
  const float* row_scales;       // hybrid: [rows] or nullptr
  float scale;                   // hybrid without row_scales
  void* output;
  int32_t* status;
  int count, rows, cols, blocksize;
  int chunks;  // thread groups of kThreads per row
};

template <bool F16>
__device__ __forceinline__ void Store8(void* output, size_t index, const float (&v)[8]) {
  if constexpr (F16) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      w[i] = static_cast<uint32_t>(__half_as_ushort(__float2half_rn(v[2 * i]))) |
             static_cast<uint32_t>(__half_as_ushort(__float2half_rn(v[2 * i + 1]))) << 16;
    }
    *reinterpret_cast<uint4*>(static_cast<uint16_t*>(output) + index) =
        make_uint4(w[0], w[1], w[2], w[3]);
  } else {
    float4* dst = reinterpret_cast<float4*>(static_cast<float*>(output) + index);
    dst[0] = make_float4(v[0], v[1], v[2], v[3]);
    dst[1] = make_float4(v[4], v[5], v[6], v[7]);
  }
}

template <bool F16>
__device__ __forceinline__ void Store1(void* output, size_t index, float v) {
  if constexpr (F16) {
    static_cast<uint16_t*>(output)[index] = __half_as_ushort(__float2half_rn(v));
  } else {
    static_cast<float*>(output)[index] = v;
  }
}

// Signed value of nibble i of `word`, times 16: what (int8)(byte << 4) and (int8)(byte & 0xF0)
// hold in Unpack4Bit.
__device__ __forceinline__ float Nibble16(uint32_t word, int i) {
  return static_cast<float>((static_cast<int32_t>(word << (28 - 4 * i)) >> 28) * 16);
}

__device__ __forceinline__ void ScanLookups(const LookupArgs& a) {
  __shared__ int first_bad;
  if (threadIdx.x == 0) first_bad = 0x7FFFFFFF;
  __syncthreads();
  int mine = 0x7FFFFFFF;
  for (int i = threadIdx.x; i < a.count; i += kThreads) {
    const int32_t idx = a.lookup[i];
    if ((idx < 0 || idx >= a.rows) && i < mine) mine = i;
  }
  if (mine != 0x7FFFFFFF) atomicMin(&first_bad, mine);
  __syncthreads();
  if (threadIdx.x == 0) {
    const bool bad = first_bad != 0x7FFFFFFF;
    a.status[0] = bad ? 1 : 0;
    a.status[1] = bad ? first_bad : -1;
    a.status[2] = bad ? a.lookup[first_bad] : 0;
  }
}

// BITS: 4 or 8. WIDE: 8 columns per thread, else 2 (Int4) or 1 (Int8).
// RUNS: the float32 form for many rows (see below); few rows are latency and keep the short kernel.
template <int BITS, bool F16, bool WIDE, bool RUNS = false>
__global__ __launch_bounds__(kThreads) void EmbeddingLookupKernel(LookupArgs a) {
  if (blockIdx.x == 0 && a.status != nullptr) ScanLookups(a);
  const int row = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x - row * a.chunks;
  const int32_t idx = a.lookup[row];
  if (idx < 0 || idx >= a.rows) return;
  constexpr int kCols = WIDE ? 8 : (BITS == 4 ? 2 : 1);
  if constexpr (WIDE && !F16 && RUNS) {
    // float32 rows: a wavefront covers 512 columns as two runs of 256, lane L with columns
    // 4 L .. 4 L + 3 of each, so that every store instruction writes one contiguous kilobyte
    // (eight whole cache lines). With a thread's eight columns side by side, each of its two
    // stores would touch every line of two kilobytes by half.
    const int lane = static_cast<int>(threadIdx.x) & 63;
    const int wave_base = (chunk * kThreads + (static_cast<int>(threadIdx.x) & ~63)) * kCols;
    // Both runs' loads stand in one basic block (addresses clamped into the row, not tested):
    // with a test between them the second run's loads wait for the first run's store.
    int col[2];
    uint32_t word[2];
    float scale[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      col[half] = wave_base + half * 256 + lane * 4;
      const int at = min(col[half], a.cols - 4);
      const size_t element = static_cast<size_t>(idx) * a.cols + at;
      if (a.block_scales != nullptr) {
        const size_t blocks_per_row = static_cast<size_t>(a.cols / a.blocksize);
        scale[half] =
            HalfBitsToFloatFast(a.block_scales[idx * blocks_per_row + at / a.blocksize]);
      } else {
        scale[half] = a.row_scales != nullptr ? a.row_scales[idx] : a.scale;
      }
      if constexpr (BITS == 4) {
        word[half] = *reinterpret_cast<const uint16_t*>(a.table + element / 2);
      } else {
        word[half] = *reinterpret_cast<const uint32_t*>(a.table + element);
      }
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      float4 v;
      if constexpr (BITS == 4) {
        const float scale0 = scale[half] * 0.0625f;
        v = make_float4(Nibble16(word[half], 0) * scale0, Nibble16(word[half], 1) * scale0,
                        Nibble16(word[half], 2) * scale0, Nibble16(word[half], 3) * scale0);
      } else {
        const float sc = scale[half];
        v = make_float4(static_cast<float>(static_cast<int32_t>(word[half] << 24) >> 24) * sc,
                        static_cast<float>(static_cast<int32_t>(word[half] << 16) >> 24) * sc,
                        static_cast<float>(static_cast<int32_t>(word[half] << 8) >> 24) * sc,
                        static_cast<float>(static_cast<int32_t>(word[half]) >> 24) * sc);
      }
      if (col[half] < a.cols) {
        *reinterpret_cast<float4*>(static_cast<float*>(a.output) +
                                   static_cast<size_t>(row) * a.cols + col[half]) = v;
      }
    }
    return;
  }
  const int col = (chunk * kThreads + static_cast<int>(threadIdx.x)) * kCols;
  if (col >= a.cols) return;
  const size_t element = static_cast<size_t>(idx) * a.cols + col;
  float scale;
  if (a.block_scales != nullptr) {
    const size_t blocks_per_row = static_cast<size_t>(a.cols / a.blocksize);
    scale = HalfBitsToFloatFast(a.block_scales[idx * blocks_per_row + col / a.blocksize]);
  } else {
    scale = a.row_scales != nullptr ? a.row_scales[idx] : a.scale;
  }
  const size_t out_index = static_cast<size_t>(row) * a.cols + col;
  if constexpr (BITS == 4) {
    const float scale0 = scale * 0.0625f;
    if constexpr (WIDE) {
      const uint32_t word = *reinterpret_cast<const uint32_t*>(a.table + element / 2);
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = Nibble16(word, i) * scale0;
      Store8<F16>(a.output, out_index, v);
    } else {
      const uint32_t byte = a.table[element / 2];
      Store1<F16>(a.output, out_index, Nibble16(byte, 0) * scale0);
      Store1<F16>(a.output, out_index + 1, Nibble16(byte, 1) * scale0);
    }
  } else {
    const int8_t* values = reinterpret_cast<const int8_t*>(a.table) + element;
    if constexpr (WIDE) {
      const uint2 words = *reinterpret_cast<const uint2*>(values);
      float v[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = static_cast<float>(static_cast<int32_t>(words.x << (24 - 8 * i)) >> 24) * scale;
        v[4 + i] = static_cast<float>(static_cast<int32_t>(words.y << (24 - 8 * i)) >> 24) * scale;
      }
      Store8<F16>(a.output, out_index, v);
    } else {
      Store1<F16>(a.output, out_index, static_cast<float>(*values) * scale);
    }
  }
}

template <int BITS, bool F16>
hipError_t LaunchTyped(LookupArgs a, bool wide, hipStream_t stream) {
  const int per_thread = wide ? 8 : (BITS == 4 ? 2 : 1);
  const int threads_per_row = (a.cols + per_thread - 1) / per_thread;
  a.chunks = (threads_per_row + kThreads - 1) / kThreads;
  const int64_t blocks = static_cast<int64_t>(a.chunks) * a.count;
  if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
  if (wide && !F16 && a.count >= kRunsMinRows) {
    EmbeddingLookupKernel<BITS, F16, true, true>
        <<<static_cast<unsigned>(blocks), kThreads, 0, stream>>>(a);
  } else if (wide) {
    EmbeddingLookupKernel<BITS, F16, true><<<static_cast<unsigned>(blocks), kThreads, 0, stream>>>(a);
  } else {
    EmbeddingLookupKernel<BITS, F16, false><<<static_cast<unsigned>(blocks), kThreads, 0, stream>>>(a);
  }
  return hipGetLastError();
}

__global__ void LookupStatusOnlyKernel(LookupArgs a) { ScanLookups(a); }

}  // namespace

hipError_t LaunchEmbeddingLookup(const int32_t* lookup, int count, const void* table,
                                 int value_bits, int rows, int cols, const uint16_t* block_scales,
                                 int blocksize, const float* row_scales, float scale, int out_f16,
                                 void* output, int32_t* status, hipStream_t stream) {
  LookupArgs a{};
  a.lookup = lookup;
  a.table = static_cast<const uint8_t*>(table);
  a.block_scales = block_scales;
  a.row_scales = row_scales;
  a.scale = scale;
  a.output = output;
  a.status = status;
  a.count = count;
  a.rows = rows;
  a.cols = cols;
  a.blocksize = block_scales ? blocksize : cols;
  if (count == 0 || cols == 0) {
    // nothing to gather; the status words are still rewritten
    if (status == nullptr) return hipSuccess;
    LookupStatusOnlyKernel<<<1, kThreads, 0, stream>>>(a);
    return hipGetLastError();
  }
  // 8 columns per thread need rows, blocks and the buffers themselves aligned to 8 columns.
  const bool wide = cols % 8 == 0 && a.blocksize % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(table) % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(output) % 16 == 0;
  if (value_bits == 4) {
    return out_f16 ? LaunchTyped<4, true>(a, wide, stream) : LaunchTyped<4, false>(a, wide, stream);
  }
  return out_f16 ? LaunchTyped<8, true>(a, wide, stream) : LaunchTyped<8, false>(a, wide, stream);
}

}  // namespace lrtfc

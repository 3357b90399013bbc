// TEST INFRASTRUCTURE, x86 only: the hybrid row x vector product as the reference's OPTIMIZED
// x86 build runs it -- the SSE branch of SseMatrixBatchVectorMultiplyAccumulateImpl
// (tflite/kernels/internal/optimized/sse_tensor_utils.cc:308-379), which is what
// Register_FULLY_CONNECTED() reaches on a default -msse4.x Linux build and which, like the
// reference, runs on one thread (dense hybrid FC never uses the thread pool,
// fully_connected.cc:847-851). It exists as the second tier of the CPU baseline; the product
// never calls it. Results are those of the portable kernel bit for bit: the integer dot is
// exact in any order and the float tail is the same two operations
// (tests/test_oracle_kat.py::test_sse_dot_is_bit_identical_to_portable).
//
// Domain: weights in [-127, 127], as symmetric weight quantization produces them; at -128 the
// sign transfer onto the weight wraps (in the reference's kernel too).
//
// The idiom is the one the reference uses (|a| as the unsigned operand of pmaddubsw, the
// sign of a moved onto b, then pmaddwd with ones); the loop structure here is this file's own:
// two 16-byte blocks per turn on two accumulators, one horizontal add at the end, a scalar
// tail for the last < 16 columns.
#include "oracle.h"

#if defined(__x86_64__) || defined(__i386__)
#include <smmintrin.h>
#include <tmmintrin.h>

namespace {
inline __m128i Dot16(__m128i vec, __m128i row) {
  const __m128i row_signed = _mm_sign_epi8(row, vec);  // row * sign(vec)
  const __m128i vec_abs = _mm_abs_epi8(vec);           // -128 stays 0x80 = 128 unsigned
  const __m128i pairs = _mm_maddubs_epi16(vec_abs, row_signed);
  return _mm_madd_epi16(pairs, _mm_set1_epi16(1));
}
}  // namespace

extern "C" int orc_have_sse(void) { return 1; }

extern "C" void orc_matrix_batch_vector_multiply_accumulate_sse(
    const int8_t* matrix, int m_rows, int m_cols, const int8_t* vectors,
    const float* scaling_factors, int n_batch, float* result, const float* per_channel_scale,
    const int32_t* input_offset, const int32_t* row_sums) {
  const int vec_cols = m_cols & ~31;
  for (int b = 0; b < n_batch; ++b) {
    const int8_t* vec = vectors + static_cast<size_t>(b) * m_cols;
    const float batch_scale = scaling_factors[b];
    const int32_t batch_offset = input_offset ? input_offset[b] : 0;
    for (int r = 0; r < m_rows; ++r) {
      const int8_t* row = matrix + static_cast<size_t>(r) * m_cols;
      __m128i acc0 = _mm_setzero_si128(), acc1 = _mm_setzero_si128();
      int c = 0;
      for (; c < vec_cols; c += 32) {
        acc0 = _mm_add_epi32(
            acc0, Dot16(_mm_loadu_si128(reinterpret_cast<const __m128i*>(vec + c)),
                        _mm_loadu_si128(reinterpret_cast<const __m128i*>(row + c))));
        acc1 = _mm_add_epi32(
            acc1, Dot16(_mm_loadu_si128(reinterpret_cast<const __m128i*>(vec + c + 16)),
                        _mm_loadu_si128(reinterpret_cast<const __m128i*>(row + c + 16))));
      }
      if (c + 16 <= m_cols) {
        acc0 = _mm_add_epi32(
            acc0, Dot16(_mm_loadu_si128(reinterpret_cast<const __m128i*>(vec + c)),
                        _mm_loadu_si128(reinterpret_cast<const __m128i*>(row + c))));
        c += 16;
      }
      __m128i acc = _mm_add_epi32(acc0, acc1);
      acc = _mm_hadd_epi32(acc, acc);
      acc = _mm_hadd_epi32(acc, acc);
      int32_t dot = _mm_cvtsi128_si32(acc);
      for (; c < m_cols; ++c) dot += row[c] * vec[c];
      // sse_tensor_utils.cc:319-324, 369-373: the offset term only when both are non-zero.
      if (row_sums && batch_offset) dot -= batch_offset * row_sums[r];
      const float row_scale =
          per_channel_scale ? per_channel_scale[r] * batch_scale : batch_scale;
      result[static_cast<size_t>(b) * m_rows + r] += static_cast<float>(dot) * row_scale;
    }
  }
}
#else
extern "C" int orc_have_sse(void) { return 0; }
extern "C" void orc_matrix_batch_vector_multiply_accumulate_sse(
    const int8_t*, int, int, const int8_t*, const float*, int, float*, const float*,
    const int32_t*, const int32_t*) {}
#endif

// Measurement aids, not part of the op. First: a kernel that only streams `bytes` bytes out of device
// memory, with the access pattern of the decode kernels (every wavefront walks its own
// contiguous 32 KiB run through a ring of sixteen outstanding non-temporal 1 KiB loads) and
// nothing else to do. Timed beside a GEMV on the same bytes it tells how much of that kernel's
// time is the memory system's and how much is the kernel's own (prologue, epilogue, tail).
//
// Second: a kernel that only issues v_mfma_i32_32x32x32_i8 on register operands, one wavefront
// per SIMD as in the prefill GEMM, eight independent accumulators so that the instructions go
// back to back. Launched for a few hundred milliseconds it shows the int8 rate this part's
// matrix cores sustain under its power limit, for operands that toggle like random data and
// for constant ones: the ceiling of the GEMM's main loop, with no operand traffic at all.
#include "kernels.h"

namespace lrtfc {
namespace {

using i32x16 = int __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t MixBits(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

constexpr int kProbeAccumulators = 8;

__global__ __launch_bounds__(256) void MfmaRateKernel(int iterations, int random_operands,
                                                      int32_t* sink) {
  const uint32_t id = blockIdx.x * 256 + threadIdx.x;
  i32x4 a[4], b[4];
  for (int i = 0; i < 4; ++i) {
    for (int e = 0; e < 4; ++e) {
      a[i][e] = random_operands ? static_cast<int>(MixBits(id * 64 + i * 8 + e)) : 0x05050505;
      b[i][e] = random_operands ? static_cast<int>(MixBits(id * 64 + i * 8 + e + 4)) : 0x03030303;
    }
  }
  i32x16 acc[kProbeAccumulators];
  for (int i = 0; i < kProbeAccumulators; ++i) {
    for (int e = 0; e < 16; ++e) acc[i][e] = 0;
  }
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int i = 0; i < kProbeAccumulators; ++i) {
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[(i + (i >> 2)) & 3], acc[i], 0, 0, 0);
    }
  }
  int32_t r = 0;
  for (int i = 0; i < kProbeAccumulators; ++i) {
    for (int e = 0; e < 16; ++e) r ^= acc[i][e];
  }
  sink[id] = r;
}

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWaveSize;
constexpr int kRing = 16;
constexpr int kRunVecs = 2048;  // 16-byte pieces per wavefront: 32 KiB

__global__ __launch_bounds__(kThreads) void StreamReadKernel(const i32x4* __restrict__ src,
                                                             size_t vecs, int32_t* sink) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const size_t wave = static_cast<size_t>(blockIdx.x) * kWaves + threadIdx.x / kWaveSize;
  const size_t begin = wave * kRunVecs;
  if (begin >= vecs) return;
  const size_t last = vecs - 1;
  const i32x4* base = src + begin + lane;
  const int steps = static_cast<int>(min(static_cast<size_t>(kRunVecs), vecs - begin) / kWaveSize);
  auto at = [&](int s) {
    return __builtin_nontemporal_load(
        src + min(begin + static_cast<size_t>(min(s, max(steps, 1) - 1)) * kWaveSize + lane, last));
  };
  (void)base;
  i32x4 ring[kRing];
#pragma unroll
  for (int u = 0; u < kRing; ++u) ring[u] = at(u);
  i32x4 acc = {0, 0, 0, 0};
  int s0 = 0;
  for (; s0 + kRing < steps; s0 += kRing) {
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
      acc ^= ring[u];
      ring[u] = at(s0 + kRing + u);
    }
  }
#pragma unroll
  for (int u = 0; u < kRing; ++u) acc ^= ring[u];
  // Keeps the loads alive; the comparison practically never holds.
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5EED1234 && sink) sink[0] = 1;
}

}  // namespace

hipError_t LaunchStreamRead(const void* src, size_t bytes, int32_t* sink, hipStream_t stream) {
  const size_t vecs = bytes / 16;
  if (vecs == 0) return hipSuccess;
  const size_t waves = (vecs + kRunVecs - 1) / kRunVecs;
  const unsigned grid = static_cast<unsigned>((waves + kWaves - 1) / kWaves);
  hipLaunchKernelGGL(StreamReadKernel, dim3(grid), dim3(kThreads), 0, stream,
                     static_cast<const i32x4*>(src), vecs, sink);
  return hipGetLastError();
}


hipError_t LaunchMfmaRate(int workgroups, int iterations, int random_operands, int32_t* sink,
                          hipStream_t stream) {
  hipLaunchKernelGGL(MfmaRateKernel, dim3(workgroups), dim3(256), 0, stream, iterations,
                     random_operands, sink);
  return hipGetLastError();
}

double MfmaRateOpsPerLaunch(int workgroups, int iterations) {
  return 65536.0 * kProbeAccumulators * iterations * 4.0 * workgroups;
}

}  // namespace lrtfc

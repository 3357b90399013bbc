// Measurement aids of the benchmark, not part of the op and not part of the kernel library: this
// file builds into its own shared library (liblitert_amd_bench_probes.so) with its own header
// (bench_probes.h beside it). First: a kernel that only streams `bytes` bytes out of device
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
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "bench_probes.h"

namespace {

constexpr int kWaveSize = 64;
using i32x4 = int __attribute__((ext_vector_type(4)));

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

thread_local char g_last_error[256] = "";

int Fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
  va_end(ap);
  return status;
}

int FromHip(hipError_t err, const char* what) {
  if (err == hipSuccess) return LRTPROBE_OK;
  return Fail(LRTPROBE_HIP_ERROR, "%s: %s", what, hipGetErrorString(err));
}

// One launch may hold at most this many MFMAs per wavefront-slot of the chip: about 0.1 s on a
// 256-CU part. Sustained measurements launch back to back instead of launching longer.
constexpr double kMaxMfmaPerLaunch = 256.0 * 4 * 2.0e6;

}  // namespace

extern "C" {

const char* lrtprobe_last_error(void) { return g_last_error; }

int lrtprobe_stream_read(const void* src, size_t bytes, int32_t* sink, void* stream) {
  if (bytes < 16) return LRTPROBE_OK;
  if (!src) return Fail(LRTPROBE_INVALID_ARGUMENT, "null pointer");
  if ((reinterpret_cast<uintptr_t>(src) & 15) != 0) {
    return Fail(LRTPROBE_INVALID_ARGUMENT, "src must be 16-byte aligned");
  }
  const size_t vecs = bytes / 16;
  const size_t waves = (vecs + kRunVecs - 1) / kRunVecs;
  const unsigned grid = static_cast<unsigned>((waves + kWaves - 1) / kWaves);
  hipLaunchKernelGGL(StreamReadKernel, dim3(grid), dim3(kThreads), 0,
                     reinterpret_cast<hipStream_t>(stream), static_cast<const i32x4*>(src), vecs,
                     sink);
  return FromHip(hipGetLastError(), "stream read probe");
}

int lrtprobe_mfma_rate(int workgroups, int iterations, int random_operands, int32_t* sink,
                       double* ops_per_launch, void* stream) {
  if (!sink) return Fail(LRTPROBE_INVALID_ARGUMENT, "null pointer");
  if (workgroups < 1 || workgroups > 65536 || iterations < 1) {
    return Fail(LRTPROBE_INVALID_ARGUMENT,
                "workgroups %d (1..65536) or iterations %d (>= 1) out of range", workgroups,
                iterations);
  }
  const double mfmas = 4.0 * kProbeAccumulators * static_cast<double>(iterations) * workgroups;
  if (mfmas > kMaxMfmaPerLaunch) {
    return Fail(LRTPROBE_INVALID_ARGUMENT,
                "workgroups %d x iterations %d is more than one launch may hold (about 0.1 s of "
                "matrix-core time); launch back to back for longer measurements",
                workgroups, iterations);
  }
  if (ops_per_launch) *ops_per_launch = 65536.0 * mfmas;
  hipLaunchKernelGGL(MfmaRateKernel, dim3(workgroups), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), iterations, random_operands, sink);
  return FromHip(hipGetLastError(), "matrix-core rate probe");
}

}  // extern "C"

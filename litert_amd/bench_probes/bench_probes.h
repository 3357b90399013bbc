/* Measurement aids of bench.py. NOT part of the op's boundary: nothing here has a counterpart
 * in the reference, nothing here is called by the kernel library or the delegate, and the
 * library this header describes (liblitert_amd_bench_probes.so) is loaded by the benchmark and
 * its own test only. Plain C ABI: device pointers, sizes, a `void*` HIP stream. */
#ifndef LITERT_AMD_BENCH_PROBES_H_
#define LITERT_AMD_BENCH_PROBES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { LRTPROBE_OK = 0, LRTPROBE_INVALID_ARGUMENT = 1, LRTPROBE_HIP_ERROR = 3 };

/* Message of the calling thread's last failed call. */
const char* lrtprobe_last_error(void);

/* A launch that does nothing but read `bytes` bytes (whole 16-byte pieces; src 16-byte aligned)
 * from device memory with the decode kernels' access pattern: every wavefront walks its own
 * contiguous 32 KiB run through a ring of sixteen outstanding non-temporal 1 KiB loads. Timed
 * on the same bytes as a GEMV it shows what the memory system alone needs for a launch of that
 * size. `sink` (device int32, may be NULL) is practically never written. */
int lrtprobe_stream_read(const void* src, size_t bytes, int32_t* sink, void* stream);

/* A launch of `workgroups` x 4 wavefronts (one per SIMD of a CU, as in the prefill GEMM) that
 * do nothing but issue 8 x `iterations` v_mfma_i32_32x32x32_i8 each on register operands --
 * pseudo-random bit patterns (random_operands != 0) or constants. Launched back to back for
 * some hundred milliseconds it gives the int8 rate the matrix cores sustain under the part's
 * power limit, with no operand traffic at all. One launch is limited to about 0.1 s of
 * matrix-core time (workgroups x iterations <= 64,000,000); larger requests are refused.
 * `sink` (device) receives workgroups x 256 int32; *ops_per_launch (host, may be NULL) the
 * integer operations (2 per multiply-add) of one launch. */
int lrtprobe_mfma_rate(int workgroups, int iterations, int random_operands, int32_t* sink,
                       double* ops_per_launch, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LITERT_AMD_BENCH_PROBES_H_ */

// C-ABI layer of the gfx950 FULLY_CONNECTED kernels: argument checking, the
// Prepare-time host math, and dispatch to the kernel launchers.
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <map>
#include <mutex>
#include <utility>

#include "kernels.h"

namespace {

thread_local char g_last_error[512] = "";

int Fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
  va_end(ap);
  return status;
}

int FromHip(hipError_t err, const char* what) {
  if (err == hipSuccess) return LRTFC_OK;
  if (err == hipErrorNotSupported) return Fail(LRTFC_UNSUPPORTED, "%s: not supported", what);
  return Fail(LRTFC_HIP_ERROR, "%s: %s", what, hipGetErrorString(err));
}

hipStream_t AsStream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Process-wide state, shared by every interpreter and thread that uses the library: whether a
// gfx950 device has been found, and the per-device scratch addresses below. Written under
// g_init_mutex by lrtfc_init, read without it by the compute entry points.
std::atomic<bool> g_initialised{false};
std::mutex g_init_mutex;

// Scratch of lrtfc_fc_hybrid_static_scratch, the entry point that allocates nothing: the
// activation workspace (quantized rows, scaling factors, zero points) that lrtfc_fc_hybrid
// takes as an argument lives in this array instead. Every device the library runs on holds
// its own copy at its own address until the process ends; in host code the array's name is
// only a handle for hipGetSymbolAddress, never a device address. lrtfc_init looks the address
// up once per device and the entry point passes that pointer to the kernels.
static __device__ __align__(256) unsigned char scratch[LRTFC_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices] = {};

int RequireInit() {
  if (g_initialised) return LRTFC_OK;
  return Fail(LRTFC_NO_DEVICE, "lrtfc_init() has not succeeded: no gfx950 device selected");
}

#define LRTFC_REQUIRE(cond, ...) \
  do {                           \
    if (!(cond)) return Fail(LRTFC_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

// Fused activations of the float-output paths: the clamps and the sign bit.
bool FloatActivationOk(int activation) {
  return (activation >= LRTFC_ACT_NONE && activation <= LRTFC_ACT_RELU6) ||
         activation == LRTFC_ACT_SIGN_BIT;
}

// Batches from this size on go to the MFMA GEMM when its tiling fits.
constexpr int kGemmMinBatches = 128;
// On the re-tiled filter: up to this many rows the GEMV wins always (16 rows per pass over the
// filter), and up to 32 rows where it can take them in one pass; beyond that the GEMM, which
// streams the filter once.
constexpr int kPackedGemmMinBatches = 16;

// Workspace layout for the hybrid paths (kernels.h).
using Workspace = lrtfc::ActivationWorkspace;
size_t WorkspaceBytes(int batches, int depth) {
  return lrtfc::ActivationWorkspaceBytes(batches, depth);
}
Workspace SplitWorkspace(void* base, int batches, int depth) {
  return lrtfc::SplitActivationWorkspace(base, batches, depth);
}

}  // namespace

namespace lrtfc {
hipError_t EnsureDynamicLds(const void* kernel, size_t bytes) {
  if (bytes <= 48 * 1024) return hipSuccess;
  int device = 0;
  if (hipError_t err = hipGetDevice(&device)) return err;
  static std::mutex mu;
  static std::map<std::pair<const void*, int>, size_t> granted;
  std::lock_guard<std::mutex> lock(mu);
  size_t& have = granted[std::make_pair(kernel, device)];
  if (bytes > have) {
    if (hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(bytes))) {
      return err;
    }
    have = bytes;
  }
  return hipSuccess;
}
}  // namespace lrtfc

extern "C" {

int lrtfc_abi_version(void) { return LRTFC_ABI_VERSION; }

const char* lrtfc_last_error(void) { return g_last_error; }

int lrtfc_init(int device_ordinal) {
  std::lock_guard<std::mutex> lock(g_init_mutex);
  int count = 0;
  hipError_t err = hipGetDeviceCount(&count);
  if (err != hipSuccess || count == 0) {
    g_initialised = false;
    return Fail(LRTFC_NO_DEVICE, "no HIP device visible (%s)",
                err == hipSuccess ? "device count is 0" : hipGetErrorString(err));
  }
  if (device_ordinal < 0 || device_ordinal >= count) {
    return Fail(LRTFC_INVALID_ARGUMENT, "device %d out of range (%d visible)", device_ordinal,
                count);
  }
  hipDeviceProp_t prop;
  err = hipGetDeviceProperties(&prop, device_ordinal);
  if (err != hipSuccess) return FromHip(err, "hipGetDeviceProperties");
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    // Another caller's successful init of a gfx950 device stands.
    return Fail(LRTFC_NO_DEVICE, "device %d is %s; this library is built for gfx950 only",
                device_ordinal, prop.gcnArchName);
  }
  err = hipSetDevice(device_ordinal);
  if (err != hipSuccess) return FromHip(err, "hipSetDevice");
  if (device_ordinal < kMaxDevices && g_scratch_ptr[device_ordinal].load() == nullptr) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return FromHip(err, "hipGetSymbolAddress(scratch)");
    g_scratch_ptr[device_ordinal] = ptr;
  }
  g_initialised = true;
  return LRTFC_OK;
}

// ---- Prepare-time math -------------------------------------------------------

int lrtfc_quantize_multiplier(double real_multiplier, int32_t* quantized_multiplier, int* shift) {
  LRTFC_REQUIRE(quantized_multiplier && shift, "null output pointer");
  if (real_multiplier == 0.) {
    *quantized_multiplier = 0;
    *shift = 0;
    return LRTFC_OK;
  }
  const double q = std::frexp(real_multiplier, shift);
  int64_t q_fixed = static_cast<int64_t>(std::round(q * 2147483648.0));
  LRTFC_REQUIRE(q_fixed <= (1ll << 31), "multiplier significand out of range");
  if (q_fixed == (1ll << 31)) {
    q_fixed /= 2;
    ++*shift;
  }
  if (*shift < -31) {  // would shift every bit out: flush to zero
    *shift = 0;
    q_fixed = 0;
  }
  *quantized_multiplier = static_cast<int32_t>(q_fixed);
  return LRTFC_OK;
}

int lrtfc_prepare_per_channel(float input_scale, const float* filter_scales, int num_channels,
                              float output_scale, int32_t* multipliers, int32_t* shifts) {
  LRTFC_REQUIRE(filter_scales && multipliers && shifts, "null pointer");
  LRTFC_REQUIRE(num_channels >= 0, "negative channel count");
  for (int i = 0; i < num_channels; ++i) {
    const double effective = static_cast<double>(input_scale) *
                             static_cast<double>(filter_scales[i]) /
                             static_cast<double>(output_scale);
    int s = 0;
    const int rc = lrtfc_quantize_multiplier(effective, &multipliers[i], &s);
    if (rc != LRTFC_OK) return rc;
    shifts[i] = s;
  }
  return LRTFC_OK;
}

int lrtfc_prepare_per_tensor(float input_scale, float filter_scale, int has_bias,
                             float bias_scale, float output_scale, int32_t* multiplier,
                             int32_t* shift) {
  LRTFC_REQUIRE(multiplier && shift, "null output pointer");
  if (has_bias) {
    const double product = static_cast<double>(input_scale) * static_cast<double>(filter_scale);
    const double diff = std::abs(product - static_cast<double>(bias_scale));
    LRTFC_REQUIRE(diff / static_cast<double>(output_scale) <= 0.02,
                  "bias scale differs from input_scale * filter_scale by more than 0.02 output "
                  "quanta");
  }
  // The product is formed in float before widening, as the reference does.
  const double product = static_cast<double>(input_scale * filter_scale);
  LRTFC_REQUIRE(product >= 0, "negative input_scale * filter_scale");
  int s = 0;
  const int rc =
      lrtfc_quantize_multiplier(product / static_cast<double>(output_scale), multiplier, &s);
  *shift = s;
  return rc;
}

int lrtfc_activation_range_int8(int activation, float output_scale, int32_t output_zero_point,
                                int32_t* act_min, int32_t* act_max) {
  LRTFC_REQUIRE(act_min && act_max, "null output pointer");
  const int32_t qmin = -128, qmax = 127;
  auto quantize = [&](float f, int32_t* q) {
    const float rounded = std::round(f / output_scale);
    if (!(rounded >= static_cast<float>(std::numeric_limits<int32_t>::min()) &&
          rounded <= static_cast<float>(std::numeric_limits<int32_t>::max()))) {
      return false;
    }
    *q = output_zero_point + static_cast<int32_t>(rounded);
    return true;
  };
  int32_t lo = qmin, hi = qmax, q = 0;
  bool ok = true;
  switch (activation) {
    case LRTFC_ACT_RELU:
      ok = quantize(0.0f, &q);
      lo = std::max(qmin, q);
      break;
    case LRTFC_ACT_RELU6:
      ok = quantize(0.0f, &q);
      lo = std::max(qmin, q);
      ok = ok && quantize(6.0f, &q);
      hi = std::min(qmax, q);
      break;
    case LRTFC_ACT_RELU_N1_TO_1:
      ok = quantize(-1.0f, &q);
      lo = std::max(qmin, q);
      ok = ok && quantize(1.0f, &q);
      hi = std::min(qmax, q);
      break;
    default:
      break;
  }
  LRTFC_REQUIRE(ok, "activation bound does not fit int32 at this output scale");
  *act_min = lo;
  *act_max = hi;
  return LRTFC_OK;
}

// ---- weight preparation ------------------------------------------------------

int lrtfc_row_sums_int8(const int8_t* filter, int out_depth, int depth, int32_t* row_sums,
                        void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(out_depth >= 0 && depth >= 0, "negative dimension");
  if (out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(filter && row_sums, "null pointer");
  return FromHip(lrtfc::LaunchRowSumsInt8(filter, out_depth, depth, row_sums, AsStream(stream)),
                 "row sums");
}

int lrtfc_unpack_int4(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                      void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(num_elements >= 0, "negative element count");
  if (num_elements == 0) return LRTFC_OK;
  LRTFC_REQUIRE(packed && unpacked, "null pointer");
  LRTFC_REQUIRE((num_elements + 1) / 2 <= 0x7fffffffll * 256, "tensor too large");
  return FromHip(lrtfc::LaunchUnpackInt4(packed, num_elements, unpacked, AsStream(stream)),
                 "int4 unpack");
}

int lrtfc_xor_sign_bit(const uint8_t* src, uint8_t* dst, size_t bytes, void* stream) {
  if (int rc = RequireInit()) return rc;
  if (bytes == 0) return LRTFC_OK;
  LRTFC_REQUIRE(src && dst, "null pointer");
  return FromHip(lrtfc::LaunchXorSignBit(src, dst, bytes, AsStream(stream)), "sign bit flip");
}

int lrtfc_unpack_int2(const uint8_t* packed, int64_t num_elements, int8_t* unpacked,
                      void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(num_elements >= 0, "negative element count");
  if (num_elements == 0) return LRTFC_OK;
  LRTFC_REQUIRE(packed && unpacked, "null pointer");
  LRTFC_REQUIRE((num_elements + 3) / 4 <= 0x7fffffffll * 256, "tensor too large");
  return FromHip(lrtfc::LaunchUnpackInt2(packed, num_elements, unpacked, AsStream(stream)),
                 "int2 unpack");
}

int lrtfc_blockwise_int4_kfsum(const uint8_t* packed_filter, const uint16_t* scales_f16,
                               int out_depth, int depth, int blocksize, float* kfsum,
                               void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(out_depth >= 0 && depth >= 0, "negative dimension");
  LRTFC_REQUIRE(blocksize > 0 && depth % blocksize == 0, "blocksize %d does not divide depth %d",
                blocksize, depth);
  if (out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(packed_filter && scales_f16 && kfsum, "null pointer");
  return FromHip(lrtfc::LaunchBlockwiseInt4Kfsum(packed_filter, scales_f16, out_depth, depth,
                                                 blocksize, kfsum, AsStream(stream)),
                 "blockwise kfsum");
}

// ---- Eval --------------------------------------------------------------------

int lrtfc_fc_int8(const int8_t* input, const int8_t* filter, const int32_t* bias,
                  const int32_t* multipliers, const int32_t* shifts, int per_channel,
                  const int32_t* filter_row_sums, int8_t* output, int batches, int depth,
                  int out_depth, int32_t input_offset, int32_t filter_offset,
                  int32_t output_offset, int32_t act_min, int32_t act_max, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth >= 0 && out_depth >= 0, "negative dimension");
  // Empty output: nothing to do (tflite/kernels/fully_connected.cc:1966-1968).
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(output, "null output");
  if (depth == 0) {
    // filter.dims[1] == 0 zero-fills the output (fully_connected.cc:1970-1973).
    return FromHip(lrtfc::LaunchZeroFill(output, static_cast<size_t>(batches) * out_depth,
                                         AsStream(stream)),
                   "zero fill");
  }
  LRTFC_REQUIRE(input && filter && multipliers && shifts, "null pointer");
  LRTFC_REQUIRE(act_min <= act_max, "activation range is empty");
  LRTFC_REQUIRE(!(per_channel && filter_offset != 0),
                "per-channel filters are symmetric: filter_offset must be 0");
  LRTFC_REQUIRE(input_offset == 0 || filter_row_sums,
                "filter_row_sums is required when input_offset != 0");
  lrtfc::FcInt8Args a{};
  a.input = input;
  a.filter = filter;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.filter_row_sums = filter_row_sums;
  a.bias_i32 = bias;
  a.multipliers = multipliers;
  a.shifts = shifts;
  a.per_channel = per_channel;
  a.input_offset = input_offset;
  a.filter_offset = filter_offset;
  a.output_offset = output_offset;
  a.act_min = act_min;
  a.act_max = act_max;
  a.output_i8 = output;
  if (batches >= kGemmMinBatches && lrtfc::FcInt8GemmMfmaSupports(a)) {
    return FromHip(lrtfc::LaunchFcInt8GemmMfma(a, AsStream(stream)), "int8 MFMA GEMM");
  }
  return FromHip(
      lrtfc::LaunchFcInt8Gemv(a, lrtfc::Int8Epilogue::kRequantize, AsStream(stream)),
      "int8 GEMV");
}

int lrtfc_fc_int8_preferred_layout(int batches, int depth, int out_depth, int32_t filter_offset) {
  lrtfc::FcInt8Args a{};
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.filter_offset = filter_offset;
  (void)batches;  // the re-tiled form serves every batch size (GEMV up to 16 rows, GEMM above)
  return lrtfc::FcInt8PackedGemvSupports(a) ? LRTFC_LAYOUT_PACKED : LRTFC_LAYOUT_ROW_MAJOR;
}

int lrtfc_fc_hybrid_fused_max_batches(int depth, int out_depth) {
  (void)out_depth;
  return lrtfc::FcInt8PackedGemvFusedMaxRows(depth);
}

int lrtfc_fc_blockwise_int4_preferred_layout(int depth, int blocksize) {
  return lrtfc::FcInt4PackedSupports(depth, blocksize) ? LRTFC_LAYOUT_PACKED
                                                       : LRTFC_LAYOUT_ROW_MAJOR;
}

size_t lrtfc_packed_int8_filter_bytes(int out_depth, int depth) {
  if (out_depth <= 0 || depth <= 0) return 0;
  return lrtfc::PackedInt8FilterBytes(out_depth, depth);
}

int lrtfc_pack_int8_filter(const int8_t* filter, int out_depth, int depth, int8_t* packed,
                           void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(out_depth >= 0 && depth >= 0, "negative dimension");
  if (out_depth == 0 || depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(filter && packed, "null pointer");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(packed) & 15) == 0, "packed must be 16-byte aligned");
  return FromHip(lrtfc::LaunchPackInt8Filter(filter, out_depth, depth, packed, AsStream(stream)),
                 "pack int8 filter");
}

int lrtfc_fc_int8_packed(const int8_t* input, const int8_t* packed_filter, const int32_t* bias,
                         const int32_t* multipliers, const int32_t* shifts, int per_channel,
                         const int32_t* filter_row_sums, int8_t* output, int batches, int depth,
                         int out_depth, int32_t input_offset, int32_t output_offset,
                         int32_t act_min, int32_t act_max, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && packed_filter && multipliers && shifts && output, "null pointer");
  LRTFC_REQUIRE(act_min <= act_max, "activation range is empty");
  LRTFC_REQUIRE(input_offset == 0 || filter_row_sums,
                "filter_row_sums is required when input_offset != 0");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(packed_filter) & 15) == 0,
                "packed filter must be 16-byte aligned");
  lrtfc::FcInt8Args a{};
  a.input = input;
  a.filter = packed_filter;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.filter_row_sums = filter_row_sums;
  a.bias_i32 = bias;
  a.multipliers = multipliers;
  a.shifts = shifts;
  a.per_channel = per_channel;
  a.input_offset = input_offset;
  a.output_offset = output_offset;
  a.act_min = act_min;
  a.act_max = act_max;
  a.output_i8 = output;
  if (batches > kPackedGemmMinBatches && !lrtfc::FcInt8PackedGemvTakesRowsInOnePass(a) &&
      lrtfc::FcInt8PackedGemmSupports(a)) {
    return FromHip(lrtfc::LaunchFcInt8PackedGemm(a, lrtfc::Int8Epilogue::kRequantize,
                                                 AsStream(stream)),
                   "packed int8 GEMM");
  }
  return FromHip(lrtfc::LaunchFcInt8PackedGemv(a, lrtfc::Int8Epilogue::kRequantize, nullptr, 0, 0,
                                               AsStream(stream)),
                 "packed int8 GEMV");
}

int lrtfc_fc_hybrid_packed(const float* input, const int8_t* packed_filter,
                           const float* per_channel_scales, float filter_scale,
                           const int32_t* filter_row_sums, const float* bias, float* output,
                           int batches, int depth, int out_depth, int asymmetric_quantize_inputs,
                           int activation, int quant_variant, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && packed_filter && output, "null pointer");
  LRTFC_REQUIRE(!asymmetric_quantize_inputs || filter_row_sums,
                "filter_row_sums is required for asymmetric activation quantization");
  LRTFC_REQUIRE(FloatActivationOk(activation),
                "activation %d is not one of None/Relu/ReluN1To1/Relu6/SignBit", activation);
  LRTFC_REQUIRE(quant_variant >= 0 && quant_variant <= LRTFC_QUANT_NEON_LEGACY,
                "unknown quantizer variant");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(packed_filter) & 15) == 0,
                "packed filter must be 16-byte aligned");
  lrtfc::FcInt8Args a{};
  a.filter = packed_filter;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.filter_row_sums = filter_row_sums;
  a.per_channel_scales = per_channel_scales;
  a.filter_scale = filter_scale;
  a.bias_f32 = bias;
  a.activation = activation;
  a.output_f32 = output;
  return FromHip(lrtfc::LaunchFcInt8PackedGemv(a, lrtfc::Int8Epilogue::kHybrid, input,
                                               asymmetric_quantize_inputs, quant_variant,
                                               AsStream(stream)),
                 "packed hybrid GEMV");
}

namespace {
int FcHybridInt8Packed(const int8_t* quantized_input, const float* scaling_factors,
                       const int32_t* zero_points, const int8_t* packed_filter,
                       const float* per_channel_scales, float filter_scale,
                       const int32_t* filter_row_sums, const float* bias, float* output,
                       int batches, int depth, int out_depth, int activation, int zero_input_exit,
                       void* stream, int batch_matmul = 0) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(quantized_input && scaling_factors && packed_filter && output, "null pointer");
  LRTFC_REQUIRE(!zero_points || filter_row_sums,
                "filter_row_sums is required with activation zero points");
  LRTFC_REQUIRE(FloatActivationOk(activation),
                "activation %d is not one of None/Relu/ReluN1To1/Relu6/SignBit", activation);
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(packed_filter) & 15) == 0,
                "packed filter must be 16-byte aligned");
  lrtfc::FcInt8Args a{};
  a.input = quantized_input;
  a.filter = packed_filter;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.filter_row_sums = filter_row_sums;
  a.scaling_factors = scaling_factors;
  a.zero_points = zero_points;
  a.per_channel_scales = per_channel_scales;
  a.filter_scale = filter_scale;
  a.bias_f32 = bias;
  a.activation = activation;
  a.output_f32 = output;
  a.zero_input_exit = zero_input_exit;
  a.batch_matmul = batch_matmul;
  if (batches > kPackedGemmMinBatches && !lrtfc::FcInt8PackedGemvTakesRowsInOnePass(a) &&
      lrtfc::FcInt8PackedGemmSupports(a)) {
    return FromHip(lrtfc::LaunchFcInt8PackedGemm(a, lrtfc::Int8Epilogue::kHybrid,
                                                 AsStream(stream)),
                   "packed hybrid GEMM");
  }
  return FromHip(lrtfc::LaunchFcInt8PackedGemv(a, lrtfc::Int8Epilogue::kHybrid, nullptr, 0,
                                               LRTFC_QUANT_PORTABLE, AsStream(stream)),
                 "packed hybrid GEMV");
}
}  // namespace

int lrtfc_fc_hybrid_int8_packed(const int8_t* quantized_input, const float* scaling_factors,
                                const int32_t* zero_points, const int8_t* packed_filter,
                                const float* per_channel_scales, float filter_scale,
                                const int32_t* filter_row_sums, const float* bias, float* output,
                                int batches, int depth, int out_depth, int activation,
                                void* stream) {
  return FcHybridInt8Packed(quantized_input, scaling_factors, zero_points, packed_filter,
                            per_channel_scales, filter_scale, filter_row_sums, bias, output,
                            batches, depth, out_depth, activation, /*zero_input_exit=*/0, stream);
}

int lrtfc_fc_hybrid_packed_workspace(const float* input, const int8_t* packed_filter,
                                     const float* per_channel_scales, float filter_scale,
                                     const int32_t* filter_row_sums, const float* bias,
                                     float* output, int batches, int depth, int out_depth,
                                     int asymmetric_quantize_inputs, int activation,
                                     int quant_variant, void* workspace, size_t workspace_bytes,
                                     void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && workspace, "null pointer");
  LRTFC_REQUIRE(workspace_bytes >= WorkspaceBytes(batches, depth),
                "workspace too small: %zu < %zu bytes", workspace_bytes,
                WorkspaceBytes(batches, depth));
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  const Workspace w = SplitWorkspace(workspace, batches, depth);
  int rc = lrtfc_batch_quantize_floats(input, batches, depth, w.q, w.sf, w.zp,
                                       asymmetric_quantize_inputs, quant_variant, stream);
  if (rc != LRTFC_OK) return rc;
  return FcHybridInt8Packed(w.q, w.sf, asymmetric_quantize_inputs ? w.zp : nullptr, packed_filter,
                            per_channel_scales, filter_scale, filter_row_sums, bias, output,
                            batches, depth, out_depth, activation, /*zero_input_exit=*/1, stream);
}

namespace {
size_t TransposedBytes(int64_t lhs_matrices, int rows, int depth) {
  const size_t bytes = static_cast<size_t>(lhs_matrices) * rows * depth * sizeof(float);
  return (bytes + 255) & ~static_cast<size_t>(255);
}
}  // namespace

size_t lrtfc_batch_matmul_workspace_bytes(int lhs_matrices, int rows, int depth, int adj_x) {
  if (lhs_matrices <= 0 || rows <= 0 || depth <= 0) return 0;
  const int64_t quant_rows = static_cast<int64_t>(lhs_matrices) * rows;
  if (quant_rows > 0x7fffffff) return 0;
  return WorkspaceBytes(static_cast<int>(quant_rows), depth) +
         (adj_x ? TransposedBytes(lhs_matrices, rows, depth) : 0);
}

int lrtfc_batch_matmul_hybrid_packed_nd(const float* lhs, const int* lhs_batch_dims, int rows,
                                        int depth, int adj_x, const int8_t* packed_weights,
                                        const int* weight_batch_dims, int units,
                                        const float* per_channel_scales, float filter_scale,
                                        const int32_t* row_sums, float* output,
                                        int asymmetric_quantize_inputs, int quant_variant,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(lhs_batch_dims && weight_batch_dims, "null pointer");
  LRTFC_REQUIRE(rows >= 0 && depth > 0 && units >= 0, "bad dimension");
  int64_t lhs_matrices = 1, out_matrices = 1;
  int out_dims[3];
  for (int i = 0; i < 3; ++i) {
    const int l = lhs_batch_dims[i], w = weight_batch_dims[i];
    LRTFC_REQUIRE(l >= 0 && w >= 0, "bad dimension");
    LRTFC_REQUIRE(l == w || l == 1 || w == 1,
                  "batch dimension %d: %d against %d can not be broadcast", i, l, w);
    out_dims[i] = l == 1 ? w : l;  // batch_matmul.h:33-38
    lhs_matrices *= l;
    out_matrices *= out_dims[i];
    LRTFC_REQUIRE(out_matrices <= 0x7fffffff, "too many matrices");
  }
  if (out_matrices == 0 || rows == 0 || units == 0) return LRTFC_OK;
  const int64_t quant_rows = lhs_matrices * rows;
  LRTFC_REQUIRE(quant_rows <= 0x7fffffff, "too many rows");
  LRTFC_REQUIRE(lhs && packed_weights && row_sums && output && workspace, "null pointer");
  const size_t need =
      lrtfc_batch_matmul_workspace_bytes(static_cast<int>(lhs_matrices), rows, depth, adj_x);
  LRTFC_REQUIRE(workspace_bytes >= need, "workspace too small: %zu < %zu bytes", workspace_bytes,
                need);
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  void* quant_space = workspace;
  if (adj_x) {
    // The op's own first step (batch_matmul.cc:811-813): [.., depth, rows] -> [.., rows, depth].
    float* transposed = static_cast<float*>(workspace);
    quant_space = static_cast<char*>(workspace) + TransposedBytes(lhs_matrices, rows, depth);
    int rc = FromHip(lrtfc::LaunchTransposeLastTwoF32(lhs, static_cast<int>(lhs_matrices), depth,
                                                      rows, transposed, AsStream(stream)),
                     "left operand transposition");
    if (rc != LRTFC_OK) return rc;
    lhs = transposed;
  }
  // BatchQuantizeFloats over every row of the float operand (batch_matmul.cc:472-497); symmetric
  // quantization leaves the offsets at zero (:487-489).
  const Workspace w = SplitWorkspace(quant_space, static_cast<int>(quant_rows), depth);
  int rc = lrtfc_batch_quantize_floats(lhs, static_cast<int>(quant_rows), depth, w.q, w.sf, w.zp,
                                       asymmetric_quantize_inputs, quant_variant, stream);
  if (rc != LRTFC_OK) return rc;
  const int32_t* zp = asymmetric_quantize_inputs ? w.zp : nullptr;
  // Output matrix (b0, b1, b2) pairs the left matrix and the weight matrix whose indices keep
  // b_i where that side's dimension is not 1 (the extents of batch_matmul.h:42-52, :139-146).
  // Consecutive output matrices that share a weight matrix and take consecutive left matrices
  // are one product over all their rows.
  const size_t matrix_bytes = lrtfc::PackedInt8FilterBytes(units, depth);
  auto side_index = [&](const int* dims, int64_t o) {
    int64_t index = 0;
    int b[3];
    b[2] = static_cast<int>(o % out_dims[2]);
    b[1] = static_cast<int>((o / out_dims[2]) % out_dims[1]);
    b[0] = static_cast<int>(o / (static_cast<int64_t>(out_dims[2]) * out_dims[1]));
    for (int i = 0; i < 3; ++i) index = index * dims[i] + (dims[i] == 1 ? 0 : b[i]);
    return index;
  };
  int64_t o = 0;
  while (o < out_matrices) {
    const int64_t l0 = side_index(lhs_batch_dims, o), w0 = side_index(weight_batch_dims, o);
    int64_t run = 1;
    while (o + run < out_matrices && side_index(weight_batch_dims, o + run) == w0 &&
           side_index(lhs_batch_dims, o + run) == l0 + run &&
           (run + 1) * static_cast<int64_t>(rows) <= 0x7fffffff) {
      ++run;
    }
    const size_t row0 = static_cast<size_t>(l0) * rows;
    rc = FcHybridInt8Packed(w.q + row0 * depth, w.sf + row0, zp ? zp + row0 : nullptr,
                            packed_weights + static_cast<size_t>(w0) * matrix_bytes,
                            per_channel_scales, filter_scale,
                            row_sums + static_cast<size_t>(w0) * units, nullptr,
                            output + static_cast<size_t>(o) * rows * units,
                            static_cast<int>(run * rows), depth, units, LRTFC_ACT_NONE, 0, stream,
                            /*batch_matmul=*/1);
    if (rc != LRTFC_OK) return rc;
    o += run;
  }
  return LRTFC_OK;
}

int lrtfc_batch_matmul_hybrid_packed(const float* lhs, int lhs_batches, int rows, int depth,
                                     const int8_t* packed_weights, int weight_matrices, int units,
                                     const float* per_channel_scales, float filter_scale,
                                     const int32_t* row_sums, float* output,
                                     int asymmetric_quantize_inputs, int quant_variant,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(lhs_batches >= 0 && weight_matrices >= 0, "bad dimension");
  LRTFC_REQUIRE(lhs_batches == weight_matrices || lhs_batches == 1 || weight_matrices == 1,
                "%d input batches against %d weight matrices: only equal counts, or one side "
                "broadcast, are supported", lhs_batches, weight_matrices);
  const int lhs_dims[3] = {1, 1, lhs_batches}, weight_dims[3] = {1, 1, weight_matrices};
  return lrtfc_batch_matmul_hybrid_packed_nd(lhs, lhs_dims, rows, depth, /*adj_x=*/0,
                                             packed_weights, weight_dims, units,
                                             per_channel_scales, filter_scale, row_sums, output,
                                             asymmetric_quantize_inputs, quant_variant, workspace,
                                             workspace_bytes, stream);
}

int lrtfc_batch_quantize_floats(const float* values, int n_batch, int n_data, int8_t* quantized,
                                float* scaling_factors, int32_t* zero_points, int do_asymmetric,
                                int variant, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(n_batch >= 0 && n_data >= 0, "negative dimension");
  if (n_batch == 0) return LRTFC_OK;
  LRTFC_REQUIRE(values && quantized && scaling_factors, "null pointer");
  LRTFC_REQUIRE(!do_asymmetric || zero_points, "zero_points is required for asymmetric mode");
  LRTFC_REQUIRE(variant >= 0 && variant <= LRTFC_QUANT_NEON_LEGACY, "unknown quantizer variant");
  LRTFC_REQUIRE(n_data > 0, "empty rows cannot be quantized");
  return FromHip(lrtfc::LaunchBatchQuantize(values, n_batch, n_data, quantized, scaling_factors,
                                            zero_points, do_asymmetric, variant,
                                            AsStream(stream)),
                 "batch quantize");
}

namespace {
int FcHybridInt8RowMajor(const int8_t* quantized_input, const float* scaling_factors,
                         const int32_t* zero_points, const int8_t* filter,
                         const float* per_channel_scales, float filter_scale,
                         const int32_t* filter_row_sums, const float* bias, float* output,
                         int batches, int depth, int out_depth, int activation,
                         int zero_input_exit, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth >= 0 && out_depth >= 0, "negative dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(output, "null output");
  LRTFC_REQUIRE(depth > 0, "depth 0 is handled by the caller (zero fill)");
  LRTFC_REQUIRE(quantized_input && scaling_factors && filter, "null pointer");
  LRTFC_REQUIRE(!zero_points || filter_row_sums,
                "filter_row_sums is required with activation zero points");
  LRTFC_REQUIRE(FloatActivationOk(activation),
                "activation %d is not one of None/Relu/ReluN1To1/Relu6/SignBit", activation);
  lrtfc::FcInt8Args a{};
  a.input = quantized_input;
  a.filter = filter;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.filter_row_sums = filter_row_sums;
  a.scaling_factors = scaling_factors;
  a.zero_points = zero_points;
  a.per_channel_scales = per_channel_scales;
  a.filter_scale = filter_scale;
  a.bias_f32 = bias;
  a.activation = activation;
  a.output_f32 = output;
  a.zero_input_exit = zero_input_exit;
  return FromHip(lrtfc::LaunchFcInt8Gemv(a, lrtfc::Int8Epilogue::kHybrid, AsStream(stream)),
                 "hybrid GEMV");
}
}  // namespace

int lrtfc_fc_hybrid_int8(const int8_t* quantized_input, const float* scaling_factors,
                         const int32_t* zero_points, const int8_t* filter,
                         const float* per_channel_scales, float filter_scale,
                         const int32_t* filter_row_sums, const float* bias, float* output,
                         int batches, int depth, int out_depth, int activation, void* stream) {
  return FcHybridInt8RowMajor(quantized_input, scaling_factors, zero_points, filter,
                              per_channel_scales, filter_scale, filter_row_sums, bias, output,
                              batches, depth, out_depth, activation, /*zero_input_exit=*/0,
                              stream);
}

size_t lrtfc_activation_workspace_bytes(int batches, int depth) {
  if (batches <= 0 || depth <= 0) return 0;
  return WorkspaceBytes(batches, depth);
}

int lrtfc_fc_hybrid(const float* input, const int8_t* filter, const float* per_channel_scales,
                    float filter_scale, const int32_t* filter_row_sums, const float* bias,
                    float* output, int batches, int depth, int out_depth,
                    int asymmetric_quantize_inputs, int activation, int quant_variant,
                    void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth >= 0 && out_depth >= 0, "negative dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(output, "null output");
  if (depth == 0) {
    return FromHip(lrtfc::LaunchZeroFill(output, sizeof(float) * batches * out_depth,
                                         AsStream(stream)),
                   "zero fill");
  }
  LRTFC_REQUIRE(input && workspace, "null pointer");
  LRTFC_REQUIRE(workspace_bytes >= WorkspaceBytes(batches, depth),
                "workspace too small: %zu < %zu bytes", workspace_bytes,
                WorkspaceBytes(batches, depth));
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  const Workspace w = SplitWorkspace(workspace, batches, depth);
  int rc = lrtfc_batch_quantize_floats(input, batches, depth, w.q, w.sf, w.zp,
                                       asymmetric_quantize_inputs, quant_variant, stream);
  if (rc != LRTFC_OK) return rc;
  // Symmetric quantization still writes zero points of 0, so the offset form of the
  // product applies to both modes, as in EvalHybridDense.
  return FcHybridInt8RowMajor(w.q, w.sf, w.zp, filter, per_channel_scales, filter_scale,
                              filter_row_sums, bias, output, batches, depth, out_depth, activation,
                              /*zero_input_exit=*/1, stream);
}

size_t lrtfc_static_scratch_bytes(void) { return LRTFC_STATIC_SCRATCH_BYTES; }

int lrtfc_fc_hybrid_static_scratch(const float* input, const int8_t* filter,
                                   const float* per_channel_scales, float filter_scale,
                                   const int32_t* filter_row_sums, const float* bias,
                                   float* output, int batches, int depth, int out_depth,
                                   int asymmetric_quantize_inputs, int activation,
                                   int quant_variant, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth >= 0 && out_depth >= 0, "negative dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(WorkspaceBytes(batches, depth) <= LRTFC_STATIC_SCRATCH_BYTES,
                "%d rows of depth %d need %zu bytes of activation scratch; the static scratch "
                "holds %d (use lrtfc_fc_hybrid with a workspace of the caller's)",
                batches, depth, WorkspaceBytes(batches, depth), LRTFC_STATIC_SCRATCH_BYTES);
  int device = -1;
  if (hipError_t err = hipGetDevice(&device)) return FromHip(err, "hipGetDevice");
  void* ptr = (device >= 0 && device < kMaxDevices) ? g_scratch_ptr[device].load() : nullptr;
  if (ptr == nullptr) {
    return Fail(LRTFC_NO_DEVICE,
                "lrtfc_init() has not run for device %d: its scratch address is unknown", device);
  }
  // Same two launches as lrtfc_fc_hybrid; the quantizer rewrites every byte the product reads,
  // so what the previous call left in the array does not matter.
  return lrtfc_fc_hybrid(input, filter, per_channel_scales, filter_scale, filter_row_sums, bias,
                         output, batches, depth, out_depth, asymmetric_quantize_inputs, activation,
                         quant_variant, ptr, LRTFC_STATIC_SCRATCH_BYTES, stream);
}

int lrtfc_fc_blockwise_int4_quantized(const int8_t* quantized_input,
                                      const float* scaling_factors, const int32_t* zero_points,
                                      const uint8_t* packed_filter, const uint16_t* scales_f16,
                                      const float* kfsum, const float* bias, float* output,
                                      int batches, int depth, int out_depth, int blocksize,
                                      void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth >= 0 && out_depth >= 0, "negative dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(output, "null output");
  LRTFC_REQUIRE(depth > 0 && depth % 2 == 0, "depth %d must be positive and even", depth);
  LRTFC_REQUIRE(blocksize > 0 && depth % blocksize == 0, "blocksize %d does not divide depth %d",
                blocksize, depth);
  LRTFC_REQUIRE(quantized_input && scaling_factors && zero_points && packed_filter &&
                    scales_f16 && kfsum,
                "null pointer");
  lrtfc::FcInt4Args a{};
  a.input = quantized_input;
  a.scaling_factors = scaling_factors;
  a.zero_points = zero_points;
  a.packed_filter = packed_filter;
  a.scales_f16 = scales_f16;
  a.kfsum = kfsum;
  a.bias = bias;
  a.output = output;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.blocksize = blocksize;
  return FromHip(lrtfc::LaunchFcBlockwiseInt4(a, AsStream(stream)), "blockwise int4 GEMV");
}

size_t lrtfc_packed_int4_blockwise_bytes(int out_depth, int depth) {
  if (out_depth <= 0 || depth <= 0) return 0;
  return lrtfc::PackedInt4BlockwiseBytes(out_depth, depth);
}

int lrtfc_pack_int4_blockwise(const uint8_t* packed_filter, const uint16_t* scales_f16,
                              int out_depth, int depth, int blocksize, uint8_t* retiled,
                              void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(out_depth >= 0 && depth >= 0, "negative dimension");
  if (out_depth == 0 || depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(lrtfc::FcInt4PackedSupports(depth, blocksize),
                "the re-tiled form needs blocksize 32 dividing the depth (got blocksize %d, "
                "depth %d)", blocksize, depth);
  LRTFC_REQUIRE(packed_filter && scales_f16 && retiled, "null pointer");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(retiled) & 15) == 0, "retiled must be 16-byte aligned");
  return FromHip(lrtfc::LaunchPackInt4Blockwise(packed_filter, scales_f16, out_depth, depth,
                                                retiled, AsStream(stream)),
                 "pack int4 blockwise filter");
}

namespace {
int FcInt4PackedCommon(const float* input_f32, const int8_t* q, const float* sf, const int32_t* zp,
                       const uint8_t* retiled, const float* kfsum, const float* bias,
                       float* output, int batches, int depth, int out_depth, int variant,
                       void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(lrtfc::FcInt4PackedSupports(depth, 32), "depth %d is not a multiple of 32", depth);
  LRTFC_REQUIRE(retiled && kfsum && output, "null pointer");
  LRTFC_REQUIRE(input_f32 || (q && sf && zp), "null input");
  LRTFC_REQUIRE(variant >= 0 && variant <= LRTFC_QUANT_NEON_LEGACY, "unknown quantizer variant");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(retiled) & 15) == 0,
                "retiled filter must be 16-byte aligned");
  lrtfc::FcInt4Args a{};
  a.input = q;
  a.scaling_factors = sf;
  a.zero_points = zp;
  a.kfsum = kfsum;
  a.bias = bias;
  a.output = output;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.blocksize = 32;
  return FromHip(lrtfc::LaunchFcInt4Packed(a, retiled, input_f32, variant, AsStream(stream)),
                 "re-tiled blockwise int4 GEMV");
}
}  // namespace

int lrtfc_fc_blockwise_int4_packed(const float* input, const uint8_t* retiled_filter,
                                   const float* kfsum, const float* bias, float* output,
                                   int batches, int depth, int out_depth, int quant_variant,
                                   void* stream) {
  if (batches > 0 && out_depth > 0 && !input) return Fail(LRTFC_INVALID_ARGUMENT, "null input");
  return FcInt4PackedCommon(input, nullptr, nullptr, nullptr, retiled_filter, kfsum, bias, output,
                            batches, depth, out_depth, quant_variant, stream);
}

int lrtfc_fc_blockwise_int4_packed_quantized(const int8_t* quantized_input,
                                             const float* scaling_factors,
                                             const int32_t* zero_points,
                                             const uint8_t* retiled_filter, const float* kfsum,
                                             const float* bias, float* output, int batches,
                                             int depth, int out_depth, void* stream) {
  return FcInt4PackedCommon(nullptr, quantized_input, scaling_factors, zero_points, retiled_filter,
                            kfsum, bias, output, batches, depth, out_depth, 0, stream);
}

int lrtfc_batch_quantize_floats_4bit(const float* values, int n_batch, int n_data,
                                     int8_t* quantized, float* scaling_factors,
                                     int32_t* input_offsets, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(n_batch >= 0 && n_data >= 0, "negative dimension");
  if (n_batch == 0) return LRTFC_OK;
  LRTFC_REQUIRE(values && quantized && scaling_factors && input_offsets, "null pointer");
  LRTFC_REQUIRE(n_data > 0, "empty rows cannot be quantized");
  return FromHip(lrtfc::LaunchBatchQuantize4Bit(values, n_batch, n_data, quantized,
                                                scaling_factors, input_offsets, AsStream(stream)),
                 "4-bit path row quantizer");
}

int lrtfc_fc_hybrid_int4_per_channel_packed(const float* input, const int8_t* packed_filter,
                                            const float* per_channel_scales, float filter_scale,
                                            const float* bias, float* output, int batches,
                                            int depth, int out_depth, int activation,
                                            void* workspace, size_t workspace_bytes,
                                            void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && packed_filter && output && workspace, "null pointer");
  LRTFC_REQUIRE(FloatActivationOk(activation),
                "activation %d is not one of None/Relu/ReluN1To1/Relu6/SignBit", activation);
  LRTFC_REQUIRE(workspace_bytes >= WorkspaceBytes(batches, depth),
                "workspace too small: %zu < %zu bytes", workspace_bytes,
                WorkspaceBytes(batches, depth));
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(packed_filter) & 15) == 0,
                "packed filter must be 16-byte aligned");
  const Workspace w = SplitWorkspace(workspace, batches, depth);
  int rc = lrtfc_batch_quantize_floats_4bit(input, batches, depth, w.q, w.sf, w.zp, stream);
  if (rc != LRTFC_OK) return rc;
  lrtfc::FcInt8Args a{};
  a.input = w.q;
  a.filter = packed_filter;
  a.batches = batches;
  a.depth = depth;
  a.out_depth = out_depth;
  a.scaling_factors = w.sf;
  a.zero_points = w.zp;  // the rows' input offsets on this path
  a.per_channel_scales = per_channel_scales;
  a.filter_scale = filter_scale;
  a.bias_f32 = bias;
  a.activation = activation;
  a.output_f32 = output;
  if (batches > kPackedGemmMinBatches && !lrtfc::FcInt8PackedGemvTakesRowsInOnePass(a) &&
      lrtfc::FcInt8PackedGemmSupports(a)) {
    return FromHip(lrtfc::LaunchFcInt8PackedGemm(a, lrtfc::Int8Epilogue::kHybrid4Bit,
                                                 AsStream(stream)),
                   "packed int4 per-channel hybrid GEMM");
  }
  return FromHip(lrtfc::LaunchFcInt8PackedGemv(a, lrtfc::Int8Epilogue::kHybrid4Bit, nullptr, 0,
                                               LRTFC_QUANT_PORTABLE, AsStream(stream)),
                 "packed int4 per-channel hybrid GEMV");
}

size_t lrtfc_packed_int4_per_channel_bytes(int out_depth, int depth) {
  if (out_depth <= 0 || depth <= 0) return 0;
  return lrtfc::PackedInt4PerChannelBytes(out_depth, depth);
}

int lrtfc_pack_int4_per_channel(const uint8_t* packed_filter, int out_depth, int depth,
                                uint8_t* retiled_filter, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(out_depth >= 0 && depth >= 0, "bad dimension");
  if (out_depth == 0 || depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(depth % 2 == 0, "depth %d is odd: rows of nibbles must end on a byte", depth);
  LRTFC_REQUIRE(packed_filter && retiled_filter, "null pointer");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(retiled_filter) & 15) == 0,
                "re-tiled filter must be 16-byte aligned");
  return FromHip(lrtfc::LaunchPackInt4PerChannel(packed_filter, out_depth, depth, retiled_filter,
                                                 AsStream(stream)),
                 "per-channel int4 filter re-tiling");
}

int lrtfc_fc_hybrid_int4_per_channel_nibbles(const float* input, const uint8_t* retiled_filter,
                                             const float* per_channel_scales, float filter_scale,
                                             const float* bias, float* output, int batches,
                                             int depth, int out_depth, int activation,
                                             void* workspace, size_t workspace_bytes,
                                             void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && retiled_filter && output && workspace, "null pointer");
  LRTFC_REQUIRE(FloatActivationOk(activation),
                "activation %d is not one of None/Relu/ReluN1To1/Relu6/SignBit", activation);
  LRTFC_REQUIRE(lrtfc::FcInt4PerChannelGemvSupports(depth),
                "depth %d is odd or too large for the nibble GEMV", depth);
  LRTFC_REQUIRE(workspace_bytes >= WorkspaceBytes(batches, depth),
                "workspace too small: %zu < %zu bytes", workspace_bytes,
                WorkspaceBytes(batches, depth));
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(retiled_filter) & 15) == 0,
                "re-tiled filter must be 16-byte aligned");
  if (lrtfc::FcInt4PerChannelGemvFuses(input, batches, depth)) {  // one kernel, no workspace use
    return FromHip(lrtfc::LaunchFcInt4PerChannelGemv(retiled_filter, input, nullptr, nullptr,
                                                     nullptr, per_channel_scales, filter_scale,
                                                     bias, output, batches, depth, out_depth,
                                                     activation, AsStream(stream)),
                   "per-channel int4 hybrid GEMV (nibble layout, fused quantizer)");
  }
  const Workspace w = SplitWorkspace(workspace, batches, depth);
  int rc = lrtfc_batch_quantize_floats_4bit(input, batches, depth, w.q, w.sf, w.zp, stream);
  if (rc != LRTFC_OK) return rc;
  return FromHip(lrtfc::LaunchFcInt4PerChannelGemv(retiled_filter, nullptr, w.q, w.sf, w.zp,
                                                   per_channel_scales, filter_scale, bias, output,
                                                   batches, depth, out_depth, activation,
                                                   AsStream(stream)),
                 "per-channel int4 hybrid GEMV (nibble layout)");
}

size_t lrtfc_gemm_int4_blockwise_bytes(int out_depth, int depth) {
  if (out_depth <= 0 || depth <= 0) return 0;
  return lrtfc::GemmInt4BlockwiseBytes(out_depth, depth);
}

int lrtfc_pack_int4_blockwise_gemm(const uint8_t* packed_filter, const uint16_t* scales_f16,
                                   int out_depth, int depth, int blocksize, uint8_t* gemm_filter,
                                   void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(out_depth >= 0 && depth >= 0, "negative dimension");
  if (out_depth == 0 || depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(packed_filter && scales_f16 && gemm_filter, "null pointer");
  LRTFC_REQUIRE(lrtfc::FcInt4BlockwiseGemmSupports(depth, blocksize),
                "the int4 GEMM needs block size 32 and a depth that is a multiple of 32");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(gemm_filter) & 15) == 0,
                "re-tiled filter must be 16-byte aligned");
  return FromHip(lrtfc::LaunchPackInt4BlockwiseGemm(packed_filter, scales_f16, out_depth, depth,
                                                    gemm_filter, AsStream(stream)),
                 "int4 GEMM filter re-tiling");
}

size_t lrtfc_fc_blockwise_int4_gemm_workspace_bytes(int batches, int depth) {
  if (batches <= 0 || depth <= 0) return 0;
  // Tiled int8 rows (the batch padded to whole tiles), scaling factors, zero points.
  return lrtfc::AlignUp256(lrtfc::TiledRowsBytes(batches, depth)) +
         2 * lrtfc::AlignUp256(static_cast<size_t>(batches) * 4);
}

int lrtfc_fc_blockwise_int4_gemm(const float* input, const uint8_t* gemm_filter,
                                 const float* kfsum, const float* bias, float* output,
                                 int batches, int depth, int out_depth, int quant_variant,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && gemm_filter && kfsum && output && workspace, "null pointer");
  LRTFC_REQUIRE(lrtfc::FcInt4BlockwiseGemmSupports(depth, 32), "depth %d is not a multiple of 32",
                depth);
  LRTFC_REQUIRE(workspace_bytes >= lrtfc_fc_blockwise_int4_gemm_workspace_bytes(batches, depth),
                "workspace too small: %zu < %zu bytes", workspace_bytes,
                lrtfc_fc_blockwise_int4_gemm_workspace_bytes(batches, depth));
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(gemm_filter) & 15) == 0,
                "re-tiled filter must be 16-byte aligned");
  LRTFC_REQUIRE(quant_variant >= LRTFC_QUANT_PORTABLE && quant_variant <= LRTFC_QUANT_NEON_LEGACY,
                "unknown quantizer variant %d", quant_variant);
  char* p = static_cast<char*>(workspace);
  void* tiled = p;
  p += lrtfc::AlignUp256(lrtfc::TiledRowsBytes(batches, depth));
  float* scaling_factors = reinterpret_cast<float*>(p);
  p += lrtfc::AlignUp256(static_cast<size_t>(batches) * 4);
  int32_t* zero_points = reinterpret_cast<int32_t*>(p);
  return FromHip(lrtfc::LaunchFcInt4BlockwiseGemm(input, quant_variant, scaling_factors,
                                                  zero_points, gemm_filter, kfsum, bias, output,
                                                  batches, depth, out_depth, tiled,
                                                  AsStream(stream)),
                 "blockwise int4 GEMM");
}

int lrtfc_fc_blockwise_int4_preferred_form(int batches, int depth, int out_depth) {
  if (depth <= 0 || depth % 32 != 0 || !lrtfc::FcInt4PackedSupports(depth, 32)) {
    return LRTFC_INT4_FORM_DECODE;
  }
  // Up to four rows the streaming kernel makes one pass over the filter. Beyond that the GEMMs
  // stream it once for the whole batch: the nibble-resident one where the filter stream is the
  // bound (up to 32 rows) and the filter is wide enough to give every SIMD a wavefront (one
  // wavefront per 16 channels walks the whole depth: 14336 x 4096 takes 16.8 us at 5 to 16
  // rows against 24 us in two passes of the streaming kernel and 21 us on the int8 copy), the
  // int8-expanded one from 16 rows on otherwise.
  const int channel_tiles = (out_depth + 15) / 16;
  if (batches <= 4) return LRTFC_INT4_FORM_DECODE;
  if (batches <= 32 && channel_tiles >= 512 && depth <= 8192) return LRTFC_INT4_FORM_GEMM_NIBBLES;
  return batches >= 16 ? LRTFC_INT4_FORM_GEMM_INT8 : LRTFC_INT4_FORM_DECODE;
}

size_t lrtfc_gemm_int4_blockwise_nibble_bytes(int out_depth, int depth) {
  if (out_depth <= 0 || depth <= 0) return 0;
  return lrtfc::GemmInt4BlockwiseNibbleBytes(out_depth, depth);
}

int lrtfc_pack_int4_blockwise_gemm_nibbles(const uint8_t* packed_filter,
                                           const uint16_t* scales_f16, int out_depth, int depth,
                                           int blocksize, uint8_t* nibble_filter, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(out_depth >= 0 && depth >= 0, "negative dimension");
  if (out_depth == 0 || depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(packed_filter && scales_f16 && nibble_filter, "null pointer");
  LRTFC_REQUIRE(lrtfc::FcInt4BlockwiseGemmSupports(depth, blocksize),
                "the int4 GEMM needs block size 32 and a depth that is a multiple of 32");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(nibble_filter) & 15) == 0,
                "re-tiled filter must be 16-byte aligned");
  return FromHip(lrtfc::LaunchPackInt4BlockwiseNibbles(packed_filter, scales_f16, out_depth,
                                                       depth, nibble_filter, AsStream(stream)),
                 "int4 nibble GEMM filter re-tiling");
}

int lrtfc_fc_blockwise_int4_gemm_nibbles(const float* input, const uint8_t* nibble_filter,
                                 const float* kfsum, const float* bias, float* output,
                                 int batches, int depth, int out_depth, int quant_variant,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth > 0 && out_depth >= 0, "bad dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && nibble_filter && kfsum && output && workspace, "null pointer");
  LRTFC_REQUIRE(lrtfc::FcInt4BlockwiseGemmSupports(depth, 32), "depth %d is not a multiple of 32",
                depth);
  LRTFC_REQUIRE(workspace_bytes >= lrtfc_fc_blockwise_int4_gemm_workspace_bytes(batches, depth),
                "workspace too small: %zu < %zu bytes", workspace_bytes,
                lrtfc_fc_blockwise_int4_gemm_workspace_bytes(batches, depth));
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(nibble_filter) & 15) == 0,
                "re-tiled filter must be 16-byte aligned");
  LRTFC_REQUIRE(quant_variant >= LRTFC_QUANT_PORTABLE && quant_variant <= LRTFC_QUANT_NEON_LEGACY,
                "unknown quantizer variant %d", quant_variant);
  char* p = static_cast<char*>(workspace);
  void* tiled = p;
  p += lrtfc::AlignUp256(lrtfc::TiledRowsBytes(batches, depth));
  float* scaling_factors = reinterpret_cast<float*>(p);
  p += lrtfc::AlignUp256(static_cast<size_t>(batches) * 4);
  int32_t* zero_points = reinterpret_cast<int32_t*>(p);
  return FromHip(lrtfc::LaunchFcInt4BlockwiseNibbleGemm(input, quant_variant, scaling_factors,
                                                  zero_points, nibble_filter, kfsum, bias, output,
                                                  batches, depth, out_depth, tiled,
                                                  AsStream(stream)),
                 "blockwise int4 GEMM (nibble layout)");
}

int lrtfc_embedding_lookup_blockwise_int4(const int32_t* lookup, int count, const uint8_t* table,
                                          int rows, int cols, const uint16_t* scales_f16,
                                          int blocksize, int out_type, void* output,
                                          int32_t* status, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(count >= 0 && rows >= 0 && cols >= 0, "bad dimension");
  LRTFC_REQUIRE(out_type == LRTFC_OUT_FLOAT32 || out_type == LRTFC_OUT_FLOAT16,
                "output type %d is neither float32 nor float16", out_type);
  LRTFC_REQUIRE(blocksize > 0 && cols % blocksize == 0,
                "lookup dimension %d must be divisible by blocksize %d", cols, blocksize);
  LRTFC_REQUIRE(cols % 2 == 0 && blocksize % 2 == 0,
                "Int4 rows and blocks must hold an even number of columns");
  if (count > 0 && cols > 0) {
    LRTFC_REQUIRE(lookup && table && scales_f16 && output, "null pointer");
  } else {
    LRTFC_REQUIRE(count == 0 || lookup, "null pointer");
  }
  return FromHip(lrtfc::LaunchEmbeddingLookup(lookup, count, table, 4, rows, cols, scales_f16,
                                              blocksize, nullptr, 0.0f,
                                              out_type == LRTFC_OUT_FLOAT16, output, status,
                                              AsStream(stream)),
                 "blockwise int4 embedding lookup");
}

int lrtfc_embedding_lookup_hybrid(const int32_t* lookup, int count, const void* table,
                                  int value_bits, int rows, int cols, float scale,
                                  const float* row_scales, int out_type, void* output,
                                  int32_t* status, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(count >= 0 && rows >= 0 && cols >= 0, "bad dimension");
  LRTFC_REQUIRE(value_bits == 4 || value_bits == 8, "value_bits %d is neither 4 nor 8",
                value_bits);
  LRTFC_REQUIRE(out_type == LRTFC_OUT_FLOAT32 || out_type == LRTFC_OUT_FLOAT16,
                "output type %d is neither float32 nor float16", out_type);
  LRTFC_REQUIRE(value_bits == 8 || cols % 2 == 0,
                "Int4 rows must hold an even number of columns");
  if (count > 0 && cols > 0) {
    LRTFC_REQUIRE(lookup && table && output, "null pointer");
  } else {
    LRTFC_REQUIRE(count == 0 || lookup, "null pointer");
  }
  return FromHip(lrtfc::LaunchEmbeddingLookup(lookup, count, table, value_bits, rows, cols,
                                              nullptr, 0, row_scales, scale,
                                              out_type == LRTFC_OUT_FLOAT16, output, status,
                                              AsStream(stream)),
                 "hybrid embedding lookup");
}

namespace {
// Stream order puts this kernel after everything enqueued before it, and a kernel's end makes
// its stores visible system-wide, so the host that reads `value` here may read those results.
__global__ void MarkCompletionKernel(volatile uint32_t* flag, uint32_t value) {
  if (threadIdx.x == 0) {
    __threadfence_system();
    *flag = value;
  }
}
}  // namespace

int lrtfc_mark_completion(uint32_t* flag, uint32_t value, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(flag, "null pointer");
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(flag) & 3) == 0, "flag must be 4-byte aligned");
  hipLaunchKernelGGL(MarkCompletionKernel, dim3(1), dim3(lrtfc::kWaveSize), 0, AsStream(stream),
                     flag, value);
  return FromHip(hipGetLastError(), "completion mark");
}

size_t lrtfc_int4_group_table_bytes(void) { return lrtfc::Int4GroupTableBytes(); }

int lrtfc_int4_group_preferred_form(const int* out_depths, int count, int batches, int depth) {
  if (!out_depths || count < 1) return LRTFC_INT4_FORM_DECODE;
  int64_t tiles = 0;
  for (int i = 0; i < count; ++i) tiles += (static_cast<int64_t>(out_depths[i]) + 15) / 16;
  return lrtfc::Int4NibbleGroupWins(batches, depth, tiles > 0x7fffffff ? 0x7fffffff : static_cast<int>(tiles))
             ? LRTFC_INT4_FORM_GEMM_NIBBLES
             : LRTFC_INT4_FORM_DECODE;
}

int lrtfc_int4_group_prepare(const lrtfc_int4_group_node* nodes, int count, int batches,
                             int depth, void* device_table, lrtfc_int4_group_launch* launch,
                             void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(nodes && device_table && launch, "null pointer");
  LRTFC_REQUIRE(count >= 1 && count <= LRTFC_INT4_GROUP_MAX, "a group holds 1..%d nodes, got %d",
                LRTFC_INT4_GROUP_MAX, count);
  LRTFC_REQUIRE(lrtfc::FcInt4PackedSupports(depth, 32), "depth %d is not a multiple of 32", depth);
  LRTFC_REQUIRE(batches >= 1, "a grouped launch needs at least one batch row");
  for (int i = 0; i < count; ++i) {
    LRTFC_REQUIRE(nodes[i].input && (nodes[i].retiled_filter || nodes[i].nibble_filter) &&
                      nodes[i].kfsum && nodes[i].output,
                  "null pointer in node %d", i);
    LRTFC_REQUIRE(nodes[i].out_depth >= 1, "node %d has no output channels", i);
    LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(nodes[i].retiled_filter) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(nodes[i].nibble_filter) & 15) == 0,
                  "re-tiled filter of node %d must be 16-byte aligned", i);
    LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(nodes[i].workspace) & 255) == 0,
                  "workspace of node %d must be 256-byte aligned", i);
  }
  const hipError_t err = lrtfc::PrepareInt4Group(nodes, count, batches, depth, device_table,
                                                 launch, AsStream(stream));
  LRTFC_REQUIRE(err != hipErrorInvalidValue,
                "a node of the group brings neither the filter form this shape runs on nor the "
                "decode tiling (and, for the 4-bit-resident form, a workspace)");
  return FromHip(err, "int4 group table upload");
}

int lrtfc_fc_blockwise_int4_packed_grouped(const void* device_table,
                                           const lrtfc_int4_group_launch* launch,
                                           int quant_variant, void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(device_table && launch, "null pointer");
  LRTFC_REQUIRE(launch->count >= 1 && launch->count <= LRTFC_INT4_GROUP_MAX &&
                    launch->grid_blocks >= 1 && launch->ksplit >= 1 && launch->ksplit <= 4 &&
                    launch->groups_per_wave >= 1 && launch->groups_per_wave <= 8 &&
                    (launch->ksplit == 1 || launch->groups_per_wave == 1) &&
                    launch->split_quantize >= 0 && launch->split_quantize <= 2 &&
                    (launch->form == LRTFC_INT4_FORM_DECODE ||
                     launch->form == LRTFC_INT4_FORM_GEMM_NIBBLES),
                "launch record was not filled by lrtfc_int4_group_prepare");
  LRTFC_REQUIRE(quant_variant >= 0 && quant_variant <= LRTFC_QUANT_NEON_LEGACY,
                "unknown quantizer variant");
  return FromHip(lrtfc::LaunchFcInt4PackedGrouped(device_table, *launch, quant_variant,
                                                  AsStream(stream)),
                 "grouped blockwise int4 GEMV");
}

int lrtfc_fc_blockwise_int4(const float* input, const uint8_t* packed_filter,
                            const uint16_t* scales_f16, const float* kfsum, const float* bias,
                            float* output, int batches, int depth, int out_depth, int blocksize,
                            int quant_variant, void* workspace, size_t workspace_bytes,
                            void* stream) {
  if (int rc = RequireInit()) return rc;
  LRTFC_REQUIRE(batches >= 0 && depth >= 0 && out_depth >= 0, "negative dimension");
  if (batches == 0 || out_depth == 0) return LRTFC_OK;
  LRTFC_REQUIRE(input && workspace, "null pointer");
  LRTFC_REQUIRE(depth > 0, "depth must be positive");
  LRTFC_REQUIRE(workspace_bytes >= WorkspaceBytes(batches, depth),
                "workspace too small: %zu < %zu bytes", workspace_bytes,
                WorkspaceBytes(batches, depth));
  LRTFC_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0,
                "workspace must be 256-byte aligned");
  const Workspace w = SplitWorkspace(workspace, batches, depth);
  // EvalBlockwise4Bit always quantizes asymmetrically (fully_connected.cc:1044-1047).
  int rc = lrtfc_batch_quantize_floats(input, batches, depth, w.q, w.sf, w.zp,
                                       /*do_asymmetric=*/1, quant_variant, stream);
  if (rc != LRTFC_OK) return rc;
  return lrtfc_fc_blockwise_int4_quantized(w.q, w.sf, w.zp, packed_filter, scales_f16, kfsum, bias,
                                           output, batches, depth, out_depth, blocksize, stream);
}

}  // extern "C"

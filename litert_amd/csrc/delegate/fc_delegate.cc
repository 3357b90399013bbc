// TfLiteDelegate plugin that claims quantized FULLY_CONNECTED nodes and runs them on
// an MI355X through the C ABI of include/litert_amd_fc.h.
//
// Boundary (reference tree): the plugin is loaded by TfLiteExternalDelegateCreate
// (tflite/delegates/external/external_delegate.cc:39-60, 215-223) through
// tflite_plugin_create_delegate / tflite_plugin_destroy_delegate
// (external_delegate_interface.h:65-74). Delegate::Prepare inspects the execution
// plan and hands the nodes it supports to ReplaceNodeSubsetsWithDelegateKernels
// (tflite/core/c/common.h:982-986); the runtime then drives the kernel registration's
// init / prepare / invoke / free for each partition (tflite/core/subgraph.cc:523-637,
// 1691-1775). Nodes the predicate below declines stay on the CPU kernels.
//
// Device residency: constant tensors (filter, bias, scales) are uploaded and
// pre-reduced once in `prepare`; activations cross PCIe once in and once out per
// partition invoke, and tensors produced and consumed inside one partition never
// leave HBM.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <vector>

#include "litert_amd_delegate.h"
#include "litert_amd_fc.h"
#include "tflite_abi.h"

namespace {

constexpr int kMaxFcVersion = 14;  // tflite/core/kernels/register.cc:84-86
constexpr int kMaxBatchMatMulVersion = 4;  // tflite/core/kernels/register.cc:327-329

struct Options {
  int device = 0;
  int streams = 4;  // HIP streams a partition spreads independent nodes over (1..4)
  int quant_variant = LRTFC_QUANT_PORTABLE;
  bool claim_int8 = true;
  bool claim_hybrid = true;
  bool claim_int4_blockwise = true;
  bool claim_int4_per_channel = true;
  bool claim_embedding_lookup = true;
  bool claim_batch_matmul = true;
  // Decode-sized host inputs are read by the kernels straight from page-locked host memory
  // instead of being copied to the device first ("direct_inputs": "0" turns that off).
  bool direct_inputs = true;
  // How an invoke waits for the device: by polling a word of page-locked memory that a
  // one-wavefront kernel behind the partition's last command stores to ("completion": "poll"),
  // or in hipStreamSynchronize ("sync"). Polling sees the end about 3.5 us earlier.
  bool poll_completion = true;
};

// Device memory the application registered for a tensor (litert_amd_register_device_buffer);
// a TfLiteBufferHandle is an index into DelegateState::buffers. The memory stays the
// application's: freeing a handle only empties its slot.
struct RegisteredBuffer {
  void* device = nullptr;
  size_t bytes = 0;
};

// What a metrics collection (litert_amd_start_metrics .. litert_amd_stop_metrics) adds up over
// the partition invokes between the two calls.
struct MetricsState {
  bool on = false;
  int detail_level = 0;
  int64_t invokes = 0;        // partition invokes
  int64_t nodes = 0;          // FULLY_CONNECTED / EMBEDDING_LOOKUP nodes those invokes ran
  int64_t uploaded = 0;       // bytes copied host -> device
  int64_t downloaded = 0;     // bytes copied device -> host
  double host_us = 0.0;       // wall time inside the partitions' invoke callbacks
  double device_us = 0.0;     // first enqueued copy to last finished one, per invoke, by HIP events
  double gather_us = 0.0, enqueue_us = 0.0, wait_us = 0.0, scatter_us = 0.0;  // host_us by phase
};

struct DelegateState {
  Options options;
  TfLiteDelegate delegate;
  std::vector<RegisteredBuffer> buffers;
  MetricsState metrics;
};

// The registered memory behind a tensor that carries one of this delegate's handles, or
// null: the tensor then lives in host memory as usual.
const RegisteredBuffer* BoundBuffer(const DelegateState* state, const TfLiteTensor& t) {
  if (t.delegate != &state->delegate || t.buffer_handle == kTfLiteNullBufferHandle) return nullptr;
  if (t.buffer_handle < 0 || static_cast<size_t>(t.buffer_handle) >= state->buffers.size()) {
    return nullptr;
  }
  const RegisteredBuffer& b = state->buffers[t.buffer_handle];
  return b.device ? &b : nullptr;
}

enum class FcKind {
  kNone, kInt8, kHybrid, kInt4Blockwise, kHybridInt4, kEmbeddingLookup, kBatchMatMul
};

int64_t NumElements(const TfLiteIntArray* dims) {
  int64_t n = 1;
  for (int i = 0; i < dims->size; ++i) n *= dims->data[i];
  return n;
}

bool IsConstant(const TfLiteTensor& t) {
  // tflite/kernels/kernel_util.h:191-193
  return t.allocation_type == kTfLiteMmapRo && t.data.raw != nullptr;
}

const TfLiteTensor* OptionalInput(const TfLiteContext* ctx, const TfLiteNode* node, int i) {
  if (i >= node->inputs->size) return nullptr;
  const int idx = node->inputs->data[i];
  if (idx == kTfLiteOptionalTensor) return nullptr;
  return &ctx->tensors[idx];
}

bool ClippingActivation(TfLiteFusedActivation a) {
  return a == kTfLiteActNone || a == kTfLiteActRelu || a == kTfLiteActReluN1To1 ||
         a == kTfLiteActRelu6;
}

// EMBEDDING_LOOKUP nodes whose table is quantized and whose rows come out as floats: what
// EvalBlockwise and EvalHybrid of the builtin accept (tflite/kernels/embedding_lookup.cc:49-100,
// 194-225, 397-412) for Int4 and Int8 tables. Float tables (a plain row copy), UInt8 and Int2
// tables stay on the CPU.
FcKind ClassifyEmbeddingLookup(const TfLiteContext* ctx, const TfLiteNode* node,
                               const Options& opt, std::string* why_not) {
  auto no = [&](const char* reason) {
    if (why_not) *why_not = reason;
    return FcKind::kNone;
  };
  if (!opt.claim_embedding_lookup) return no("embedding lookup disabled by option");
  if (node->inputs->size != 2 || node->outputs->size != 1) return no("needs 2 inputs, 1 output");
  const TfLiteTensor& lookup = ctx->tensors[node->inputs->data[0]];
  const TfLiteTensor& value = ctx->tensors[node->inputs->data[1]];
  const TfLiteTensor& output = ctx->tensors[node->outputs->data[0]];
  if (!lookup.dims || lookup.dims->size != 1 || lookup.type != kTfLiteInt32) {
    return no("lookup is not a rank-1 int32 tensor");
  }
  if (!value.dims || value.dims->size < 2) return no("table has fewer than 2 dimensions");
  if (!IsConstant(value)) return no("table is not a constant tensor");
  if (output.type != kTfLiteFloat32 && output.type != kTfLiteFloat16) {
    return no("output is not float32 or float16");
  }
  const int rows = value.dims->data[0];
  int64_t cols = 1;
  for (int i = 1; i < value.dims->size; ++i) cols *= value.dims->data[i];
  if (cols > 0x7FFFFFFF) return no("row too long");
  if (value.quantization.type == kTfLiteBlockwiseQuantization) {
    if (value.type != kTfLiteInt4) return no("blockwise table is not Int4");
    if (value.dims->size != 2) return no("blockwise table is not rank 2");
    const auto* bq = static_cast<const TfLiteBlockwiseQuantization*>(value.quantization.params);
    if (!bq || bq->blocksize <= 0 || cols % bq->blocksize != 0) return no("bad blocksize");
    if (cols % 2 != 0 || bq->blocksize % 2 != 0) return no("odd row or block length");
    if (bq->scale < 0 || static_cast<size_t>(bq->scale) >= ctx->tensors_size) {
      return no("scale tensor index out of range");
    }
    const TfLiteTensor& scales = ctx->tensors[bq->scale];
    if (scales.type != kTfLiteFloat16 || !IsConstant(scales)) return no("scales not const fp16");
    if (NumElements(scales.dims) != static_cast<int64_t>(rows) * (cols / bq->blocksize)) {
      return no("scale count != rows x blocks");
    }
    return FcKind::kEmbeddingLookup;
  }
  if (value.type != kTfLiteInt8 && value.type != kTfLiteInt4) {
    return no("table type is left to the CPU kernels");
  }
  if (value.type == kTfLiteInt4 && cols % 2 != 0) return no("odd row length");
  if (value.quantization.type == kTfLiteAffineQuantization) {
    const auto* q = static_cast<const TfLiteAffineQuantization*>(value.quantization.params);
    if (!q || !q->scale || !q->zero_point || q->scale->size < 1 || q->zero_point->size < 1) {
      return no("table has no scales");
    }
    if (q->zero_point->data[0] != 0) return no("non-zero table zero point");
    if (q->scale->size > 1) {
      if (q->quantized_dimension != 0 || q->scale->size != rows) {
        return no("per-row scales do not match the rows");
      }
      if (q->zero_point->size != rows && q->zero_point->size != 1) return no("bad zero points");
    }
  }
  return FcKind::kEmbeddingLookup;
}

// Shape facts of a BATCH_MATMUL node with a float left operand and a constant int8 right one:
// the op extends both shapes to rank 5 and broadcasts the three batch dimensions pair by pair
// (tflite/kernels/batch_matmul.cc:356-391, reference/batch_matmul.h:120-146); adj_x / adj_y say
// which of an operand's last two dimensions is the accumulation depth.
struct BatchMatMulShape {
  int lhs_batches = 1, matrices = 1, rows = 0, depth = 0, units = 0;
  int64_t out_batches = 1;
  int lhs_dims[3] = {1, 1, 1}, weight_dims[3] = {1, 1, 1};
};
bool BatchMatMulGeometry(const TfLiteTensor& lhs, const TfLiteTensor& rhs, bool adj_x, bool adj_y,
                         BatchMatMulShape* out, const char** why) {
  const int lr = lhs.dims->size, rr = rhs.dims->size;
  if (lr < 2 || lr > 5 || rr < 2 || rr > 5) return *why = "operand rank outside 2..5", false;
  BatchMatMulShape g;
  g.rows = lhs.dims->data[adj_x ? lr - 1 : lr - 2];
  g.depth = lhs.dims->data[adj_x ? lr - 2 : lr - 1];
  g.units = adj_y ? rhs.dims->data[rr - 2] : rhs.dims->data[rr - 1];
  if ((adj_y ? rhs.dims->data[rr - 1] : rhs.dims->data[rr - 2]) != g.depth) {
    return *why = "accumulation depths differ", false;
  }
  for (int i = 0; i < 3; ++i) {
    const int l = i - (5 - lr) >= 0 ? lhs.dims->data[i - (5 - lr)] : 1;
    const int r = i - (5 - rr) >= 0 ? rhs.dims->data[i - (5 - rr)] : 1;
    if (l != r && l != 1 && r != 1) return *why = "batch dimensions do not broadcast", false;
    if (l < 0 || r < 0) return *why = "negative dimension", false;
    g.lhs_dims[i] = l;
    g.weight_dims[i] = r;
    g.out_batches *= l == 1 ? r : l;
    const int64_t lhs_batches = static_cast<int64_t>(g.lhs_batches) * l;
    const int64_t matrices = static_cast<int64_t>(g.matrices) * r;
    if (lhs_batches > 0x7fffffff || matrices > 0x7fffffff || g.out_batches > 0x7fffffff) {
      return *why = "too many matrices", false;
    }
    g.lhs_batches = static_cast<int>(lhs_batches);
    g.matrices = static_cast<int>(matrices);
  }
  if (g.depth <= 0) return *why = "empty depth", false;
  *out = g;
  return true;
}

// BATCH_MATMUL in its hybrid form (batch_matmul.cc:363-374: float32 x int8): the right operand
// a constant int8 tensor with affine quantization, one scale or one per output unit.
FcKind ClassifyBatchMatMul(const TfLiteContext* ctx, const TfLiteNode* node,
                           const TfLiteRegistration* registration, const Options& opt,
                           std::string* why_not) {
  auto no = [&](const char* reason) {
    if (why_not) *why_not = reason;
    return FcKind::kNone;
  };
  if (!opt.claim_batch_matmul) return no("batch matmul disabled by option");
  if (registration->version > kMaxBatchMatMulVersion) return no("op version newer than 4");
  if (!node->builtin_data) return no("no builtin data");
  if (node->inputs->size != 2 || node->outputs->size != 1) return no("needs 2 inputs, 1 output");
  const auto* params = static_cast<const TfLiteBatchMatMulParams*>(node->builtin_data);
  const TfLiteTensor& lhs = ctx->tensors[node->inputs->data[0]];
  const TfLiteTensor& rhs = ctx->tensors[node->inputs->data[1]];
  const TfLiteTensor& output = ctx->tensors[node->outputs->data[0]];
  if (lhs.type != kTfLiteFloat32 || rhs.type != kTfLiteInt8 || output.type != kTfLiteFloat32) {
    return no("not the float32 x int8 form");
  }
  if (!lhs.dims || !rhs.dims) return no("operand has no shape");
  if (!IsConstant(rhs)) return no("right operand is not a constant tensor");
  if (rhs.quantization.type != kTfLiteAffineQuantization) return no("right operand not affine");
  BatchMatMulShape g;
  const char* why = "";
  if (!BatchMatMulGeometry(lhs, rhs, params->adj_x, params->adj_y, &g, &why)) return no(why);
  const auto* q = static_cast<const TfLiteAffineQuantization*>(rhs.quantization.params);
  if (!q || !q->scale || q->scale->size < 1) return no("right operand has no scales");
  if (q->scale->size > 1) {
    // EvalHybrid indexes the scales by output unit (batch_matmul.h:201-203).
    const int units_dim = params->adj_y ? rhs.dims->size - 2 : rhs.dims->size - 1;
    if (q->quantized_dimension != units_dim || q->scale->size != g.units) {
      return no("per-channel scales do not run along the output units");
    }
  }
  if (lrtfc_fc_int8_preferred_layout(1, g.depth, g.units, 0) != LRTFC_LAYOUT_PACKED) {
    return no("depth beyond what the kernels stage in LDS");
  }
  return FcKind::kBatchMatMul;
}

// The node-claim predicate: the same tensor / quantization-parameter / fused-activation
// combinations the builtin kernel accepts for these three paths
// (tflite/kernels/fully_connected.cc:254-308, 440-761), nothing else.
FcKind Classify(const TfLiteContext* ctx, const TfLiteNode* node,
                const TfLiteRegistration* registration, const Options& opt,
                std::string* why_not) {
  auto no = [&](const char* reason) {
    if (why_not) *why_not = reason;
    return FcKind::kNone;
  };
  if (registration->builtin_code == kTfLiteBuiltinEmbeddingLookup) {
    return ClassifyEmbeddingLookup(ctx, node, opt, why_not);
  }
  if (registration->builtin_code == kTfLiteBuiltinBatchMatmul) {
    return ClassifyBatchMatMul(ctx, node, registration, opt, why_not);
  }
  if (registration->builtin_code != kTfLiteBuiltinFullyConnected) return no("not FULLY_CONNECTED");
  if (registration->version > kMaxFcVersion) return no("op version newer than 14");
  if (!node->builtin_data) return no("no builtin data");
  const auto* params = static_cast<const TfLiteFullyConnectedParams*>(node->builtin_data);
  if (params->weights_format != kTfLiteFullyConnectedWeightsFormatDefault) {
    return no("shuffled weights format");
  }
  if (node->inputs->size != 2 && node->inputs->size != 3) return no("needs 2 or 3 inputs");
  if (node->outputs->size != 1) return no("needs exactly one output");
  const TfLiteTensor& input = ctx->tensors[node->inputs->data[0]];
  const TfLiteTensor& filter = ctx->tensors[node->inputs->data[1]];
  const TfLiteTensor* bias = OptionalInput(ctx, node, 2);
  const TfLiteTensor& output = ctx->tensors[node->outputs->data[0]];
  if (!filter.dims || filter.dims->size != 2) return no("filter is not rank 2");
  if (!IsConstant(filter)) return no("filter is not a constant tensor");
  if (filter.sparsity != nullptr) return no("sparse filter");
  if (bias && !IsConstant(*bias)) return no("bias is not a constant tensor");
  if (!input.dims || input.dims->size < 1) return no("input has no shape");
  const int out_depth = filter.dims->data[0];
  const int depth = filter.dims->data[1];
  if (bias && NumElements(bias->dims) != out_depth) return no("bias size != output channels");

  if (input.type == kTfLiteUInt8 && output.type == kTfLiteUInt8 && filter.type == kTfLiteUInt8) {
    // The legacy uint8 op (fully_connected.cc:1607-1626): per-tensor only, any zero points. It runs
    // on the int8 kernels with every tensor taken as value - 128 (PrepareNode, KernelInvoke).
    if (!opt.claim_int8) return no("int8 path disabled by option");
    if (!ClippingActivation(params->activation)) return no("activation not a clamp");
    if (bias && bias->type != kTfLiteInt32) return no("bias is not int32");
    if (input.quantization.type != kTfLiteAffineQuantization ||
        filter.quantization.type != kTfLiteAffineQuantization) {
      return no("input/filter lack affine quantization");
    }
    const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
    if (!fq || !fq->scale || fq->scale->size != 1) return no("uint8 filter is not per-tensor");
    if (output.params.scale <= 0.0f || input.params.scale <= 0.0f) return no("missing scales");
    return FcKind::kInt8;
  }
  if (input.type == kTfLiteInt8 && output.type == kTfLiteInt8 &&
      (filter.type == kTfLiteInt8 || filter.type == kTfLiteInt4 || filter.type == kTfLiteInt2)) {
    if (!opt.claim_int8) return no("int8 path disabled by option");
    if (!ClippingActivation(params->activation)) return no("activation not a clamp");
    if (bias && bias->type != kTfLiteInt32) return no("bias is not int32");
    if (input.quantization.type != kTfLiteAffineQuantization ||
        filter.quantization.type != kTfLiteAffineQuantization) {
      return no("input/filter lack affine quantization");
    }
    const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
    if (!fq || !fq->scale || fq->scale->size < 1) return no("filter has no scales");
    if (fq->scale->size > 1) {
      if (fq->quantized_dimension != 0) return no("quantized_dimension != 0");
      if (fq->scale->size != out_depth) return no("scale count != output channels");
    }
    if (fq->zero_point) {
      const bool per_channel = fq->scale->size > 1;
      for (int i = 0; i < fq->zero_point->size; ++i) {
        // Int4 and Int2 filters: Prepare insists on zero points of 0 (fully_connected.cc:754-759).
        if ((per_channel || filter.type == kTfLiteInt4 || filter.type == kTfLiteInt2) &&
            fq->zero_point->data[i] != 0) {
          return no("non-zero filter zero point");
        }
      }
    }
    if (output.params.scale <= 0.0f || input.params.scale <= 0.0f) return no("missing scales");
    return FcKind::kInt8;
  }

  if (input.type == kTfLiteFloat32 && output.type == kTfLiteFloat32) {
    if (bias && bias->type != kTfLiteFloat32) return no("bias is not float32");
    if (filter.type == kTfLiteInt8) {
      if (!opt.claim_hybrid) return no("hybrid path disabled by option");
      // The hybrid path accepts every fused activation (fully_connected.cc:748-753); tanh and
      // sigmoid go through Eigen in the reference (no bit-level contract) and are left to the
      // CPU. The sign bit is exact.
      if (!ClippingActivation(params->activation) && params->activation != kTfLiteActSignBit) {
        return no("activation is tanh or sigmoid");
      }
      if (filter.quantization.type != kTfLiteAffineQuantization) return no("filter not affine");
      const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
      if (!fq || !fq->scale || fq->scale->size < 1) return no("filter has no scales");
      if (fq->scale->size > 1 && (fq->quantized_dimension != 0 || fq->scale->size != out_depth)) {
        return no("per-channel scales do not match output channels");
      }
      if (depth == 0) return no("empty depth");
      return FcKind::kHybrid;
    }
    if (filter.type == kTfLiteInt2 && filter.quantization.type == kTfLiteAffineQuantization) {
      // An Int2 filter under float activations: the builtin unpacks it to int8 on every Eval and
      // runs EvalHybridDense on the result (fully_connected.cc:812-818). Here: unpacked once at
      // prepare, then the int8 hybrid path.
      if (!opt.claim_hybrid) return no("hybrid path disabled by option");
      if (!ClippingActivation(params->activation) && params->activation != kTfLiteActSignBit) {
        return no("activation is tanh or sigmoid");
      }
      const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
      if (!fq || !fq->scale || fq->scale->size < 1) return no("filter has no scales");
      if (fq->scale->size > 1 && (fq->quantized_dimension != 0 || fq->scale->size != out_depth)) {
        return no("per-channel scales do not match output channels");
      }
      if (fq->zero_point) {
        for (int i = 0; i < fq->zero_point->size; ++i) {
          if (fq->zero_point->data[i] != 0) return no("non-zero filter zero point");
        }
      }
      if (depth == 0) return no("empty depth");
      return FcKind::kHybrid;
    }
    if (filter.type == kTfLiteInt4 && filter.quantization.type == kTfLiteBlockwiseQuantization) {
      if (!opt.claim_int4_blockwise) return no("int4 blockwise path disabled by option");
      // Gate of the builtin's 4-bit path (fully_connected.cc:609-633): even depth,
      // at least 4 output channels and 32 of depth.
      if (depth % 2 != 0 || out_depth < 4 || depth < 32) return no("shape outside 4-bit gate");
      const auto* bq = static_cast<const TfLiteBlockwiseQuantization*>(filter.quantization.params);
      if (!bq || bq->blocksize <= 0 || depth % bq->blocksize != 0) return no("bad blocksize");
      if (bq->scale < 0 || static_cast<size_t>(bq->scale) >= ctx->tensors_size) {
        return no("scale tensor index out of range");
      }
      const TfLiteTensor& scales = ctx->tensors[bq->scale];
      if (scales.type != kTfLiteFloat16 || !IsConstant(scales)) return no("scales not const fp16");
      if (NumElements(scales.dims) != static_cast<int64_t>(out_depth) * (depth / bq->blocksize)) {
        return no("scale count != channels x blocks");
      }
      return FcKind::kInt4Blockwise;
    }
    if (filter.type == kTfLiteInt4 && filter.quantization.type == kTfLiteAffineQuantization) {
      // The builtin's optimized 4-bit path (EvalHybridDense4Bit) inside its gate, the ordinary
      // hybrid kernels on the unpacked filter outside it.
      if (!opt.claim_int4_per_channel) return no("int4 per-channel path disabled by option");
      if (!ClippingActivation(params->activation) && params->activation != kTfLiteActSignBit) {
        return no("activation is tanh or sigmoid");
      }
      const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
      if (!fq || !fq->scale || fq->scale->size < 1) return no("filter has no scales");
      if (fq->scale->size > 1 && (fq->quantized_dimension != 0 || fq->scale->size != out_depth)) {
        return no("per-channel scales do not match output channels");
      }
      if (depth % 2 != 0 || out_depth < 4 || depth < 32) {
        // Outside the gate of the 4-bit path (fully_connected.cc:609-613) the builtin unpacks the
        // nibbles to int8 on every Eval and runs the ordinary hybrid kernels on them
        // (EvalHybridDense, fully_connected.cc:805-814). Here: unpacked once at prepare, then the
        // int8 hybrid path.
        if (!opt.claim_hybrid) return no("hybrid path disabled by option");
        if (depth == 0) return no("empty depth");
        return FcKind::kHybrid;
      }
      // Both kernels of this path stage a whole activation row in LDS; rows too deep for that
      // are declined here rather than failing at invoke.
      if (lrtfc_fc_int8_preferred_layout(1, depth, out_depth, 0) != LRTFC_LAYOUT_PACKED) {
        return no("depth beyond what the 4-bit path kernels stage in LDS");
      }
      return FcKind::kHybridInt4;
    }
    return no("float activations with this filter type are left to the CPU kernels");
  }
  return no("tensor type combination not handled");
}

// ---- device memory ---------------------------------------------------------------

class DeviceBuffer {
 public:
  DeviceBuffer() = default;
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  DeviceBuffer(DeviceBuffer&& o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) {
    o.ptr_ = nullptr;
    o.bytes_ = 0;
  }
  ~DeviceBuffer() { Release(); }
  void Release() {
    if (ptr_) (void)hipFree(ptr_);
    ptr_ = nullptr;
    bytes_ = 0;
  }
  hipError_t Ensure(size_t bytes) {
    if (bytes <= bytes_) return hipSuccess;
    Release();
    hipError_t err = hipMalloc(&ptr_, bytes);
    if (err == hipSuccess) bytes_ = bytes;
    return err;
  }
  hipError_t Upload(const void* host, size_t bytes, hipStream_t stream) {
    hipError_t err = Ensure(bytes);
    if (err != hipSuccess || bytes == 0) return err;
    return hipMemcpyAsync(ptr_, host, bytes, hipMemcpyHostToDevice, stream);
  }
  template <typename T>
  T* as() const {
    return static_cast<T*>(ptr_);
  }
  void* get() const { return ptr_; }
  size_t bytes() const { return bytes_; }

 private:
  void* ptr_ = nullptr;
  size_t bytes_ = 0;
};

// Page-locked host memory (allocated, never registered): the staging area through which a
// partition's inputs and outputs cross PCIe in one copy each.
class PinnedBuffer {
 public:
  PinnedBuffer() = default;
  PinnedBuffer(const PinnedBuffer&) = delete;
  PinnedBuffer& operator=(const PinnedBuffer&) = delete;
  ~PinnedBuffer() { Release(); }
  void Release() {
    if (ptr_) (void)hipHostFree(ptr_);
    ptr_ = nullptr;
    bytes_ = 0;
  }
  hipError_t Ensure(size_t bytes) {
    if (bytes <= bytes_) return hipSuccess;
    Release();
    hipError_t err = hipHostMalloc(&ptr_, bytes, hipHostMallocDefault);
    if (err == hipSuccess) bytes_ = bytes;
    return err;
  }
  uint8_t* get() const { return static_cast<uint8_t*>(ptr_); }

 private:
  void* ptr_ = nullptr;
  size_t bytes_ = 0;
};

struct FcNode {
  int node_index = -1;
  FcKind kind = FcKind::kNone;
  int input = -1, filter = -1, bias = -1, output = -1, scales = -1;
  TfLiteFullyConnectedParams params{};
  int batches = 0, depth = 0, out_depth = 0, blocksize = 0;
  bool per_channel = false;
  float filter_scale = 1.0f;
  int32_t input_offset = 0, filter_offset = 0, output_offset = 0, act_min = 0, act_max = 0;
  // A uint8 node: its rows and its result pass through these as int8 (value - 128).
  bool uint8_io = false;
  DeviceBuffer u8_rows_dev, u8_result_dev;
  const void* uploaded_filter = nullptr;  // host pointer the device copies were made from
  // The filter lives on the device in the layout the node's shape runs fastest on: the
  // model's own (row-major / nibble-packed rows) or the re-tiled copy. Only one is kept.
  bool have_model_layout = false, have_retiled = false, use_retiled = false;
  // Per-channel int4 hybrid nodes keep the filter at 4 bits per weight for decode batches
  // (retiled_dev then holds nibble tiles) and as re-tiled int8 for prefill batches.
  bool nibble_layout = false, have_nibbles = false;
  // Blockwise-int4 nodes run prefill batches on the filter re-tiled for the matrix-core GEMM
  // (retiled_dev then holds that form) and decode batches on the streaming form.
  bool gemm_layout = false, have_gemm = false;
  // ... and batches in between on the GEMM that keeps the filter at 4 bits per weight
  // (gemm_layout is set too; retiled_dev then holds that form).
  bool gemm_nibbles = false;
  // A member of a grouped launch whose shape runs faster on the 4-bit-resident matrix-core form
  // (lrtfc_int4_group_preferred_form) keeps that form of its filter here, beside the decode
  // tiling that the same node needs when a resize changes the group's batch count.
  DeviceBuffer group_nibbles_dev;
  const void* group_nibbles_from = nullptr;  // host filter the copy was made from
  bool split_quantize = false;  // quantize rows in a launch of their own, not in the prologue
  // EMBEDDING_LOOKUP nodes: input = the lookup vector, filter = the table (filter_dev), batches =
  // lookups, depth = out_depth = columns of a row; block scales in scales_dev or per-row scales
  // in pcs_dev; status_slot = the node's place in PartitionKernel::lookup_status.
  int table_rows = 0, value_bits = 0, status_slot = -1;
  bool out_f16 = false;
  // BATCH_MATMUL nodes: input = the float operand, filter = the int8 one; batches = rows of one
  // matrix product, out_depth = output units; retiled_dev holds `matrices` re-tiled weight
  // matrices one after another, row_sums_dev their row sums.
  int lhs_batches = 1, matrices = 1;
  bool adj_x = false, adj_y = false;
  int lhs_dims[3] = {1, 1, 1}, weight_dims[3] = {1, 1, 1};
  // Scheduling inside the partition: the stream the node runs on, the node that produces its
  // input (-1: the input is uploaded from the host), and whether a node on another stream
  // waits for this one.
  int lane = 0, producer = -1;
  bool signal = false;
  // Grouped launch (several independent int4 nodes of one depth in one kernel): index into
  // PartitionKernel::groups, or -1.
  int group = -1;
  DeviceBuffer filter_dev, retiled_dev, bias_dev, mult_dev, shift_dev, row_sums_dev, pcs_dev,
      scales_dev, kfsum_dev;
};

// Rows above which the fused kernels' prologue (every workgroup quantizes every row) costs
// more than a separate quantization launch; deep int4 rows fuse at most two batch rows.
constexpr int kInt4FusedMaxDepth = 4096;
constexpr int kInt4DeepFusedMaxBatches = 2;
// Up to this many rows a per-channel int4 node streams its filter as nibbles (one pass per 16
// rows); above, the MFMA GEMM on the int8 expansion streams it once.
constexpr int kInt4PerChannelNibbleMaxBatches = 32;

// Up to this many bytes of host outputs per partition are written by the kernels directly into
// page-locked host memory instead of being copied there afterwards. The invariant this rests on:
// a kernel writes every element of its output exactly once and never reads it (no atomics, no
// zero-fill-then-accumulate, no split-depth partial sums parked in the output); anything else
// would run its read-modify-write over PCIe against host memory. It holds for the kernels the
// node kinds below launch today; a new kind, or a kernel form that breaks it, must stay out of
// the list and take the copy-out path.
constexpr size_t kDirectOutputMaxBytes = 16 << 20;
// Up to this many bytes of host inputs per partition are read by the kernels straight from
// page-locked host memory, when every node that reads them is decode-shaped (a row is then
// fetched a handful of times, not once per tile of a GEMM).
constexpr size_t kDirectInputMaxBytes = 64 << 10;
constexpr int kDirectInputMaxBatches = 16;

bool WritesOutputOnce(FcKind kind) {
  switch (kind) {
    case FcKind::kInt8:
    case FcKind::kHybrid:
    case FcKind::kInt4Blockwise:
    case FcKind::kHybridInt4:
    case FcKind::kEmbeddingLookup:
    case FcKind::kBatchMatMul:
      return true;
    default:
      return false;
  }
}

struct PartitionKernel {
  DelegateState* state = nullptr;
  std::vector<FcNode> nodes;
  // Device homes of the activation tensors: one arena laid out at prepare, the uploaded
  // tensors first, then the downloaded ones, then those that never leave the device. The two
  // outer regions each cross PCIe in ONE copy per invoke, through page-locked staging.
  DeviceBuffer arena;
  std::map<int, size_t> arena_offset;  // tensor index -> byte offset in the arena
  size_t upload_bytes = 0, download_offset = 0, download_bytes = 0;
  PinnedBuffer upload_stage, download_stage;
  // A boundary tensor (uploaded or downloaded) that carries a buffer handle of this delegate
  // lives in the registered memory itself for as long as the binding lasts: the kernels read and
  // write it there. `bindings` is the device address each boundary tensor had at the last
  // invoke (uploads, then downloads; nullptr = not bound or not usable in place).
  std::map<int, void*> alias;
  std::vector<void*> bindings;
  // Small sets of host outputs are written by the kernels straight into the page-locked
  // download staging area (device-visible host memory), which saves the copy command behind the
  // last kernel: direct_outputs, decided at prepare, holds when no node of the partition reads
  // any of the downloaded tensors back.
  bool direct_outputs = false;
  uint8_t* download_stage_device = nullptr;  // the staging area as the device addresses it
  // The mirror image for small sets of host inputs (decode rows): the kernels read them straight
  // from the page-locked upload staging area, which saves the copy command ahead of the first
  // kernel. A row is read once per workgroup and the device's L2 serves all but the first read;
  // what it costs is one round trip over PCIe inside the kernel's prologue instead of a copy
  // command and its launch gap in front of the kernel.
  bool direct_inputs = false;
  uint8_t* upload_stage_device = nullptr;
  void* Activation(int tensor) const {
    auto bound = alias.find(tensor);
    if (bound != alias.end()) return bound->second;
    auto it = arena_offset.find(tensor);
    if (it == arena_offset.end()) return nullptr;
    if (direct_inputs && it->second < upload_bytes) return upload_stage_device + it->second;
    if (direct_outputs && it->second >= download_offset &&
        it->second < download_offset + download_bytes) {
      return download_stage_device + (it->second - download_offset);
    }
    return arena.as<uint8_t>() + it->second;
  }
  // The word an invoke polls for its own serial number (Options::poll_completion).
  PinnedBuffer completion;
  uint32_t* completion_dev = nullptr;
  uint32_t completion_serial = 0;
  // Three int32 per EMBEDDING_LOOKUP node, in page-locked host memory the lookup kernels write
  // straight into: {0 or 1, first offending position, the index found there}.
  PinnedBuffer lookup_status;
  int32_t* lookup_status_dev = nullptr;
  int lookup_nodes = 0;
  std::vector<int> uploads;                 // activation tensors read from the host each invoke
  std::vector<int> downloads;               // tensors written back to the host each invoke
  // Nodes that do not depend on each other (the q/k/v or gate/up projections of a decoder
  // layer, say) run on different streams so that their launch and prologue latencies overlap;
  // a chain of dependent nodes stays on one stream. All streams have the default priority.
  static constexpr int kMaxStreams = 4;
  int num_streams = 1;
  hipStream_t streams[kMaxStreams] = {};
  hipStream_t stream = nullptr;  // streams[0]: uploads, downloads, prepare-time work
  DeviceBuffer workspace[kMaxStreams];
  hipEvent_t upload_done = nullptr;
  hipEvent_t metrics_begin = nullptr, metrics_end = nullptr;  // timing events, made on first use
  hipEvent_t lane_done[kMaxStreams] = {};
  std::vector<hipEvent_t> node_done;  // per node; only the signalling ones are created
  bool lane_used[kMaxStreams] = {};
  struct Unit {
    int level;  // distance from the partition's inputs
    int first;  // node index (of the group's first member)
    int group;  // index into groups, or -1 for a node on its own
  };
  std::vector<Unit> order;  // launch order
  struct Group {
    std::vector<int> members;  // node indices, ascending
    DeviceBuffer table;
    DeviceBuffer workspace;  // one activation workspace per member when rows exceed two
    lrtfc_int4_group_launch launch{};
  };
  std::vector<Group> groups;
  // What TfLiteRegistration::profiling_string reports for this partition (built at prepare).
  std::string profile_text;
  ~PartitionKernel() {
    for (hipEvent_t e : node_done) {
      if (e) (void)hipEventDestroy(e);
    }
    if (upload_done) (void)hipEventDestroy(upload_done);
    if (metrics_begin) (void)hipEventDestroy(metrics_begin);
    if (metrics_end) (void)hipEventDestroy(metrics_end);
    for (int i = 0; i < kMaxStreams; ++i) {
      if (lane_done[i]) (void)hipEventDestroy(lane_done[i]);
      if (streams[i]) (void)hipStreamDestroy(streams[i]);
    }
  }
};

#define RETURN_IF_HIP(ctx, expr)                                                          \
  do {                                                                                    \
    const hipError_t e__ = (expr);                                                        \
    if (e__ != hipSuccess) {                                                              \
      (ctx)->ReportError((ctx), "litert_amd delegate: %s failed: %s", #expr,             \
                         hipGetErrorString(e__));                                         \
      return kTfLiteError;                                                                \
    }                                                                                     \
  } while (0)

#define RETURN_IF_FC(ctx, expr)                                                           \
  do {                                                                                    \
    const int rc__ = (expr);                                                              \
    if (rc__ != LRTFC_OK) {                                                               \
      (ctx)->ReportError((ctx), "litert_amd delegate: %s", lrtfc_last_error());          \
      return kTfLiteError;                                                                \
    }                                                                                     \
  } while (0)

// ---- kernel registration callbacks -----------------------------------------------------

void* KernelInit(TfLiteContext* ctx, const char* buffer, size_t /*length*/) {
  const auto* params = reinterpret_cast<const TfLiteDelegateParams*>(buffer);
  if (!params || !params->delegate || !params->nodes_to_replace) return reinterpret_cast<void*>(-1);
  auto* state = static_cast<DelegateState*>(params->delegate->data_);
  auto kernel = std::make_unique<PartitionKernel>();
  kernel->state = state;
  kernel->num_streams = state->options.streams;
  bool streams_ok = hipSetDevice(state->options.device) == hipSuccess;
  for (int i = 0; streams_ok && i < kernel->num_streams; ++i) {
    streams_ok = hipStreamCreate(&kernel->streams[i]) == hipSuccess &&
                 hipEventCreateWithFlags(&kernel->lane_done[i], hipEventDisableTiming) == hipSuccess;
  }
  streams_ok = streams_ok &&
               hipEventCreateWithFlags(&kernel->upload_done, hipEventDisableTiming) == hipSuccess;
  if (!streams_ok) {
    ctx->ReportError(ctx, "litert_amd delegate: cannot create HIP streams on device %d",
                     state->options.device);
    return reinterpret_cast<void*>(-1);  // TfLiteKernelInitFailed(), tflite/core/c/common.cc:867
  }
  kernel->stream = kernel->streams[0];
  std::map<int, bool> produced;
  for (int i = 0; i < params->nodes_to_replace->size; ++i) {
    const int node_index = params->nodes_to_replace->data[i];
    TfLiteNode* node = nullptr;
    TfLiteRegistration* reg = nullptr;
    if (ctx->GetNodeAndRegistration(ctx, node_index, &node, &reg) != kTfLiteOk) {
      return reinterpret_cast<void*>(-1);
    }
    std::string why;
    const FcKind kind = Classify(ctx, node, reg, state->options, &why);
    if (kind == FcKind::kNone) {
      ctx->ReportError(ctx, "litert_amd delegate: node %d handed to the kernel is unsupported: %s",
                       node_index, why.c_str());
      return reinterpret_cast<void*>(-1);
    }
    FcNode n;
    n.node_index = node_index;
    n.kind = kind;
    n.input = node->inputs->data[0];
    n.filter = node->inputs->data[1];
    n.bias = (kind != FcKind::kEmbeddingLookup && kind != FcKind::kBatchMatMul &&
              node->inputs->size == 3)
                 ? node->inputs->data[2]
                 : kTfLiteOptionalTensor;
    n.output = node->outputs->data[0];
    if (kind == FcKind::kBatchMatMul) {
      const auto* bp = static_cast<const TfLiteBatchMatMulParams*>(node->builtin_data);
      n.adj_x = bp->adj_x;
      n.adj_y = bp->adj_y;
      n.params.asymmetric_quantize_inputs = bp->asymmetric_quantize_inputs;
    } else if (kind != FcKind::kEmbeddingLookup) {
      n.params = *static_cast<const TfLiteFullyConnectedParams*>(node->builtin_data);
    }
    if (!produced.count(n.input)) {
      bool listed = false;
      for (int t : kernel->uploads) listed = listed || (t == n.input);
      if (!listed) kernel->uploads.push_back(n.input);
    }
    produced[n.output] = true;
    kernel->nodes.push_back(std::move(n));
  }
  {
    std::map<int, int> producer_of;  // tensor -> node that writes it
    for (size_t i = 0; i < kernel->nodes.size(); ++i) {
      FcNode& n = kernel->nodes[i];
      auto it = producer_of.find(n.input);
      n.producer = it == producer_of.end() ? -1 : it->second;
      producer_of[n.output] = static_cast<int>(i);
    }
  }
  // Every tensor the runtime lists as an output of the partition goes back to the host.
  for (int i = 0; i < params->output_tensors->size; ++i) {
    kernel->downloads.push_back(params->output_tensors->data[i]);
  }
  return kernel.release();
}

void KernelFree(TfLiteContext* /*ctx*/, void* buffer) {
  if (buffer && buffer != reinterpret_cast<void*>(-1)) delete static_cast<PartitionKernel*>(buffer);
}

// The workspace of lrtfc_activation_workspace_bytes(batches, depth) bytes, carved as the
// library carves it: quantized rows, then scaling factors, then zero points, each region
// starting on a 256-byte boundary.
struct ActivationScratch {
  int8_t* q;
  float* sf;
  int32_t* zp;
};

ActivationScratch SplitScratch(void* workspace, int batches, int depth) {
  auto round_up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
  auto* base = static_cast<uint8_t*>(workspace);
  ActivationScratch w;
  w.q = reinterpret_cast<int8_t*>(base);
  const size_t q_bytes = round_up(static_cast<size_t>(batches) * depth);
  w.sf = reinterpret_cast<float*>(base + q_bytes);
  w.zp = reinterpret_cast<int32_t*>(base + q_bytes + round_up(static_cast<size_t>(batches) * 4));
  return w;
}

#define RETURN_IF_OK(expr)                      \
  do {                                          \
    const TfLiteStatus st__ = (expr);           \
    if (st__ != kTfLiteOk) return st__;         \
  } while (0)

// Makes the re-tiled copy of an int8 filter from the row-major one and drops the latter.
TfLiteStatus RetileInt8(TfLiteContext* ctx, FcNode* n, hipStream_t s) {
  RETURN_IF_HIP(ctx, n->retiled_dev.Ensure(lrtfc_packed_int8_filter_bytes(n->out_depth, n->depth)));
  RETURN_IF_FC(ctx, lrtfc_pack_int8_filter(n->filter_dev.as<int8_t>(), n->out_depth, n->depth,
                                           n->retiled_dev.as<int8_t>(), s));
  RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
  n->have_retiled = true;
  n->filter_dev.Release();
  n->have_model_layout = false;
  return kTfLiteOk;
}

// EMBEDDING_LOOKUP: shapes as embedding_lookup.cc:49-100 leaves them (output = lookups x the
// table's row shape), the table and its scales uploaded once.
TfLiteStatus PrepareLookupNode(TfLiteContext* ctx, PartitionKernel* k, FcNode* n) {
  const TfLiteTensor& lookup = ctx->tensors[n->input];
  const TfLiteTensor& value = ctx->tensors[n->filter];
  const TfLiteTensor& output = ctx->tensors[n->output];
  n->table_rows = value.dims->data[0];
  int64_t cols = 1;
  for (int i = 1; i < value.dims->size; ++i) cols *= value.dims->data[i];
  n->depth = n->out_depth = static_cast<int>(cols);
  n->batches = static_cast<int>(NumElements(lookup.dims));
  n->value_bits = value.type == kTfLiteInt4 ? 4 : 8;
  n->out_f16 = output.type == kTfLiteFloat16;
  n->use_retiled = true;  // no activation workspace, no grouping
  if (NumElements(output.dims) != static_cast<int64_t>(n->batches) * cols) {
    ctx->ReportError(ctx, "litert_amd delegate: node %d output shape does not hold %d x %lld values",
                     n->node_index, n->batches, static_cast<long long>(cols));
    return kTfLiteError;
  }
  hipStream_t s = k->stream;
  n->blocksize = 0;
  n->per_channel = false;
  n->filter_scale = value.params.scale;
  const bool fresh = n->uploaded_filter != value.data.raw;
  if (value.quantization.type == kTfLiteBlockwiseQuantization) {
    const auto* bq = static_cast<const TfLiteBlockwiseQuantization*>(value.quantization.params);
    n->blocksize = bq->blocksize;
    n->scales = bq->scale;
    const TfLiteTensor& scales = ctx->tensors[bq->scale];
    if (fresh) {
      RETURN_IF_HIP(ctx, n->scales_dev.Upload(scales.data.raw,
                                              static_cast<size_t>(NumElements(scales.dims)) * 2, s));
    }
  } else if (value.quantization.type == kTfLiteAffineQuantization) {
    const auto* q = static_cast<const TfLiteAffineQuantization*>(value.quantization.params);
    n->per_channel = q->scale->size > 1;  // one scale per row, embedding_lookup.cc:376-383
    if (n->per_channel && fresh) {
      RETURN_IF_HIP(ctx, n->pcs_dev.Upload(q->scale->data, static_cast<size_t>(n->table_rows) * 4, s));
    }
  }
  if (fresh && value.bytes > 0) {
    RETURN_IF_HIP(ctx, n->filter_dev.Upload(value.data.raw, value.bytes, s));
    RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
  }
  n->have_model_layout = true;
  n->uploaded_filter = value.data.raw;
  return kTfLiteOk;
}

// BATCH_MATMUL: the constant int8 operand is put into [matrix][unit][depth] order on the host
// (the op transposes it once as well, batch_matmul.cc:776-782), uploaded, reduced to row sums
// and re-tiled matrix by matrix.
TfLiteStatus PrepareBatchMatMulNode(TfLiteContext* ctx, PartitionKernel* k, FcNode* n) {
  const TfLiteTensor& lhs = ctx->tensors[n->input];
  const TfLiteTensor& rhs = ctx->tensors[n->filter];
  const TfLiteTensor& output = ctx->tensors[n->output];
  BatchMatMulShape g;
  const char* why = "";
  if (!BatchMatMulGeometry(lhs, rhs, n->adj_x, n->adj_y, &g, &why)) {
    ctx->ReportError(ctx, "litert_amd delegate: node %d: %s", n->node_index, why);
    return kTfLiteError;
  }
  n->lhs_batches = g.lhs_batches;
  n->matrices = g.matrices;
  std::copy(g.lhs_dims, g.lhs_dims + 3, n->lhs_dims);
  std::copy(g.weight_dims, g.weight_dims + 3, n->weight_dims);
  n->batches = g.rows;
  n->depth = g.depth;
  n->out_depth = g.units;
  const int64_t out_batches = g.out_batches;
  if (NumElements(output.dims) != out_batches * g.rows * g.units) {
    ctx->ReportError(ctx, "litert_amd delegate: node %d output shape does not hold %lld x %d x %d values",
                     n->node_index, static_cast<long long>(out_batches), g.rows, g.units);
    return kTfLiteError;
  }
  const auto* q = static_cast<const TfLiteAffineQuantization*>(rhs.quantization.params);
  n->per_channel = q->scale->size > 1;
  n->filter_scale = rhs.params.scale;
  n->use_retiled = true;
  n->split_quantize = true;  // rows are always quantized by a launch of their own
  hipStream_t s = k->stream;
  if (n->uploaded_filter == rhs.data.raw && n->have_retiled) return kTfLiteOk;
  const size_t matrix = static_cast<size_t>(g.units) * g.depth;
  const size_t total = matrix * g.matrices;
  if (total == 0) return kTfLiteOk;
  std::vector<int8_t> ordered;
  const int8_t* src = reinterpret_cast<const int8_t*>(rhs.data.raw);
  if (!n->adj_y) {  // [.., depth, units] -> [.., units, depth]
    ordered.resize(total);
    for (int m = 0; m < g.matrices; ++m) {
      for (int d = 0; d < g.depth; ++d) {
        for (int u = 0; u < g.units; ++u) {
          ordered[m * matrix + static_cast<size_t>(u) * g.depth + d] =
              src[m * matrix + static_cast<size_t>(d) * g.units + u];
        }
      }
    }
    src = ordered.data();
  }
  RETURN_IF_HIP(ctx, n->filter_dev.Upload(src, total, s));
  RETURN_IF_HIP(ctx, hipStreamSynchronize(s));  // `ordered` is a local
  const size_t packed_bytes = lrtfc_packed_int8_filter_bytes(g.units, g.depth);
  RETURN_IF_HIP(ctx, n->retiled_dev.Ensure(packed_bytes * g.matrices));
  RETURN_IF_HIP(ctx, n->row_sums_dev.Ensure(static_cast<size_t>(g.matrices) * g.units * 4));
  for (int m = 0; m < g.matrices; ++m) {
    const int8_t* w = n->filter_dev.as<int8_t>() + m * matrix;
    RETURN_IF_FC(ctx, lrtfc_row_sums_int8(w, g.units, g.depth,
                                          n->row_sums_dev.as<int32_t>() + static_cast<size_t>(m) * g.units, s));
    RETURN_IF_FC(ctx, lrtfc_pack_int8_filter(w, g.units, g.depth,
                                             n->retiled_dev.as<int8_t>() + m * packed_bytes, s));
  }
  if (n->per_channel) {
    RETURN_IF_HIP(ctx, n->pcs_dev.Upload(q->scale->data, static_cast<size_t>(g.units) * 4, s));
  }
  RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
  n->filter_dev.Release();  // only the re-tiled matrices are kept
  n->have_retiled = true;
  n->uploaded_filter = rhs.data.raw;
  return kTfLiteOk;
}

TfLiteStatus PrepareNode(TfLiteContext* ctx, PartitionKernel* k, FcNode* n) {
  if (n->kind == FcKind::kEmbeddingLookup) return PrepareLookupNode(ctx, k, n);
  if (n->kind == FcKind::kBatchMatMul) return PrepareBatchMatMulNode(ctx, k, n);
  const TfLiteTensor& input = ctx->tensors[n->input];
  const TfLiteTensor& filter = ctx->tensors[n->filter];
  const TfLiteTensor* bias = n->bias == kTfLiteOptionalTensor ? nullptr : &ctx->tensors[n->bias];
  const TfLiteTensor& output = ctx->tensors[n->output];
  n->out_depth = filter.dims->data[0];
  n->depth = filter.dims->data[1];
  const int64_t in_elems = NumElements(input.dims);
  n->batches = n->depth > 0 ? static_cast<int>(in_elems / n->depth) : 0;
  if (n->depth > 0 && static_cast<int64_t>(n->batches) * n->depth != in_elems) {
    ctx->ReportError(ctx, "litert_amd delegate: node %d input size %lld is not a multiple of depth %d",
                     n->node_index, static_cast<long long>(in_elems), n->depth);
    return kTfLiteError;
  }
  if (n->depth > 0 && NumElements(output.dims) != static_cast<int64_t>(n->batches) * n->out_depth) {
    ctx->ReportError(ctx, "litert_amd delegate: node %d output shape does not hold %d x %d values",
                     n->node_index, n->batches, n->out_depth);
    return kTfLiteError;
  }
  hipStream_t s = k->stream;
  if (n->uploaded_filter != filter.data.raw) {
    n->have_model_layout = n->have_retiled = n->have_nibbles = n->have_gemm = false;
  }
  const size_t weights = static_cast<size_t>(n->out_depth) * n->depth;

  if (n->kind == FcKind::kInt8) {
    const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
    n->per_channel = fq->scale->size > 1;
    // uint8 tensors are handled as int8, value - 128: every zero point moves down with them, and
    // each term (w - zw)(x - zx), the multiplier and the clamped result stay what they were.
    n->uint8_io = input.type == kTfLiteUInt8;
    const int32_t moved = n->uint8_io ? 128 : 0;
    n->input_offset = -(input.params.zero_point - moved);
    n->filter_offset = n->per_channel ? 0 : -(filter.params.zero_point - moved);
    n->output_offset = output.params.zero_point - moved;
    std::vector<int32_t> mult(n->per_channel ? n->out_depth : 1), shift(mult.size());
    if (n->per_channel) {
      RETURN_IF_FC(ctx, lrtfc_prepare_per_channel(input.params.scale, fq->scale->data,
                                                  n->out_depth, output.params.scale, mult.data(),
                                                  shift.data()));
    } else {
      // GetQuantizedConvolutionMultipler reads the per-tensor params.scale fields.
      RETURN_IF_FC(ctx, lrtfc_prepare_per_tensor(input.params.scale, filter.params.scale,
                                                 bias != nullptr, bias ? bias->params.scale : 0.0f,
                                                 output.params.scale, &mult[0], &shift[0]));
    }
    RETURN_IF_FC(ctx, lrtfc_activation_range_int8(n->params.activation, output.params.scale,
                                                  output.params.zero_point - moved, &n->act_min,
                                                  &n->act_max));
    if (n->uint8_io) {
      RETURN_IF_HIP(ctx, n->u8_rows_dev.Ensure(static_cast<size_t>(n->batches) * n->depth));
      RETURN_IF_HIP(ctx, n->u8_result_dev.Ensure(static_cast<size_t>(n->batches) * n->out_depth));
    }
    RETURN_IF_HIP(ctx, n->mult_dev.Upload(mult.data(), mult.size() * 4, s));
    RETURN_IF_HIP(ctx, n->shift_dev.Upload(shift.data(), shift.size() * 4, s));
    RETURN_IF_HIP(ctx, hipStreamSynchronize(s));  // mult/shift are stack-owned
    n->use_retiled = weights > 0 &&
                     lrtfc_fc_int8_preferred_layout(n->batches, n->depth, n->out_depth,
                                                    n->filter_offset) == LRTFC_LAYOUT_PACKED;
    if (weights > 0 && !(n->use_retiled ? n->have_retiled : n->have_model_layout)) {
      if (!n->have_model_layout) {
        if (filter.type == kTfLiteInt4) {
          // Unpacked once here; the builtin unpacks on every Eval (fully_connected.cc:1670-1677).
          DeviceBuffer packed;
          RETURN_IF_HIP(ctx, packed.Upload(filter.data.raw, (weights + 1) / 2, s));
          RETURN_IF_HIP(ctx, n->filter_dev.Ensure(weights));
          RETURN_IF_FC(ctx, lrtfc_unpack_int4(packed.as<uint8_t>(), static_cast<int64_t>(weights),
                                              n->filter_dev.as<int8_t>(), s));
          RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        } else if (filter.type == kTfLiteInt2) {
          // Four values per byte over the flat tensor (fully_connected.cc:812-818, 1678-1685).
          DeviceBuffer packed;
          RETURN_IF_HIP(ctx, packed.Upload(filter.data.raw, (weights + 3) / 4, s));
          RETURN_IF_HIP(ctx, n->filter_dev.Ensure(weights));
          RETURN_IF_FC(ctx, lrtfc_unpack_int2(packed.as<uint8_t>(), static_cast<int64_t>(weights),
                                              n->filter_dev.as<int8_t>(), s));
          RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        } else {
          RETURN_IF_HIP(ctx, n->filter_dev.Upload(filter.data.raw, weights, s));
          if (n->uint8_io) {
            RETURN_IF_FC(ctx, lrtfc_xor_sign_bit(n->filter_dev.as<uint8_t>(),
                                                 n->filter_dev.as<uint8_t>(), weights, s));
          }
        }
        RETURN_IF_HIP(ctx, n->row_sums_dev.Ensure(static_cast<size_t>(n->out_depth) * 4));
        RETURN_IF_FC(ctx, lrtfc_row_sums_int8(n->filter_dev.as<int8_t>(), n->out_depth, n->depth,
                                              n->row_sums_dev.as<int32_t>(), s));
        n->have_model_layout = true;
      }
      if (n->use_retiled) RETURN_IF_OK(RetileInt8(ctx, n, s));
    }
    if (bias) RETURN_IF_HIP(ctx, n->bias_dev.Upload(bias->data.raw, static_cast<size_t>(n->out_depth) * 4, s));
  } else if (n->kind == FcKind::kHybrid) {
    const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
    n->per_channel = fq->scale->size > 1;  // VerifyPerChannelQuantization, fully_connected.cc:827
    n->filter_scale = filter.params.scale;
    n->use_retiled = weights > 0 && lrtfc_fc_int8_preferred_layout(1, n->depth, n->out_depth, 0) ==
                                        LRTFC_LAYOUT_PACKED;
    n->split_quantize = n->batches > lrtfc_fc_hybrid_fused_max_batches(n->depth, n->out_depth);
    if (weights > 0 && !(n->use_retiled ? n->have_retiled : n->have_model_layout)) {
      if (!n->have_model_layout) {
        if (filter.type == kTfLiteInt4) {
          // An Int4 filter outside the 4-bit gate: UnpackPackedIntToInt8 over the flat tensor
          // (fully_connected.cc:805-814), once here instead of on every Eval.
          DeviceBuffer packed;
          RETURN_IF_HIP(ctx, packed.Upload(filter.data.raw, (weights + 1) / 2, s));
          RETURN_IF_HIP(ctx, n->filter_dev.Ensure(weights));
          RETURN_IF_FC(ctx, lrtfc_unpack_int4(packed.as<uint8_t>(), static_cast<int64_t>(weights),
                                              n->filter_dev.as<int8_t>(), s));
          RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        } else if (filter.type == kTfLiteInt2) {
          // Four values per byte over the flat tensor (fully_connected.cc:812-818, 1678-1685).
          DeviceBuffer packed;
          RETURN_IF_HIP(ctx, packed.Upload(filter.data.raw, (weights + 3) / 4, s));
          RETURN_IF_HIP(ctx, n->filter_dev.Ensure(weights));
          RETURN_IF_FC(ctx, lrtfc_unpack_int2(packed.as<uint8_t>(), static_cast<int64_t>(weights),
                                              n->filter_dev.as<int8_t>(), s));
          RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        } else {
          RETURN_IF_HIP(ctx, n->filter_dev.Upload(filter.data.raw, weights, s));
        }
        RETURN_IF_HIP(ctx, n->row_sums_dev.Ensure(static_cast<size_t>(n->out_depth) * 4));
        RETURN_IF_FC(ctx, lrtfc_row_sums_int8(n->filter_dev.as<int8_t>(), n->out_depth, n->depth,
                                              n->row_sums_dev.as<int32_t>(), s));
        n->have_model_layout = true;
      }
      if (n->use_retiled) RETURN_IF_OK(RetileInt8(ctx, n, s));
    }
    if (n->per_channel) {
      RETURN_IF_HIP(ctx, n->pcs_dev.Upload(fq->scale->data, static_cast<size_t>(n->out_depth) * 4, s));
    }
    if (bias) RETURN_IF_HIP(ctx, n->bias_dev.Upload(bias->data.raw, static_cast<size_t>(n->out_depth) * 4, s));
  } else if (n->kind == FcKind::kHybridInt4) {
    // EvalHybridDense4Bit: the filter scales (one, or one per channel) follow
    // fully_connected.cc:1146-1158; the nibbles are unpacked and re-tiled once.
    const auto* fq = static_cast<const TfLiteAffineQuantization*>(filter.quantization.params);
    n->per_channel = fq->scale->size > 1;
    n->filter_scale = fq->scale->data[0];
    n->use_retiled = true;
    n->nibble_layout = n->batches <= kInt4PerChannelNibbleMaxBatches;
    if (weights > 0 && !(n->nibble_layout ? n->have_nibbles : n->have_retiled)) {
      DeviceBuffer nibbles;
      RETURN_IF_HIP(ctx, nibbles.Upload(filter.data.raw, (weights + 1) / 2, s));
      if (n->nibble_layout) {
        n->retiled_dev.Release();
        RETURN_IF_HIP(ctx, n->retiled_dev.Ensure(
                               lrtfc_packed_int4_per_channel_bytes(n->out_depth, n->depth)));
        RETURN_IF_FC(ctx, lrtfc_pack_int4_per_channel(nibbles.as<uint8_t>(), n->out_depth, n->depth,
                                                      n->retiled_dev.as<uint8_t>(), s));
        RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        n->have_nibbles = true;
        n->have_retiled = false;
      } else {
        RETURN_IF_HIP(ctx, n->filter_dev.Ensure(weights));
        RETURN_IF_FC(ctx, lrtfc_unpack_int4(nibbles.as<uint8_t>(), static_cast<int64_t>(weights),
                                            n->filter_dev.as<int8_t>(), s));
        RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        n->retiled_dev.Release();
        RETURN_IF_OK(RetileInt8(ctx, n, s));
        n->have_nibbles = false;
      }
    }
    if (n->per_channel) {
      RETURN_IF_HIP(ctx, n->pcs_dev.Upload(fq->scale->data, static_cast<size_t>(n->out_depth) * 4, s));
    }
    if (bias) RETURN_IF_HIP(ctx, n->bias_dev.Upload(bias->data.raw, static_cast<size_t>(n->out_depth) * 4, s));
  } else {  // blockwise int4
    const auto* bq = static_cast<const TfLiteBlockwiseQuantization*>(filter.quantization.params);
    n->blocksize = bq->blocksize;
    n->scales = bq->scale;
    const TfLiteTensor& scales = ctx->tensors[bq->scale];
    n->use_retiled = weights > 0 && lrtfc_fc_blockwise_int4_preferred_layout(
                                        n->depth, n->blocksize) == LRTFC_LAYOUT_PACKED;
    n->split_quantize = n->depth > kInt4FusedMaxDepth && n->batches > kInt4DeepFusedMaxBatches;
    const int form = n->use_retiled ? lrtfc_fc_blockwise_int4_preferred_form(
                                          n->batches, n->depth, n->out_depth)
                                    : LRTFC_INT4_FORM_DECODE;
    const bool want_nibbles = form == LRTFC_INT4_FORM_GEMM_NIBBLES;
    n->gemm_layout = form != LRTFC_INT4_FORM_DECODE;
    if (n->gemm_layout && n->have_gemm && want_nibbles != n->gemm_nibbles) n->have_gemm = false;
    n->gemm_nibbles = want_nibbles;
    if (n->gemm_layout) {
      if (!n->have_gemm) {
        DeviceBuffer nibbles, block_scales;
        RETURN_IF_HIP(ctx, nibbles.Upload(filter.data.raw, weights / 2, s));
        RETURN_IF_HIP(ctx, block_scales.Upload(
                               scales.data.raw, static_cast<size_t>(NumElements(scales.dims)) * 2, s));
        RETURN_IF_HIP(ctx, n->kfsum_dev.Ensure(static_cast<size_t>(n->out_depth) * 4));
        RETURN_IF_FC(ctx, lrtfc_blockwise_int4_kfsum(nibbles.as<uint8_t>(),
                                                     block_scales.as<uint16_t>(), n->out_depth,
                                                     n->depth, n->blocksize,
                                                     n->kfsum_dev.as<float>(), s));
        n->retiled_dev.Release();
        if (n->gemm_nibbles) {
          RETURN_IF_HIP(ctx, n->retiled_dev.Ensure(
                                 lrtfc_gemm_int4_blockwise_nibble_bytes(n->out_depth, n->depth)));
          RETURN_IF_FC(ctx, lrtfc_pack_int4_blockwise_gemm_nibbles(
                                nibbles.as<uint8_t>(), block_scales.as<uint16_t>(), n->out_depth,
                                n->depth, n->blocksize, n->retiled_dev.as<uint8_t>(), s));
        } else {
          RETURN_IF_HIP(ctx, n->retiled_dev.Ensure(
                                 lrtfc_gemm_int4_blockwise_bytes(n->out_depth, n->depth)));
          RETURN_IF_FC(ctx, lrtfc_pack_int4_blockwise_gemm(
                                nibbles.as<uint8_t>(), block_scales.as<uint16_t>(), n->out_depth,
                                n->depth, n->blocksize, n->retiled_dev.as<uint8_t>(), s));
        }
        RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        n->filter_dev.Release();
        n->scales_dev.Release();
        n->have_gemm = true;
        n->have_retiled = n->have_model_layout = false;
      }
    } else if (weights > 0 && !(n->use_retiled ? n->have_retiled : n->have_model_layout)) {
      n->have_gemm = false;
      if (!n->have_model_layout) {
        RETURN_IF_HIP(ctx, n->filter_dev.Upload(filter.data.raw, weights / 2, s));
        RETURN_IF_HIP(ctx, n->scales_dev.Upload(scales.data.raw,
                                                static_cast<size_t>(NumElements(scales.dims)) * 2, s));
        RETURN_IF_HIP(ctx, n->kfsum_dev.Ensure(static_cast<size_t>(n->out_depth) * 4));
        RETURN_IF_FC(ctx, lrtfc_blockwise_int4_kfsum(n->filter_dev.as<uint8_t>(),
                                                     n->scales_dev.as<uint16_t>(), n->out_depth,
                                                     n->depth, n->blocksize,
                                                     n->kfsum_dev.as<float>(), s));
        n->have_model_layout = true;
      }
      if (n->use_retiled) {
        RETURN_IF_HIP(ctx, n->retiled_dev.Ensure(
                               lrtfc_packed_int4_blockwise_bytes(n->out_depth, n->depth)));
        RETURN_IF_FC(ctx, lrtfc_pack_int4_blockwise(n->filter_dev.as<uint8_t>(),
                                                    n->scales_dev.as<uint16_t>(), n->out_depth,
                                                    n->depth, n->blocksize,
                                                    n->retiled_dev.as<uint8_t>(), s));
        RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
        n->have_retiled = true;
        n->filter_dev.Release();  // the scales travel inside the re-tiled copy
        n->scales_dev.Release();
        n->have_model_layout = false;
      }
    }
    if (bias) RETURN_IF_HIP(ctx, n->bias_dev.Upload(bias->data.raw, static_cast<size_t>(n->out_depth) * 4, s));
  }
  n->uploaded_filter = filter.data.raw;

  return kTfLiteOk;
}

TfLiteStatus BuildGroupTables(TfLiteContext* ctx, PartitionKernel* k);

// After every node is prepared (shapes and kernel forms known): which nodes share a launch,
// which stream each unit runs on, which nodes other streams wait for.
TfLiteStatus PlanSchedule(TfLiteContext* ctx, PartitionKernel* k) {
  const int count = static_cast<int>(k->nodes.size());
  // Arena layout (tensor sizes are final here).
  {
    k->arena_offset.clear();
    size_t next = 0;
    auto place = [&](int t) {
      if (k->arena_offset.count(t)) return;
      k->arena_offset[t] = next;
      next += (ctx->tensors[t].bytes + 255) & ~static_cast<size_t>(255);
    };
    for (int t : k->uploads) place(t);
    k->upload_bytes = next;
    k->download_offset = next;
    for (int t : k->downloads) place(t);
    k->download_bytes = next - k->download_offset;
    for (const FcNode& n : k->nodes) {
      place(n.input);
      place(n.output);
    }
    RETURN_IF_HIP(ctx, k->arena.Ensure(next));
    RETURN_IF_HIP(ctx, k->upload_stage.Ensure(k->upload_bytes));
    RETURN_IF_HIP(ctx, k->download_stage.Ensure(k->download_bytes));
    // Outputs straight into host memory: worth it while the copy command's fixed cost matters
    // more than PCIe write combining (decode-sized outputs), and only for tensors nobody in the
    // partition reads (a reader would fetch them over PCIe, workgroup by workgroup).
    k->direct_outputs = false;
    k->download_stage_device = nullptr;
    if (k->download_bytes > 0 && k->download_bytes <= kDirectOutputMaxBytes) {
      bool read_back = false;
      for (const FcNode& n : k->nodes) {
        read_back = read_back || std::find(k->downloads.begin(), k->downloads.end(), n.input) !=
                                     k->downloads.end();
        read_back = read_back || n.depth == 0;  // such a node's output is cleared with a memset
        read_back = read_back || !WritesOutputOnce(n.kind);
      }
      void* device_view = nullptr;
      if (!read_back &&
          hipHostGetDevicePointer(&device_view, k->download_stage.get(), 0) == hipSuccess) {
        k->direct_outputs = true;
        k->download_stage_device = static_cast<uint8_t*>(device_view);
      }
    }
  }
  {
    k->direct_inputs = false;
    k->upload_stage_device = nullptr;
    if (k->state->options.direct_inputs && k->upload_bytes > 0 &&
        k->upload_bytes <= kDirectInputMaxBytes) {
      bool decode_shaped = true;
      for (const FcNode& n : k->nodes) {
        if (std::find(k->uploads.begin(), k->uploads.end(), n.input) == k->uploads.end()) continue;
        const bool kind_ok = n.kind == FcKind::kInt8 || n.kind == FcKind::kHybrid ||
                             n.kind == FcKind::kInt4Blockwise || n.kind == FcKind::kHybridInt4;
        decode_shaped = decode_shaped && kind_ok && n.batches <= kDirectInputMaxBatches;
      }
      void* device_view = nullptr;
      if (decode_shaped &&
          hipHostGetDevicePointer(&device_view, k->upload_stage.get(), 0) == hipSuccess) {
        k->direct_inputs = true;
        k->upload_stage_device = static_cast<uint8_t*>(device_view);
      }
    }
  }
  // Levels: a node without a producer inside the partition is at level 0, a consumer one
  // above its producer (an FC node has one activation input, so one producer at most).
  std::vector<int> level(count, 0);
  for (int i = 0; i < count; ++i) {
    if (k->nodes[i].producer >= 0) level[i] = level[k->nodes[i].producer] + 1;
  }
  // Groups: blockwise-int4 nodes on the fused re-tiled kernel that share level, depth and
  // batch count -- wherever they stand in the plan. Nodes of one level cannot depend on each
  // other, so each such set (cut into pieces of LRTFC_INT4_GROUP_MAX) is one launch.
  k->groups.clear();
  for (FcNode& n : k->nodes) n.group = -1;
  // (Nodes whose rows are quantized by a launch of their own group too: the group then has
  // one such launch for all its rows, into per-node workspaces.)
  auto groupable = [&](const FcNode& n) {
    return n.kind == FcKind::kInt4Blockwise && n.use_retiled && !n.gemm_layout && n.depth > 0 &&
           n.batches > 0 && n.out_depth > 0;
  };
  {
    std::map<std::tuple<int, int, int>, std::vector<int>> sets;  // (level, depth, batches)
    for (int i = 0; i < count; ++i) {
      const FcNode& n = k->nodes[i];
      if (groupable(n)) sets[std::make_tuple(level[i], n.depth, n.batches)].push_back(i);
    }
    for (const auto& entry : sets) {
      const std::vector<int>& all = entry.second;
      for (size_t at = 0; at < all.size(); at += LRTFC_INT4_GROUP_MAX) {
        const size_t end = std::min(all.size(), at + static_cast<size_t>(LRTFC_INT4_GROUP_MAX));
        if (end - at < 2) continue;
        PartitionKernel::Group g;
        g.members.assign(all.begin() + at, all.begin() + end);
        for (int m : g.members) k->nodes[m].group = static_cast<int>(k->groups.size());
        k->groups.push_back(std::move(g));
      }
    }
  }
  // Groups whose shape the library runs faster on the filters kept at 4 bits per weight for the
  // matrix cores: their members get that form of their filters as well.
  for (const PartitionKernel::Group& g : k->groups) {
    std::vector<int> out_depths;
    for (int m : g.members) out_depths.push_back(k->nodes[m].out_depth);
    const FcNode& head = k->nodes[g.members.front()];
    const bool nibbles = lrtfc_int4_group_preferred_form(
                             out_depths.data(), static_cast<int>(out_depths.size()), head.batches,
                             head.depth) == LRTFC_INT4_FORM_GEMM_NIBBLES;
    for (int m : g.members) {
      FcNode& n = k->nodes[m];
      const TfLiteTensor& filter = ctx->tensors[n.filter];
      if (!nibbles) {
        n.group_nibbles_dev.Release();
        n.group_nibbles_from = nullptr;
        continue;
      }
      if (n.group_nibbles_from == filter.data.raw) continue;
      const TfLiteTensor& scales = ctx->tensors[n.scales];
      const size_t weights = static_cast<size_t>(n.out_depth) * n.depth;
      DeviceBuffer model_nibbles, block_scales;
      hipStream_t s = k->stream;
      RETURN_IF_HIP(ctx, model_nibbles.Upload(filter.data.raw, weights / 2, s));
      RETURN_IF_HIP(ctx, block_scales.Upload(
                             scales.data.raw, static_cast<size_t>(NumElements(scales.dims)) * 2, s));
      RETURN_IF_HIP(ctx, n.group_nibbles_dev.Ensure(
                             lrtfc_gemm_int4_blockwise_nibble_bytes(n.out_depth, n.depth)));
      RETURN_IF_FC(ctx, lrtfc_pack_int4_blockwise_gemm_nibbles(
                            model_nibbles.as<uint8_t>(), block_scales.as<uint16_t>(), n.out_depth,
                            n.depth, n.blocksize, n.group_nibbles_dev.as<uint8_t>(), s));
      RETURN_IF_HIP(ctx, hipStreamSynchronize(s));  // the two uploads are locals
      n.group_nibbles_from = filter.data.raw;
    }
  }
  for (FcNode& n : k->nodes) {  // a node that left its group keeps no such copy
    if (n.group < 0) {
      n.group_nibbles_dev.Release();
      n.group_nibbles_from = nullptr;
    }
  }
  // Launch order: units (a group, or a node on its own) by level, then by first node. A unit
  // only reads what lower levels wrote, so this is a topological order of the partition.
  k->order.clear();
  for (int i = 0; i < count; ++i) {
    const int g = k->nodes[i].group;
    if (g >= 0 && k->groups[g].members.front() != i) continue;  // listed with its group
    k->order.push_back(PartitionKernel::Unit{level[i], i, g});
  }
  std::stable_sort(k->order.begin(), k->order.end(),
                   [](const PartitionKernel::Unit& a, const PartitionKernel::Unit& b) {
                     return a.level != b.level ? a.level < b.level : a.first < b.first;
                   });
  // Streams: a unit (node or group) continues on the stream of its first node's producer
  // unless a sibling already did; units without a producer in the partition, and further
  // siblings, take streams round-robin.
  std::vector<bool> continued(count, false);
  int next_lane = 0;
  for (int i = 0; i < k->kMaxStreams; ++i) k->lane_used[i] = false;
  for (FcNode& n : k->nodes) n.signal = false;
  for (const PartitionKernel::Unit& u : k->order) {
    FcNode& n = k->nodes[u.first];
    if (n.producer >= 0 && !continued[n.producer]) {
      n.lane = k->nodes[n.producer].lane;
      continued[n.producer] = true;
    } else {
      n.lane = next_lane++ % k->num_streams;
    }
    k->lane_used[n.lane] = true;
    if (u.group >= 0) {
      for (int m : k->groups[u.group].members) k->nodes[m].lane = n.lane;
    }
  }
  for (const FcNode& n : k->nodes) {
    if (n.producer >= 0 && k->nodes[n.producer].lane != n.lane) k->nodes[n.producer].signal = true;
  }
  for (hipEvent_t& e : k->node_done) {
    if (e) (void)hipEventDestroy(e);
    e = nullptr;
  }
  k->node_done.assign(count, nullptr);
  for (int i = 0; i < count; ++i) {
    if (k->nodes[i].signal) {
      RETURN_IF_HIP(ctx, hipEventCreateWithFlags(&k->node_done[i], hipEventDisableTiming));
    }
  }
  // Scratch for the nodes that quantize in a launch of their own, per stream.
  k->lookup_nodes = 0;
  for (FcNode& n : k->nodes) {
    if (n.kind == FcKind::kEmbeddingLookup) n.status_slot = k->lookup_nodes++;
  }
  if (k->state->options.poll_completion && !k->completion_dev) {
    RETURN_IF_HIP(ctx, k->completion.Ensure(64));
    std::memset(k->completion.get(), 0, 64);
    void* dev = nullptr;
    RETURN_IF_HIP(ctx, hipHostGetDevicePointer(&dev, k->completion.get(), 0));
    k->completion_dev = static_cast<uint32_t*>(dev);
  }
  if (k->lookup_nodes > 0) {
    RETURN_IF_HIP(ctx, k->lookup_status.Ensure(static_cast<size_t>(k->lookup_nodes) * 12));
    void* dev = nullptr;
    RETURN_IF_HIP(ctx, hipHostGetDevicePointer(&dev, k->lookup_status.get(), 0));
    k->lookup_status_dev = static_cast<int32_t*>(dev);
  }
  for (const FcNode& n : k->nodes) {
    if (n.kind == FcKind::kEmbeddingLookup || n.group >= 0) continue;
    if (n.kind == FcKind::kInt4Blockwise && n.gemm_layout) {
      RETURN_IF_HIP(ctx, k->workspace[n.lane].Ensure(
                             lrtfc_fc_blockwise_int4_gemm_workspace_bytes(n.batches, n.depth)));
      continue;
    }
    if (n.kind == FcKind::kBatchMatMul) {
      RETURN_IF_HIP(ctx, k->workspace[n.lane].Ensure(lrtfc_batch_matmul_workspace_bytes(
                             n.lhs_batches, n.batches, n.depth, n.adj_x)));
      continue;
    }
    if (n.kind == FcKind::kHybridInt4 ||
        (n.kind != FcKind::kInt8 && (!n.use_retiled || n.split_quantize))) {
      RETURN_IF_HIP(ctx, k->workspace[n.lane].Ensure(
                             lrtfc_activation_workspace_bytes(n.batches, n.depth)));
    }
  }
  k->alias.clear();
  k->bindings.assign(k->uploads.size() + k->downloads.size(), nullptr);
  return BuildGroupTables(ctx, k);
}

// Group tables: device addresses of every member's tensors (stable until the next prepare or
// until a boundary tensor is bound to other memory).
TfLiteStatus BuildGroupTables(TfLiteContext* ctx, PartitionKernel* k) {
  for (PartitionKernel::Group& g : k->groups) {
    std::vector<lrtfc_int4_group_node> nodes(g.members.size());
    const FcNode& head = k->nodes[g.members.front()];
    size_t per_node = 0;
    if (head.batches > kInt4DeepFusedMaxBatches) {
      per_node = (lrtfc_activation_workspace_bytes(head.batches, head.depth) + 255) & ~size_t{255};
      RETURN_IF_HIP(ctx, g.workspace.Ensure(per_node * g.members.size()));
    }
    for (size_t m = 0; m < g.members.size(); ++m) {
      const FcNode& n = k->nodes[g.members[m]];
      nodes[m].input = static_cast<const float*>(k->Activation(n.input));
      nodes[m].retiled_filter = n.retiled_dev.as<uint8_t>();
      nodes[m].kfsum = n.kfsum_dev.as<float>();
      nodes[m].bias = n.bias == kTfLiteOptionalTensor ? nullptr : n.bias_dev.as<float>();
      nodes[m].output = static_cast<float*>(k->Activation(n.output));
      nodes[m].out_depth = n.out_depth;
      nodes[m].workspace = per_node ? g.workspace.as<uint8_t>() + per_node * m : nullptr;
      nodes[m].nibble_filter =
          n.group_nibbles_from ? n.group_nibbles_dev.as<uint8_t>() : nullptr;
    }
    const FcNode& first = k->nodes[g.members.front()];
    RETURN_IF_HIP(ctx, g.table.Ensure(lrtfc_int4_group_table_bytes()));
    RETURN_IF_FC(ctx, lrtfc_int4_group_prepare(nodes.data(), static_cast<int>(nodes.size()),
                                               first.batches, first.depth, g.table.get(),
                                               &g.launch, k->stream));
  }
  return kTfLiteOk;
}

TfLiteStatus KernelPrepare(TfLiteContext* ctx, TfLiteNode* node) {
  auto* k = static_cast<PartitionKernel*>(node->user_data);
  RETURN_IF_HIP(ctx, hipSetDevice(k->state->options.device));
  for (FcNode& n : k->nodes) {
    const TfLiteStatus st = PrepareNode(ctx, k, &n);
    if (st != kTfLiteOk) return st;
  }
  RETURN_IF_OK(PlanSchedule(ctx, k));
  RETURN_IF_HIP(ctx, hipStreamSynchronize(k->stream));
  // The profiler's summary groups executions by this text (tflite/core/c/common.h:1264-1270,
  // profile_summarizer.cc:84-88): the node kinds of the partition with their counts, and how
  // many launch units they form (a grouped launch of several nodes counts once; a unit may be
  // a row quantizer launch followed by a product launch).
  static const char* const kKindNames[] = {"none", "int8", "hybrid", "int4_blockwise",
                                           "int4_per_channel", "embedding_lookup",
                                           "batch_matmul"};
  int per_kind[7] = {0, 0, 0, 0, 0, 0, 0};
  int ungrouped = 0;
  for (const FcNode& n : k->nodes) {
    ++per_kind[static_cast<int>(n.kind)];
    if (n.group < 0) ++ungrouped;
  }
  std::string text;
  for (int kind = 1; kind < 7; ++kind) {
    if (per_kind[kind] == 0) continue;
    text += (text.empty() ? "" : " ") + std::string(kKindNames[kind]) + ":" +
            std::to_string(per_kind[kind]);
  }
  text += " launches:" + std::to_string(k->groups.size() + ungrouped);
  k->profile_text = text;
  return kTfLiteOk;
}

const char* KernelProfilingString(const TfLiteContext*, const TfLiteNode* node) {
  const auto* k = node ? static_cast<const PartitionKernel*>(node->user_data) : nullptr;
  return k ? k->profile_text.c_str() : nullptr;
}

// Which registered memory each boundary tensor is bound to now; on a change, the tensors are
// re-pointed and the address tables of the grouped launches rebuilt (nothing of this partition
// is in flight between two invokes). An output bound to memory that overlaps a bound input
// would be written while that input is still being read, so such a binding fails the invoke.
TfLiteStatus RefreshBindings(TfLiteContext* ctx, PartitionKernel* k) {
  std::vector<void*> now;
  now.reserve(k->uploads.size() + k->downloads.size());
  auto bound_address = [&](int t, void** address) {
    const TfLiteTensor& tensor = ctx->tensors[t];
    const RegisteredBuffer* bound = tensor.bytes ? BoundBuffer(k->state, tensor) : nullptr;
    *address = nullptr;
    if (!bound) return kTfLiteOk;
    if (bound->bytes < tensor.bytes) {
      ctx->ReportError(ctx, "litert_amd delegate: buffer handle %d holds %zu bytes, tensor %d needs %zu",
                       tensor.buffer_handle, bound->bytes, t, tensor.bytes);
      return kTfLiteError;
    }
    if (reinterpret_cast<uintptr_t>(bound->device) % 16 != 0) {
      ctx->ReportError(ctx, "litert_amd delegate: the memory behind buffer handle %d is not 16-byte aligned",
                       tensor.buffer_handle);
      return kTfLiteError;
    }
    *address = bound->device;
    return kTfLiteOk;
  };
  for (int t : k->uploads) {
    void* address = nullptr;
    RETURN_IF_OK(bound_address(t, &address));
    now.push_back(address);
  }
  for (int t : k->downloads) {
    void* address = nullptr;
    RETURN_IF_OK(bound_address(t, &address));
    now.push_back(address);
  }
  if (now == k->bindings) return kTfLiteOk;
  const size_t inputs = k->uploads.size();
  for (size_t o = inputs; o < now.size(); ++o) {
    if (!now[o]) continue;
    const auto* out_begin = static_cast<const uint8_t*>(now[o]);
    const auto* out_end = out_begin + ctx->tensors[k->downloads[o - inputs]].bytes;
    for (size_t i = 0; i < inputs; ++i) {
      if (!now[i]) continue;
      const auto* in_begin = static_cast<const uint8_t*>(now[i]);
      const auto* in_end = in_begin + ctx->tensors[k->uploads[i]].bytes;
      if (out_begin < in_end && in_begin < out_end) {
        ctx->ReportError(ctx, "litert_amd delegate: output tensor %d and input tensor %d are bound to overlapping device memory",
                         k->downloads[o - inputs], k->uploads[i]);
        return kTfLiteError;
      }
    }
  }
  k->alias.clear();
  for (size_t i = 0; i < now.size(); ++i) {
    if (now[i]) k->alias[i < inputs ? k->uploads[i] : k->downloads[i - inputs]] = now[i];
  }
  k->bindings = std::move(now);
  RETURN_IF_OK(BuildGroupTables(ctx, k));
  RETURN_IF_HIP(ctx, hipStreamSynchronize(k->stream));
  return kTfLiteOk;
}

// One turn of a polling loop: tell the core that this is a spin-wait.
inline void SpinPause() {
#if defined(__x86_64__) || defined(__i386__)
  __builtin_ia32_pause();
#elif defined(__aarch64__)
  asm volatile("yield" ::: "memory");
#endif
}

TfLiteStatus KernelInvoke(TfLiteContext* ctx, TfLiteNode* node) {
  auto* k = static_cast<PartitionKernel*>(node->user_data);
  RETURN_IF_HIP(ctx, hipSetDevice(k->state->options.device));
  MetricsState& metrics = k->state->metrics;
  const bool measure = metrics.on;
  // Device time costs two event records per invoke and their read-back; it is taken from
  // detail level 1 on, so that level 0 times the invoke as it runs without a collection.
  const bool measure_device = measure && metrics.detail_level >= 1;
  const auto host_begin = std::chrono::steady_clock::now();
  if (measure_device) {
    if (!k->metrics_begin) {
      RETURN_IF_HIP(ctx, hipEventCreate(&k->metrics_begin));
      RETURN_IF_HIP(ctx, hipEventCreate(&k->metrics_end));
    }
    RETURN_IF_HIP(ctx, hipEventRecord(k->metrics_begin, k->stream));
  }
  // Tensor data pointers may move between invokes: read them from the context each time.
  // A boundary tensor that carries a buffer handle of this delegate is already in device memory
  // (an input) or is to stay there (an output): the kernels work on the registered memory
  // itself. The bindings are compared with those of the last invoke; a change re-points the
  // tensors and rebuilds the grouped launches' address tables.
  RETURN_IF_OK(RefreshBindings(ctx, k));
  bool host_inputs = false;
  for (int t : k->uploads) {
    const TfLiteTensor& tensor = ctx->tensors[t];
    if (tensor.bytes == 0 || k->alias.count(t)) continue;
    std::memcpy(k->upload_stage.get() + k->arena_offset[t], tensor.data.raw, tensor.bytes);
    host_inputs = true;
  }
  const auto gathered = std::chrono::steady_clock::now();
  if (host_inputs && !k->direct_inputs) {
    RETURN_IF_HIP(ctx, hipMemcpyAsync(k->arena.get(), k->upload_stage.get(), k->upload_bytes,
                                      hipMemcpyHostToDevice, k->stream));
  }
  bool multi = false;
  for (int i = 1; i < k->num_streams; ++i) multi = multi || k->lane_used[i];
  if (multi) {
    RETURN_IF_HIP(ctx, hipEventRecord(k->upload_done, k->stream));
    for (int i = 1; i < k->num_streams; ++i) {
      if (k->lane_used[i]) RETURN_IF_HIP(ctx, hipStreamWaitEvent(k->streams[i], k->upload_done, 0));
    }
  }
  for (const PartitionKernel::Unit& unit : k->order) {
    const size_t node_i = static_cast<size_t>(unit.first);
    FcNode& n = k->nodes[node_i];
    hipStream_t s = k->streams[n.lane];
    DeviceBuffer& scratch = k->workspace[n.lane];
    if (unit.group >= 0) {
      // One launch for the whole group, behind the producers of every member; members that
      // other streams wait for record their events after it.
      PartitionKernel::Group& g = k->groups[unit.group];
      for (int m : g.members) {
        const int producer = k->nodes[m].producer;
        if (producer >= 0 && k->nodes[producer].lane != n.lane) {
          RETURN_IF_HIP(ctx, hipStreamWaitEvent(s, k->node_done[producer], 0));
        }
      }
      RETURN_IF_FC(ctx, lrtfc_fc_blockwise_int4_packed_grouped(
                            g.table.get(), &g.launch, k->state->options.quant_variant, s));
      for (int m : g.members) {
        if (k->nodes[m].signal) RETURN_IF_HIP(ctx, hipEventRecord(k->node_done[m], s));
      }
      continue;
    }
    // Cross-stream edge: wait for the producer. (Runs before the early-outs below so that a
    // consumer never waits on an event that was not recorded in this invoke.)
    if (n.producer >= 0 && k->nodes[n.producer].lane != n.lane) {
      RETURN_IF_HIP(ctx, hipStreamWaitEvent(s, k->node_done[n.producer], 0));
    }
    struct SignalOnExit {
      PartitionKernel* k;
      size_t i;
      hipStream_t s;
      ~SignalOnExit() {
        if (k->nodes[i].signal) (void)hipEventRecord(k->node_done[i], s);
      }
    } signal_on_exit{k, node_i, s};
    const TfLiteTensor& output = ctx->tensors[n.output];
    if (NumElements(output.dims) == 0) continue;  // fully_connected.cc:1966-1968
    void* out_dev = k->Activation(n.output);
    if (n.depth == 0) {                           // fully_connected.cc:1970-1973
      RETURN_IF_HIP(ctx, hipMemsetAsync(out_dev, 0, output.bytes, s));
      continue;
    }
    const void* in_dev = k->Activation(n.input);
    const bool has_bias = n.bias != kTfLiteOptionalTensor;
    const int variant = k->state->options.quant_variant;
    const float* bias_f32 = has_bias ? n.bias_dev.as<float>() : nullptr;
    switch (n.kind) {
      case FcKind::kInt8: {
        const void* rows = in_dev;
        void* result = out_dev;
        if (n.uint8_io) {
          RETURN_IF_FC(ctx, lrtfc_xor_sign_bit(static_cast<const uint8_t*>(in_dev),
                                               n.u8_rows_dev.as<uint8_t>(),
                                               static_cast<size_t>(n.batches) * n.depth, s));
          rows = n.u8_rows_dev.as<uint8_t>();
          result = n.u8_result_dev.as<uint8_t>();
        }
        if (n.use_retiled) {
          RETURN_IF_FC(ctx, lrtfc_fc_int8_packed(static_cast<const int8_t*>(rows),
                                                 n.retiled_dev.as<int8_t>(),
                                                 has_bias ? n.bias_dev.as<int32_t>() : nullptr,
                                                 n.mult_dev.as<int32_t>(), n.shift_dev.as<int32_t>(),
                                                 n.per_channel, n.row_sums_dev.as<int32_t>(),
                                                 static_cast<int8_t*>(result), n.batches, n.depth,
                                                 n.out_depth, n.input_offset, n.output_offset,
                                                 n.act_min, n.act_max, s));
        } else {
          RETURN_IF_FC(ctx, lrtfc_fc_int8(static_cast<const int8_t*>(rows),
                                          n.filter_dev.as<int8_t>(),
                                          has_bias ? n.bias_dev.as<int32_t>() : nullptr,
                                          n.mult_dev.as<int32_t>(), n.shift_dev.as<int32_t>(),
                                          n.per_channel, n.row_sums_dev.as<int32_t>(),
                                          static_cast<int8_t*>(result), n.batches, n.depth,
                                          n.out_depth, n.input_offset, n.filter_offset,
                                          n.output_offset, n.act_min, n.act_max, s));
        }
        if (n.uint8_io) {
          RETURN_IF_FC(ctx, lrtfc_xor_sign_bit(static_cast<const uint8_t*>(result),
                                               static_cast<uint8_t*>(out_dev),
                                               static_cast<size_t>(n.batches) * n.out_depth, s));
        }
        break;
      }
      case FcKind::kHybrid: {
        const float* pcs = n.per_channel ? n.pcs_dev.as<float>() : nullptr;
        const int asym = n.params.asymmetric_quantize_inputs;
        if (!n.use_retiled) {
          RETURN_IF_FC(ctx, lrtfc_fc_hybrid(static_cast<const float*>(in_dev),
                                            n.filter_dev.as<int8_t>(), pcs, n.filter_scale,
                                            n.row_sums_dev.as<int32_t>(), bias_f32,
                                            static_cast<float*>(out_dev), n.batches, n.depth,
                                            n.out_depth, asym, n.params.activation, variant,
                                            scratch.get(), scratch.bytes(), s));
        } else if (!n.split_quantize) {
          RETURN_IF_FC(ctx, lrtfc_fc_hybrid_packed(static_cast<const float*>(in_dev),
                                                   n.retiled_dev.as<int8_t>(), pcs, n.filter_scale,
                                                   n.row_sums_dev.as<int32_t>(), bias_f32,
                                                   static_cast<float*>(out_dev), n.batches,
                                                   n.depth, n.out_depth, asym, n.params.activation,
                                                   variant, s));
        } else {
          RETURN_IF_FC(ctx, lrtfc_fc_hybrid_packed_workspace(
                                static_cast<const float*>(in_dev), n.retiled_dev.as<int8_t>(), pcs,
                                n.filter_scale, n.row_sums_dev.as<int32_t>(), bias_f32,
                                static_cast<float*>(out_dev), n.batches, n.depth, n.out_depth, asym,
                                n.params.activation, variant, scratch.get(), scratch.bytes(), s));
        }
        break;
      }
      case FcKind::kHybridInt4:
        if (n.nibble_layout) {
          RETURN_IF_FC(ctx, lrtfc_fc_hybrid_int4_per_channel_nibbles(
                                static_cast<const float*>(in_dev), n.retiled_dev.as<uint8_t>(),
                                n.per_channel ? n.pcs_dev.as<float>() : nullptr, n.filter_scale,
                                bias_f32, static_cast<float*>(out_dev), n.batches, n.depth,
                                n.out_depth, n.params.activation, scratch.get(), scratch.bytes(), s));
          break;
        }
        RETURN_IF_FC(ctx, lrtfc_fc_hybrid_int4_per_channel_packed(
                              static_cast<const float*>(in_dev), n.retiled_dev.as<int8_t>(),
                              n.per_channel ? n.pcs_dev.as<float>() : nullptr, n.filter_scale,
                              bias_f32, static_cast<float*>(out_dev), n.batches, n.depth,
                              n.out_depth, n.params.activation, scratch.get(), scratch.bytes(), s));
        break;
      case FcKind::kInt4Blockwise:
        if (n.gemm_layout && n.gemm_nibbles) {
          RETURN_IF_FC(ctx, lrtfc_fc_blockwise_int4_gemm_nibbles(
                                static_cast<const float*>(in_dev), n.retiled_dev.as<uint8_t>(),
                                n.kfsum_dev.as<float>(), bias_f32, static_cast<float*>(out_dev),
                                n.batches, n.depth, n.out_depth, variant, scratch.get(),
                                scratch.bytes(), s));
        } else if (n.gemm_layout) {
          RETURN_IF_FC(ctx, lrtfc_fc_blockwise_int4_gemm(
                                static_cast<const float*>(in_dev), n.retiled_dev.as<uint8_t>(),
                                n.kfsum_dev.as<float>(), bias_f32, static_cast<float*>(out_dev),
                                n.batches, n.depth, n.out_depth, variant, scratch.get(),
                                scratch.bytes(), s));
        } else if (!n.use_retiled) {
          RETURN_IF_FC(ctx, lrtfc_fc_blockwise_int4(static_cast<const float*>(in_dev),
                                                    n.filter_dev.as<uint8_t>(),
                                                    n.scales_dev.as<uint16_t>(),
                                                    n.kfsum_dev.as<float>(), bias_f32,
                                                    static_cast<float*>(out_dev), n.batches,
                                                    n.depth, n.out_depth, n.blocksize, variant,
                                                    scratch.get(), scratch.bytes(), s));
        } else if (!n.split_quantize) {
          RETURN_IF_FC(ctx, lrtfc_fc_blockwise_int4_packed(static_cast<const float*>(in_dev),
                                                           n.retiled_dev.as<uint8_t>(),
                                                           n.kfsum_dev.as<float>(), bias_f32,
                                                           static_cast<float*>(out_dev), n.batches,
                                                           n.depth, n.out_depth, variant, s));
        } else {
          const ActivationScratch w = SplitScratch(scratch.get(), n.batches, n.depth);
          RETURN_IF_FC(ctx, lrtfc_batch_quantize_floats(static_cast<const float*>(in_dev),
                                                        n.batches, n.depth, w.q, w.sf, w.zp, 1,
                                                        variant, s));
          RETURN_IF_FC(ctx, lrtfc_fc_blockwise_int4_packed_quantized(
                                w.q, w.sf, w.zp, n.retiled_dev.as<uint8_t>(),
                                n.kfsum_dev.as<float>(), bias_f32, static_cast<float*>(out_dev),
                                n.batches, n.depth, n.out_depth, s));
        }
        break;
      case FcKind::kBatchMatMul:
        RETURN_IF_FC(ctx, lrtfc_batch_matmul_hybrid_packed_nd(
                              static_cast<const float*>(in_dev), n.lhs_dims, n.batches, n.depth,
                              n.adj_x, n.retiled_dev.as<int8_t>(), n.weight_dims, n.out_depth,
                              n.per_channel ? n.pcs_dev.as<float>() : nullptr, n.filter_scale,
                              n.row_sums_dev.as<int32_t>(), static_cast<float*>(out_dev),
                              n.params.asymmetric_quantize_inputs, variant, scratch.get(),
                              scratch.bytes(), s));
        break;
      case FcKind::kEmbeddingLookup: {
        int32_t* status = k->lookup_status_dev + 3 * n.status_slot;
        const int out_type = n.out_f16 ? LRTFC_OUT_FLOAT16 : LRTFC_OUT_FLOAT32;
        if (n.blocksize > 0) {
          RETURN_IF_FC(ctx, lrtfc_embedding_lookup_blockwise_int4(
                                static_cast<const int32_t*>(in_dev), n.batches,
                                n.filter_dev.as<uint8_t>(), n.table_rows, n.depth,
                                n.scales_dev.as<uint16_t>(), n.blocksize, out_type, out_dev, status,
                                s));
        } else {
          RETURN_IF_FC(ctx, lrtfc_embedding_lookup_hybrid(
                                static_cast<const int32_t*>(in_dev), n.batches, n.filter_dev.get(),
                                n.value_bits, n.table_rows, n.depth, n.filter_scale,
                                n.per_channel ? n.pcs_dev.as<float>() : nullptr, out_type, out_dev,
                                status, s));
        }
        break;
      }
      default:
        return kTfLiteError;
    }
  }
  hipStream_t s = k->stream;
  for (int i = 1; i < k->num_streams; ++i) {  // join: downloads follow every stream's work
    if (!k->lane_used[i]) continue;
    RETURN_IF_HIP(ctx, hipEventRecord(k->lane_done[i], k->streams[i]));
    RETURN_IF_HIP(ctx, hipStreamWaitEvent(s, k->lane_done[i], 0));
  }
  // An output that carries a buffer handle of this delegate stays in device memory, where the
  // kernels have written it, and the host copy is marked stale (the runtime fetches it through
  // CopyFromBufferHandle if a CPU node or the application asks: subgraph.cc:876-889).
  bool host_outputs = false;
  for (int t : k->downloads) {
    TfLiteTensor& tensor = ctx->tensors[t];
    if (tensor.bytes == 0) continue;
    if (k->alias.count(t)) {
      tensor.data_is_stale = true;
    } else {
      host_outputs = true;
    }
  }
  if (host_outputs && !k->direct_outputs) {
    RETURN_IF_HIP(ctx, hipMemcpyAsync(k->download_stage.get(),
                                      k->arena.as<uint8_t>() + k->download_offset,
                                      k->download_bytes, hipMemcpyDeviceToHost, s));
  }
  if (measure_device) RETURN_IF_HIP(ctx, hipEventRecord(k->metrics_end, s));
  if (k->completion_dev) {
    if (++k->completion_serial == 0) k->completion_serial = 1;  // the word starts out as 0
    RETURN_IF_FC(ctx, lrtfc_mark_completion(k->completion_dev, k->completion_serial, s));
  }
  const auto enqueued = std::chrono::steady_clock::now();
  // The runtime reads the outputs as soon as invoke returns; a consumer of a registered
  // buffer (another partition, the application's own kernels) may start right away too.
  bool finished = false;
  if (k->completion_dev) {
    // Poll for a bounded time: short partitions end inside it; a long one, or one whose kernel
    // failed and never reaches the mark, goes on to hipStreamSynchronize, which reports errors.
    const volatile uint32_t* word = reinterpret_cast<const volatile uint32_t*>(k->completion.get());
    constexpr auto kPollFor = std::chrono::microseconds(150);
    for (;;) {
      for (int spin = 0; spin < 64 && !finished; ++spin) {
        finished = *word == k->completion_serial;
        if (!finished) SpinPause();
      }
      if (finished || std::chrono::steady_clock::now() - enqueued > kPollFor) break;
    }
    if (finished) std::atomic_thread_fence(std::memory_order_acquire);
  }
  if (!finished) RETURN_IF_HIP(ctx, hipStreamSynchronize(s));
  const auto waited = std::chrono::steady_clock::now();
  if (measure_device) {
    if (finished) RETURN_IF_HIP(ctx, hipEventSynchronize(k->metrics_end));
    float ms = 0.0f;
    RETURN_IF_HIP(ctx, hipEventElapsedTime(&ms, k->metrics_begin, k->metrics_end));
    metrics.device_us += 1e3 * ms;
  }
  if (measure) {
    metrics.invokes += 1;
    metrics.nodes += static_cast<int64_t>(k->nodes.size());
    if (host_inputs) metrics.uploaded += static_cast<int64_t>(k->upload_bytes);
    if (host_outputs) metrics.downloaded += static_cast<int64_t>(k->download_bytes);
  }
  // A lookup outside the table fails the invoke, with the builtin's message
  // (tflite/kernels/embedding_lookup.cc:280-286, 365-371).
  for (const FcNode& n : k->nodes) {
    if (n.kind != FcKind::kEmbeddingLookup || n.batches == 0 || n.depth == 0) continue;
    const int32_t* status =
        reinterpret_cast<const int32_t*>(k->lookup_status.get()) + 3 * n.status_slot;
    if (status[0] != 0) {
      ctx->ReportError(ctx, "Embedding Lookup: index out of bounds. Got %d, and bounds are [0, %d]",
                       status[2], n.table_rows - 1);
      return kTfLiteError;
    }
  }
  for (int t : k->downloads) {
    TfLiteTensor& tensor = ctx->tensors[t];
    if (tensor.bytes == 0 || k->alias.count(t)) continue;
    std::memcpy(tensor.data.raw,
                k->download_stage.get() + (k->arena_offset[t] - k->download_offset), tensor.bytes);
  }
  if (measure) {
    const auto host_end = std::chrono::steady_clock::now();
    auto us = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) {
      return std::chrono::duration<double, std::micro>(b - a).count();
    };
    metrics.host_us += us(host_begin, host_end);
    metrics.gather_us += us(host_begin, gathered);
    metrics.enqueue_us += us(gathered, enqueued);
    metrics.wait_us += us(enqueued, waited);
    metrics.scatter_us += us(waited, host_end);
  }
  return kTfLiteOk;
}

TfLiteRegistration KernelRegistration() {
  TfLiteRegistration r{};
  r.init = KernelInit;
  r.free = KernelFree;
  r.prepare = KernelPrepare;
  r.invoke = KernelInvoke;
  r.profiling_string = KernelProfilingString;
  r.builtin_code = kTfLiteBuiltinDelegate;
  r.custom_name = "LiteRtAmdFullyConnected";
  r.version = 1;
  return r;
}

// ---- TfLiteDelegate::Prepare -----------------------------------------------------------

TfLiteStatus DelegatePrepare(TfLiteContext* ctx, TfLiteDelegate* delegate) {
  auto* state = static_cast<DelegateState*>(delegate->data_);
  TfLiteIntArray* plan = nullptr;
  if (ctx->GetExecutionPlan(ctx, &plan) != kTfLiteOk || !plan) {
    ctx->ReportError(ctx, "litert_amd delegate: GetExecutionPlan failed");
    return kTfLiteDelegateError;
  }
  // The plan array belongs to the runtime and dies with the next call: copy what we keep.
  std::vector<int> claimed;
  for (int i = 0; i < plan->size; ++i) {
    const int node_index = plan->data[i];
    TfLiteNode* node = nullptr;
    TfLiteRegistration* reg = nullptr;
    if (ctx->GetNodeAndRegistration(ctx, node_index, &node, &reg) != kTfLiteOk) {
      return kTfLiteDelegateError;
    }
    if (Classify(ctx, node, reg, state->options, nullptr) != FcKind::kNone) {
      claimed.push_back(node_index);
    }
  }
  auto* nodes = static_cast<TfLiteIntArray*>(
      std::malloc(sizeof(TfLiteIntArray) + sizeof(int) * claimed.size()));
  if (!nodes) return kTfLiteDelegateError;
  nodes->size = static_cast<int>(claimed.size());
  for (size_t i = 0; i < claimed.size(); ++i) nodes->data[i] = claimed[i];
  // The node list stays ours (common.h:982-986); an empty list is a valid no-op.
  const TfLiteStatus st =
      ctx->ReplaceNodeSubsetsWithDelegateKernels(ctx, KernelRegistration(), nodes, delegate);
  std::free(nodes);
  return st;
}

// ---- buffer handles (tflite/core/c/common.h:1458-1479) ---------------------------------

TfLiteStatus CopyFromBufferHandle(TfLiteContext* ctx, TfLiteDelegate* delegate,
                                  TfLiteBufferHandle handle, TfLiteTensor* tensor) {
  auto* state = static_cast<DelegateState*>(delegate->data_);
  if (handle < 0 || static_cast<size_t>(handle) >= state->buffers.size() ||
      !state->buffers[handle].device || !tensor || !tensor->data.raw ||
      state->buffers[handle].bytes < tensor->bytes) {
    if (ctx && ctx->ReportError) {
      ctx->ReportError(ctx, "litert_amd delegate: CopyFromBufferHandle: no buffer of %zu bytes behind handle %d",
                       tensor ? tensor->bytes : size_t{0}, handle);
    }
    return kTfLiteError;
  }
  RETURN_IF_HIP(ctx, hipSetDevice(state->options.device));
  RETURN_IF_HIP(ctx, hipMemcpy(tensor->data.raw, state->buffers[handle].device, tensor->bytes,
                               hipMemcpyDeviceToHost));
  return kTfLiteOk;
}

TfLiteStatus CopyToBufferHandle(TfLiteContext* ctx, TfLiteDelegate* delegate,
                                TfLiteBufferHandle handle, TfLiteTensor* tensor) {
  auto* state = static_cast<DelegateState*>(delegate->data_);
  if (handle < 0 || static_cast<size_t>(handle) >= state->buffers.size() ||
      !state->buffers[handle].device || !tensor || !tensor->data.raw ||
      state->buffers[handle].bytes < tensor->bytes) {
    if (ctx && ctx->ReportError) {
      ctx->ReportError(ctx, "litert_amd delegate: CopyToBufferHandle: no buffer of %zu bytes behind handle %d",
                       tensor ? tensor->bytes : size_t{0}, handle);
    }
    return kTfLiteError;
  }
  RETURN_IF_HIP(ctx, hipSetDevice(state->options.device));
  RETURN_IF_HIP(ctx, hipMemcpy(state->buffers[handle].device, tensor->data.raw, tensor->bytes,
                               hipMemcpyHostToDevice));
  return kTfLiteOk;
}

// Frees the handle, not the memory behind it (common.h:1473-1479).
void FreeBufferHandle(TfLiteContext*, TfLiteDelegate* delegate, TfLiteBufferHandle* handle) {
  auto* state = static_cast<DelegateState*>(delegate->data_);
  if (!handle) return;
  if (*handle >= 0 && static_cast<size_t>(*handle) < state->buffers.size()) {
    state->buffers[*handle] = RegisteredBuffer{};
  }
  *handle = kTfLiteNullBufferHandle;
}

bool ParseOptions(const char* const* keys, const char* const* values, size_t n, Options* opt,
                  std::string* error) {
  for (size_t i = 0; i < n; ++i) {
    const std::string key = keys[i] ? keys[i] : "";
    const std::string val = values[i] ? values[i] : "";
    if (key == "device") {
      opt->device = std::atoi(val.c_str());
    } else if (key == "streams") {
      opt->streams = std::atoi(val.c_str());
      if (opt->streams < 1 || opt->streams > 4) {
        *error = "streams must be between 1 and 4, got '" + val + "'";
        return false;
      }
    } else if (key == "quant_variant") {
      if (val == "portable") {
        opt->quant_variant = LRTFC_QUANT_PORTABLE;
      } else if (val == "neon_v8") {
        opt->quant_variant = LRTFC_QUANT_NEON_V8;
      } else if (val == "neon_legacy") {
        opt->quant_variant = LRTFC_QUANT_NEON_LEGACY;
      } else {
        *error = "quant_variant must be portable, neon_v8 or neon_legacy, got '" + val + "'";
        return false;
      }
    } else if (key == "direct_inputs") {
      if (val != "0" && val != "1") {
        *error = "direct_inputs must be 0 or 1, got '" + val + "'";
        return false;
      }
      opt->direct_inputs = val == "1";
    } else if (key == "completion") {
      if (val != "poll" && val != "sync") {
        *error = "completion must be poll or sync, got '" + val + "'";
        return false;
      }
      opt->poll_completion = val == "poll";
    } else if (key == "claim") {
      opt->claim_int8 = opt->claim_hybrid = opt->claim_int4_blockwise = false;
      opt->claim_int4_per_channel = opt->claim_embedding_lookup = false;
      opt->claim_batch_matmul = false;
      size_t pos = 0;
      while (pos <= val.size()) {
        const size_t comma = val.find(',', pos);
        const std::string item = val.substr(pos, comma == std::string::npos ? comma : comma - pos);
        if (item == "int8") {
          opt->claim_int8 = true;
        } else if (item == "hybrid") {
          opt->claim_hybrid = true;
        } else if (item == "int4_blockwise") {
          opt->claim_int4_blockwise = true;
        } else if (item == "int4_per_channel") {
          opt->claim_int4_per_channel = true;
        } else if (item == "embedding_lookup") {
          opt->claim_embedding_lookup = true;
        } else if (item == "batch_matmul") {
          opt->claim_batch_matmul = true;
        } else if (!item.empty()) {
          *error = "claim accepts int8, hybrid, int4_blockwise, int4_per_channel, embedding_lookup, "
                   "batch_matmul; got '" + item + "'";
          return false;
        }
        if (comma == std::string::npos) break;
        pos = comma + 1;
      }
    } else {
      *error = "unknown option '" + key + "'";
      return false;
    }
  }
  return true;
}

}  // namespace

extern "C" {

TfLiteDelegate* tflite_plugin_create_delegate(const char* const* options_keys,
                                              const char* const* options_values,
                                              size_t num_options,
                                              void (*report_error)(const char*)) {
  auto fail = [&](const std::string& msg) -> TfLiteDelegate* {
    if (report_error) report_error(("litert_amd delegate: " + msg).c_str());
    return nullptr;
  };
  auto state = std::make_unique<DelegateState>();
  std::string error;
  if (!ParseOptions(options_keys, options_values, num_options, &state->options, &error)) {
    return fail(error);
  }
  // No GPU, no delegate: the caller keeps its CPU kernels. Nothing here falls back silently.
  if (lrtfc_init(state->options.device) != LRTFC_OK) return fail(lrtfc_last_error());
  state->delegate = TfLiteDelegate{};
  state->delegate.data_ = state.get();
  state->delegate.Prepare = DelegatePrepare;
  state->delegate.CopyFromBufferHandle = CopyFromBufferHandle;
  state->delegate.CopyToBufferHandle = CopyToBufferHandle;
  state->delegate.FreeBufferHandle = FreeBufferHandle;
  state->delegate.flags = kTfLiteDelegateFlagsNone;  // static shapes; re-prepared after a resize
  state->delegate.opaque_delegate_builder = nullptr;
  return &state.release()->delegate;
}

void tflite_plugin_destroy_delegate(TfLiteDelegate* delegate) {
  if (!delegate) return;
  delete static_cast<DelegateState*>(delegate->data_);
}

// Registers device memory (a hipMalloc'ed range of `bytes` bytes on the delegate's device)
// and returns the buffer handle for it, or kTfLiteNullBufferHandle. The application then binds
// it to an input or output tensor with Interpreter::SetBufferHandle (subgraph.h:1043-1057):
// a bound input is read from that memory, a bound output is left there with data_is_stale
// set. Counterpart of StatefulNnApiDelegate::RegisterNnapiMemory
// (tflite/delegates/nnapi/nnapi_delegate.cc:6645-6660), free slots reused the same way.
TfLiteBufferHandle litert_amd_register_device_buffer(TfLiteDelegate* delegate, void* device_memory,
                                                     size_t bytes) {
  if (!delegate || !delegate->data_ || !device_memory || bytes == 0) return kTfLiteNullBufferHandle;
  auto* state = static_cast<DelegateState*>(delegate->data_);
  if (&state->delegate != delegate) return kTfLiteNullBufferHandle;
  for (size_t i = 0; i < state->buffers.size(); ++i) {
    if (!state->buffers[i].device) {
      state->buffers[i] = RegisteredBuffer{device_memory, bytes};
      return static_cast<TfLiteBufferHandle>(i);
    }
  }
  state->buffers.push_back(RegisteredBuffer{device_memory, bytes});
  return static_cast<TfLiteBufferHandle>(state->buffers.size() - 1);
}

// Metrics of the partitions this delegate runs, for the LiteRT accelerator table's
// start_metrics_collection / stop_metrics_collection
// (litert/c/internal/litert_accelerator_def.h:57-62) and for applications that hold the
// TfLiteDelegate itself. start clears the counters and switches collection on (detail_level
// is recorded; every level collects the same counters today); stop switches it off and copies
// the totals out. Both return 0, or 1 for a delegate that is not one of this library's.
int litert_amd_start_metrics(TfLiteDelegate* delegate, int detail_level) {
  if (!delegate || !delegate->data_) return 1;
  auto* state = static_cast<DelegateState*>(delegate->data_);
  if (&state->delegate != delegate || detail_level < 0) return 1;
  state->metrics = MetricsState{};
  state->metrics.on = true;
  state->metrics.detail_level = detail_level;
  return 0;
}

int litert_amd_stop_metrics(TfLiteDelegate* delegate, litert_amd_metrics* out) {
  if (!delegate || !delegate->data_ || !out) return 1;
  auto* state = static_cast<DelegateState*>(delegate->data_);
  if (&state->delegate != delegate || !state->metrics.on) return 1;
  const MetricsState& m = state->metrics;
  *out = litert_amd_metrics{m.invokes,   m.nodes,     m.uploaded,   m.downloaded, m.host_us,
                            m.device_us, m.gather_us, m.enqueue_us, m.wait_us,    m.scatter_us};
  state->metrics.on = false;
  return 0;
}

// Test and tooling hook: the claim predicate on its own (no device needed). Returns
// 0 = declined, 1 = int8, 2 = hybrid, 3 = int4 blockwise, 4 = int4 per-channel hybrid,
// 5 = EMBEDDING_LOOKUP from a quantized table, 6 = hybrid BATCH_MATMUL; `reason` (may be NULL)
// receives why a node was declined.
int litert_amd_classify_node(const TfLiteContext* ctx, const TfLiteNode* node,
                             const TfLiteRegistration* registration, char* reason,
                             size_t reason_size) {
  std::string why;
  const FcKind kind = Classify(ctx, node, registration, Options{}, &why);
  if (reason && reason_size) {
    std::snprintf(reason, reason_size, "%s", why.c_str());
  }
  return static_cast<int>(kind);
}

// Test and tooling hook: how a prepared partition (the user_data of its delegate-kernel
// node) will run, as text: per node "index:kind/stream[/gN]", N = its grouped launch.
int litert_amd_describe_partition(const void* user_data, char* out, size_t out_size) {
  if (!user_data || user_data == reinterpret_cast<const void*>(-1) || !out || !out_size) return -1;
  const auto* k = static_cast<const PartitionKernel*>(user_data);
  std::string text = "groups=" + std::to_string(k->groups.size()) + " nodes=";
  for (size_t i = 0; i < k->nodes.size(); ++i) {
    const FcNode& n = k->nodes[i];
    text += (i ? " " : "") + std::to_string(n.node_index) + ":" +
            std::to_string(static_cast<int>(n.kind)) + "/s" + std::to_string(n.lane);
    if (n.group >= 0) {
      // "n" behind the group: the member runs on the 4-bit-resident matrix-core form
      text += "/g" + std::to_string(n.group) + (n.group_nibbles_from ? "n" : "");
    }
  }
  std::snprintf(out, out_size, "%s", text.c_str());
  return static_cast<int>(k->groups.size());
}

}  // extern "C"

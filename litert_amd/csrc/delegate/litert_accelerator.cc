// LiteRT accelerator skin over the TfLiteDelegate plugin: the exported LiteRtAcceleratorImpl
// object lets the LiteRT runtime register this library as its GPU accelerator
// (litert/runtime/accelerators/gpu_registry.cc:113-128 looks the symbol up,
// registration_helper.cc:34-86 checks the ABI header and copies the callbacks). CompiledModel
// then calls create_delegate, which builds the same delegate the external-delegate entry
// points build and hands it to the runtime's wrap_delegate together with its deleter
// (the pattern of litert/runtime/accelerators/xnnpack/xnnpack_accelerator.cc:59-130).
#include <cstdio>
#include <string>
#include <vector>

#include "litert_accelerator_abi.h"
#include "litert_amd_delegate.h"
#include "tflite_abi.h"

// What LiteRtMetrics points at: litert/runtime/metrics.h:23-29. A C++ object that crosses the
// library boundary, as it does for the reference's own accelerators (the dispatch delegate
// fills one the same way, litert/runtime/dispatch/dispatch_delegate.cc:268-277), so this
// library must be built with the C++ standard library the runtime uses.
struct LiteRtMetricsT {
  struct Metric {
    std::string name;
    LiteRtAny value;
  };
  std::vector<Metric> metrics;
};

namespace {

void ReportToStderr(const char* message) {
  std::fprintf(stderr, "litert_amd accelerator: %s\n", message);
}

LiteRtStatus GetName(LiteRtAcceleratorConst /*accelerator*/, const char** name) {
  if (!name) return kLiteRtStatusErrorInvalidArgument;
  *name = "litert_amd_fc_mi355x";
  return kLiteRtStatusOk;
}

LiteRtStatus GetVersion(LiteRtAcceleratorConst /*accelerator*/, LiteRtApiVersion* version) {
  if (!version) return kLiteRtStatusErrorInvalidArgument;
  *version = LiteRtApiVersion{0, 1, 0};
  return kLiteRtStatusOk;
}

LiteRtStatus GetHardwareSupport(LiteRtAcceleratorConst /*accelerator*/,
                                LiteRtHwAcceleratorSet* supported_hardware) {
  if (!supported_hardware) return kLiteRtStatusErrorInvalidArgument;
  *supported_hardware = kLiteRtHwAcceleratorGpu;
  return kLiteRtStatusOk;
}

// The delegate runs prebuilt kernels: it does not compile the model at prepare time.
LiteRtStatus IsJitResponsible(LiteRtAcceleratorConst /*accelerator*/, bool* does_jit_compilation) {
  if (!does_jit_compilation) return kLiteRtStatusErrorInvalidArgument;
  *does_jit_compilation = false;
  return kLiteRtStatusOk;
}

void DeleteDelegate(TfLiteOpaqueDelegate* delegate) {
  tflite_plugin_destroy_delegate(reinterpret_cast<TfLiteDelegate*>(delegate));
}

LiteRtStatus CreateDelegate(LiteRtRuntimeContext* runtime_context, LiteRtEnvironment /*env*/,
                            LiteRtAcceleratorConst /*accelerator*/, LiteRtOptions /*options*/,
                            LiteRtDelegateWrapper* delegate_wrapper) {
  if (!runtime_context || !delegate_wrapper) return kLiteRtStatusErrorInvalidArgument;
  // The table must be the layout this file was written against and reach wrap_delegate.
  if (runtime_context->abi_header.struct_size <
          offsetof(LiteRtRuntimeContext, wrap_delegate) + sizeof(runtime_context->wrap_delegate) ||
      !runtime_context->wrap_delegate) {
    return kLiteRtStatusErrorInvalidArgument;
  }
  // Default options (device 0, portable quantizer, four streams, every node kind). Without a
  // gfx950 device this returns NULL and the runtime keeps its CPU kernels.
  TfLiteDelegate* delegate = tflite_plugin_create_delegate(nullptr, nullptr, 0, ReportToStderr);
  if (!delegate) return kLiteRtStatusErrorRuntimeFailure;
  const LiteRtStatus status = runtime_context->wrap_delegate(
      reinterpret_cast<TfLiteOpaqueDelegate*>(delegate), DeleteDelegate, delegate_wrapper);
  if (status != kLiteRtStatusOk) tflite_plugin_destroy_delegate(delegate);
  return status;
}

// The TfLiteDelegate behind a wrapper the runtime made in create_delegate.
TfLiteDelegate* Unwrap(LiteRtRuntimeContext* runtime_context, LiteRtDelegateWrapper wrapper) {
  if (!runtime_context || !wrapper ||
      runtime_context->abi_header.struct_size <
          offsetof(LiteRtRuntimeContext, unwrap_delegate) +
              sizeof(runtime_context->unwrap_delegate) ||
      !runtime_context->unwrap_delegate) {
    return nullptr;
  }
  TfLiteOpaqueDelegate* opaque = nullptr;
  if (runtime_context->unwrap_delegate(wrapper, &opaque) != kLiteRtStatusOk) return nullptr;
  return reinterpret_cast<TfLiteDelegate*>(opaque);
}

// litert/c/internal/litert_accelerator_def.h:57-62; called by
// LiteRtCompiledModelT::StartMetricsCollection / StopMetricsCollection
// (litert/runtime/compiled_model.cc:2262-2290).
LiteRtStatus StartMetricsCollection(LiteRtRuntimeContext* runtime_context,
                                    LiteRtDelegateWrapper delegate, int detail_level) {
  TfLiteDelegate* d = Unwrap(runtime_context, delegate);
  if (!d || detail_level < 0) return kLiteRtStatusErrorInvalidArgument;
  return litert_amd_start_metrics(d, detail_level) == 0 ? kLiteRtStatusOk
                                                        : kLiteRtStatusErrorInvalidArgument;
}

LiteRtStatus StopMetricsCollection(LiteRtRuntimeContext* runtime_context,
                                   LiteRtDelegateWrapper delegate, LiteRtMetrics metrics) {
  TfLiteDelegate* d = Unwrap(runtime_context, delegate);
  if (!d || !metrics) return kLiteRtStatusErrorInvalidArgument;
  litert_amd_metrics m{};
  if (litert_amd_stop_metrics(d, &m) != 0) return kLiteRtStatusErrorInvalidArgument;
  auto integer = [](int64_t v) {
    LiteRtAny any{};
    any.type = kLiteRtAnyTypeInt;
    any.int_value = v;
    return any;
  };
  auto real = [](double v) {
    LiteRtAny any{};
    any.type = kLiteRtAnyTypeReal;
    any.real_value = v;
    return any;
  };
  metrics->metrics = {
      {"litert_amd.partition_invokes", integer(m.partition_invokes)},
      {"litert_amd.nodes_run", integer(m.nodes_run)},
      {"litert_amd.bytes_uploaded", integer(m.bytes_uploaded)},
      {"litert_amd.bytes_downloaded", integer(m.bytes_downloaded)},
      {"litert_amd.host_time_us", real(m.host_time_us)},
      {"litert_amd.device_time_us", real(m.device_time_us)},
      {"litert_amd.host_gather_us", real(m.host_gather_us)},
      {"litert_amd.host_enqueue_us", real(m.host_enqueue_us)},
      {"litert_amd.host_wait_us", real(m.host_wait_us)},
      {"litert_amd.host_scatter_us", real(m.host_scatter_us)},
  };
  return kLiteRtStatusOk;
}

}  // namespace

// Host object only: the file is compiled by the HIP driver, whose device pass must not see a
// table of host function pointers.
#ifndef __HIP_DEVICE_COMPILE__
extern "C" {

__attribute__((visibility("default"))) const LiteRtAcceleratorDef LiteRtAcceleratorImpl = {
    /*abi_header=*/{sizeof(LiteRtAcceleratorDef), LITERT_ACCELERATOR_DEF_CURRENT_VERSION, 0, 0},
    /*get_name=*/GetName,
    /*get_version=*/GetVersion,
    /*get_hardware_support=*/GetHardwareSupport,
    /*is_tflite_delegate_responsible_for_jit_compilation=*/IsJitResponsible,
    /*create_delegate=*/CreateDelegate,
    /*start_metrics_collection=*/StartMetricsCollection,
    /*stop_metrics_collection=*/StopMetricsCollection,
    /*buffer_handlers=*/
    {{sizeof(LiteRtCustomTensorBufferHandlersDef), 1, 0, 0}, nullptr, nullptr, nullptr, nullptr,
     nullptr, nullptr, 0, 0, 0, {0}},
};

// Tooling hooks for callers that cannot build a LiteRtMetricsT themselves (a C or ctypes
// harness): make one, read it, free it.
__attribute__((visibility("default"))) LiteRtMetrics litert_amd_metrics_object_new(void) {
  return new LiteRtMetricsT();
}
__attribute__((visibility("default"))) void litert_amd_metrics_object_free(LiteRtMetrics m) {
  delete m;
}
__attribute__((visibility("default"))) int litert_amd_metrics_object_size(LiteRtMetrics m) {
  return m ? static_cast<int>(m->metrics.size()) : -1;
}
__attribute__((visibility("default"))) const char* litert_amd_metrics_object_name(LiteRtMetrics m,
                                                                                  int i) {
  return (m && i >= 0 && i < static_cast<int>(m->metrics.size())) ? m->metrics[i].name.c_str()
                                                                  : nullptr;
}
__attribute__((visibility("default"))) double litert_amd_metrics_object_value(LiteRtMetrics m,
                                                                              int i) {
  if (!m || i < 0 || i >= static_cast<int>(m->metrics.size())) return 0.0;
  const LiteRtAny& v = m->metrics[i].value;
  return v.type == kLiteRtAnyTypeInt ? static_cast<double>(v.int_value) : v.real_value;
}

}  // extern "C"
#endif  // __HIP_DEVICE_COMPILE__

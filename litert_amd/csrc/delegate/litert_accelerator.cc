// LiteRT accelerator skin over the TfLiteDelegate plugin: the exported LiteRtAcceleratorImpl
// object lets the LiteRT runtime register this library as its GPU accelerator
// (litert/runtime/accelerators/gpu_registry.cc:113-128 looks the symbol up,
// registration_helper.cc:34-86 checks the ABI header and copies the callbacks). CompiledModel
// then calls create_delegate, which builds the same delegate the external-delegate entry
// points build and hands it to the runtime's wrap_delegate together with its deleter
// (the pattern of litert/runtime/accelerators/xnnpack/xnnpack_accelerator.cc:59-130).
#include <cstdio>

#include "litert_accelerator_abi.h"
#include "tflite_abi.h"

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
    /*start_metrics_collection=*/nullptr,
    /*stop_metrics_collection=*/nullptr,
    /*buffer_handlers=*/
    {{sizeof(LiteRtCustomTensorBufferHandlersDef), 1, 0, 0}, nullptr, nullptr, nullptr, nullptr,
     nullptr, nullptr, 0, 0, 0, {0}},
};

}  // extern "C"
#endif  // __HIP_DEVICE_COMPILE__

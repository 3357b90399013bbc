/* litert_accelerator_abi.h -- the slice of LiteRT's accelerator plug-in ABI that the AMD
 * FULLY_CONNECTED delegate needs in order to be registered as a LiteRT accelerator, restated
 * so that the plugin builds without the LiteRT source tree. Layout must match the runtime that
 * loads the plugin; tests/test_abi_layout.py compiles this header next to the reference's own
 * headers and compares sizeof/offsetof.
 *
 * Sources of truth (reference tree):
 *   litert/c/internal/litert_abi_header.h                          LiteRtAbiHeader
 *   litert/c/internal/litert_accelerator_def.h:40-97               LiteRtAcceleratorDefV1 (200 bytes)
 *   litert/c/internal/litert_custom_tensor_buffer_handlers_def.h   buffer handlers (136 bytes)
 *   litert/c/internal/litert_runtime_context.h:46-262              LiteRtRuntimeContext; only
 *       wrap_delegate (offset 144) and unwrap_delegate (152) are used here
 *   litert/c/litert_common.h:246-266, 320-401                      versions, status, hardware set
 *   litert/runtime/accelerators/registration_helper.cc:34-86, 111-127   how the runtime consumes
 *       the exported `LiteRtAcceleratorImpl` object
 *
 * When building inside a LiteRT checkout, define LITERT_AMD_USE_LITERT_HEADERS and the real
 * headers are included instead. */
#ifndef LITERT_AMD_LITERT_ACCELERATOR_ABI_H_
#define LITERT_AMD_LITERT_ACCELERATOR_ABI_H_

#ifdef LITERT_AMD_USE_LITERT_HEADERS
#include "litert/c/internal/litert_accelerator_def.h"
#else

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { /* litert_common.h:260-300, the values used here */
  kLiteRtStatusOk = 0,
  kLiteRtStatusErrorInvalidArgument = 1,
  kLiteRtStatusErrorRuntimeFailure = 3,
} LiteRtStatus;

typedef struct LiteRtApiVersion { /* litert_common.h:246-250 */
  int major;
  int minor;
  int patch;
} LiteRtApiVersion;

enum { /* litert_common.h:320-325 */
  kLiteRtHwAcceleratorNone = 0,
  kLiteRtHwAcceleratorCpu = 1 << 0,
  kLiteRtHwAcceleratorGpu = 1 << 1,
  kLiteRtHwAcceleratorNpu = 1 << 2,
};
typedef int LiteRtHwAcceleratorSet; /* litert_common.h:401 */

typedef struct LiteRtAbiHeader { /* litert_abi_header.h */
  uint16_t struct_size;
  uint16_t major_version;
  uint16_t minor_version;
  uint16_t reserved;
} LiteRtAbiHeader;

/* Opaque handles (litert_common.h:57-106): pointers to types only the runtime defines. */
typedef const struct LiteRtAcceleratorT* LiteRtAcceleratorConst;
typedef struct LiteRtEnvironmentT* LiteRtEnvironment;
typedef struct LiteRtOptionsT* LiteRtOptions;
typedef struct LiteRtDelegateWrapperT* LiteRtDelegateWrapper;
typedef struct LiteRtMetricsT* LiteRtMetrics;

/* litert/c/litert_any.h:24-62: the value of one metric. */
typedef enum {
  kLiteRtAnyTypeNone = 0,
  kLiteRtAnyTypeBool = 1,
  kLiteRtAnyTypeInt = 2,
  kLiteRtAnyTypeReal = 3,
  kLiteRtAnyTypeString = 8,
  kLiteRtAnyTypeVoidPtr = 9,
} LiteRtAnyType;
typedef struct {
  LiteRtAnyType type;
  union {
    bool bool_value;
    int64_t int_value;
    double real_value;
    const char* str_value;
    const void* ptr_value;
  };
} LiteRtAny;
typedef struct TfLiteOpaqueDelegate TfLiteOpaqueDelegate;

/* litert_custom_tensor_buffer_handlers_def.h: this plugin registers no buffer types, so the
 * six handler slots stay NULL and are declared as untyped function pointers. */
typedef struct LiteRtCustomTensorBufferHandlersDef {
  LiteRtAbiHeader abi_header;
  void (*create_func)(void);
  void (*destroy_func)(void);
  void (*lock_func)(void);
  void (*unlock_func)(void);
  void (*clear_func)(void);
  void (*import_func)(void);
  int device_tag;
  int queue_tag;
  size_t num_supported_buffer_types;
  int supported_buffer_types[16];
} LiteRtCustomTensorBufferHandlersDef;

/* litert_runtime_context.h: a table of function pointers behind an ABI header. Only the two
 * delegate-wrapping entries are named; the 17 entries before them keep their place. */
typedef struct LiteRtRuntimeContext {
  LiteRtAbiHeader abi_header;
  void (*entries_before_wrap_delegate[17])(void);
  LiteRtStatus (*wrap_delegate)(TfLiteOpaqueDelegate* delegate,
                                void (*deleter)(TfLiteOpaqueDelegate*),
                                LiteRtDelegateWrapper* wrapper);
  LiteRtStatus (*unwrap_delegate)(LiteRtDelegateWrapper wrapper, TfLiteOpaqueDelegate** delegate);
} LiteRtRuntimeContext;

#define LITERT_ACCELERATOR_DEF_CURRENT_VERSION 1

typedef struct { /* litert_accelerator_def.h:40-66 */
  LiteRtAbiHeader abi_header;
  LiteRtStatus (*get_name)(LiteRtAcceleratorConst accelerator, const char** name);
  LiteRtStatus (*get_version)(LiteRtAcceleratorConst accelerator, LiteRtApiVersion* version);
  LiteRtStatus (*get_hardware_support)(LiteRtAcceleratorConst accelerator,
                                       LiteRtHwAcceleratorSet* supported_hardware);
  LiteRtStatus (*is_tflite_delegate_responsible_for_jit_compilation)(
      LiteRtAcceleratorConst accelerator, bool* does_jit_compilation);
  LiteRtStatus (*create_delegate)(LiteRtRuntimeContext* runtime_context, LiteRtEnvironment env,
                                  LiteRtAcceleratorConst accelerator, LiteRtOptions options,
                                  LiteRtDelegateWrapper* delegate_wrapper);
  LiteRtStatus (*start_metrics_collection)(LiteRtRuntimeContext* runtime_context,
                                           LiteRtDelegateWrapper delegate, int detail_level);
  LiteRtStatus (*stop_metrics_collection)(LiteRtRuntimeContext* runtime_context,
                                          LiteRtDelegateWrapper delegate, LiteRtMetrics metrics);
  LiteRtCustomTensorBufferHandlersDef buffer_handlers;
} LiteRtAcceleratorDefV1;
typedef LiteRtAcceleratorDefV1 LiteRtAcceleratorDef;

#ifdef __cplusplus
} /* extern "C" */

/* The sizes and offsets the reference asserts for its own structs
 * (litert_accelerator_def.h:74-97, litert_custom_tensor_buffer_handlers_def.h:52-68,
 * litert_runtime_context.h:259-262). */
static_assert(sizeof(LiteRtAbiHeader) == 8, "LiteRtAbiHeader");
static_assert(sizeof(LiteRtCustomTensorBufferHandlersDef) == 136, "buffer handlers size");
static_assert(offsetof(LiteRtCustomTensorBufferHandlersDef, device_tag) == 56, "device_tag");
static_assert(offsetof(LiteRtCustomTensorBufferHandlersDef, queue_tag) == 60, "queue_tag");
static_assert(offsetof(LiteRtCustomTensorBufferHandlersDef, num_supported_buffer_types) == 64,
              "num_supported_buffer_types");
static_assert(offsetof(LiteRtCustomTensorBufferHandlersDef, supported_buffer_types) == 72,
              "supported_buffer_types");
static_assert(sizeof(LiteRtAcceleratorDefV1) == 200, "LiteRtAcceleratorDefV1 size");
static_assert(offsetof(LiteRtAcceleratorDefV1, get_name) == 8, "get_name");
static_assert(offsetof(LiteRtAcceleratorDefV1, get_version) == 16, "get_version");
static_assert(offsetof(LiteRtAcceleratorDefV1, get_hardware_support) == 24, "hardware support");
static_assert(offsetof(LiteRtAcceleratorDefV1,
                       is_tflite_delegate_responsible_for_jit_compilation) == 32, "jit");
static_assert(offsetof(LiteRtAcceleratorDefV1, create_delegate) == 40, "create_delegate");
static_assert(offsetof(LiteRtAcceleratorDefV1, start_metrics_collection) == 48, "start metrics");
static_assert(offsetof(LiteRtAcceleratorDefV1, stop_metrics_collection) == 56, "stop metrics");
static_assert(offsetof(LiteRtAcceleratorDefV1, buffer_handlers) == 64, "buffer_handlers");
static_assert(offsetof(LiteRtRuntimeContext, wrap_delegate) == 144, "wrap_delegate");
static_assert(offsetof(LiteRtRuntimeContext, unwrap_delegate) == 152, "unwrap_delegate");
#endif

#endif /* LITERT_AMD_USE_LITERT_HEADERS */

#ifdef __cplusplus
extern "C" {
#endif
/* The object the LiteRT runtime looks up in a GPU accelerator library
 * (litert/runtime/accelerators/gpu_registry.cc:124-128). */
extern const LiteRtAcceleratorDef LiteRtAcceleratorImpl;
#ifdef __cplusplus
}
#endif

#endif /* LITERT_AMD_LITERT_ACCELERATOR_ABI_H_ */

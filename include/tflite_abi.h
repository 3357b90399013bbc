/* tflite_abi.h — the slice of the TensorFlow Lite C ABI that a delegate plugin
 * for FULLY_CONNECTED touches, restated so that the delegate builds without the
 * LiteRT source tree. Layout (member order, types, enum values) must match the
 * runtime that loads the plugin; tests/test_abi_layout.py compiles this header
 * next to the reference's own headers and compares sizeof/offsetof of every
 * struct below.
 *
 * Sources of truth (reference tree):
 *   tflite/core/c/c_api_types.h:76-119            TfLiteStatus
 *   tflite/converter/core/c/tflite_types.h:43-82  TfLiteType, TfLiteQuantizationParams
 *   tflite/core/c/common.h                        everything else (line numbers inline)
 *   tflite/converter/core/c/builtin_op_data.h:79-87,186-211  fused activation, FC params
 *   tflite/builtin_ops.h:39,81                    builtin operator codes
 *   tflite/delegates/external/external_delegate_interface.h:65-74  plugin entry points
 *
 * When building inside a LiteRT checkout, define LITERT_AMD_USE_TFLITE_HEADERS and
 * the real headers are included instead.
 */
#ifndef LITERT_AMD_TFLITE_ABI_H_
#define LITERT_AMD_TFLITE_ABI_H_

#ifdef LITERT_AMD_USE_TFLITE_HEADERS
#include "tflite/builtin_ops.h"
#include "tflite/core/c/builtin_op_data.h"
#include "tflite/core/c/common.h"
#else

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalars and enums ----------------------------------------------------- */

typedef enum TfLiteStatus { /* c_api_types.h:76-119 */
  kTfLiteOk = 0,
  kTfLiteError = 1,
  kTfLiteDelegateError = 2,
  kTfLiteApplicationError = 3,
  kTfLiteDelegateDataNotFound = 4,
  kTfLiteDelegateDataWriteError = 5,
  kTfLiteDelegateDataReadError = 6,
  kTfLiteUnresolvedOps = 7,
  kTfLiteCancelled = 8,
  kTfLiteOutputShapeNotKnown = 9,
} TfLiteStatus;

typedef enum { /* tflite_types.h:43-68 */
  kTfLiteNoType = 0, kTfLiteFloat32 = 1, kTfLiteInt32 = 2, kTfLiteUInt8 = 3, kTfLiteInt64 = 4,
  kTfLiteString = 5, kTfLiteBool = 6, kTfLiteInt16 = 7, kTfLiteComplex64 = 8, kTfLiteInt8 = 9,
  kTfLiteFloat16 = 10, kTfLiteFloat64 = 11, kTfLiteComplex128 = 12, kTfLiteUInt64 = 13,
  kTfLiteResource = 14, kTfLiteVariant = 15, kTfLiteUInt32 = 16, kTfLiteUInt16 = 17,
  kTfLiteInt4 = 18, kTfLiteBFloat16 = 19, kTfLiteInt2 = 20, kTfLiteUInt4 = 21,
  kTfLiteFloat8E4M3FN = 22, kTfLiteFloat8E5M2 = 23,
} TfLiteType;

typedef struct TfLiteQuantizationParams { /* tflite_types.h:79-82 */
  float scale;
  int32_t zero_point;
} TfLiteQuantizationParams;

typedef enum TfLiteDimensionType { kTfLiteDimDense = 0, kTfLiteDimSparseCSR } TfLiteDimensionType;

typedef enum TfLiteExternalContextType { /* common.h:77-86 */
  kTfLiteEigenContext = 0, kTfLiteGemmLowpContext = 1, kTfLiteEdgeTpuContext = 2,
  kTfLiteCpuBackendContext = 3, kTfLiteLiteRtBufferContext = 4, kTfLiteMaxExternalContexts = 5
} TfLiteExternalContextType;

struct TfLiteContext;
struct TfLiteDelegate;
struct TfLiteRegistration;
struct TfLiteOpaqueDelegateBuilder;
struct TfLiteAsyncKernel;
typedef struct TfLiteOperator TfLiteOperator;

typedef struct TfLiteExternalContext { /* common.h:98-103 */
  TfLiteExternalContextType type;
  TfLiteStatus (*Refresh)(struct TfLiteContext* context);
} TfLiteExternalContext;

#define kTfLiteOptionalTensor (-1) /* common.h:107 */

typedef struct TfLiteIntArray { /* common.h:112-128 */
  int size;
  int data[];
} TfLiteIntArray;

typedef struct TfLiteFloatArray { /* common.h:157-172 */
  int size;
  float data[];
} TfLiteFloatArray;

typedef struct TfLiteComplex64 { float re, im; } TfLiteComplex64;
typedef struct TfLiteComplex128 { double re, im; } TfLiteComplex128;
typedef struct TfLiteFloat16 { uint16_t data; } TfLiteFloat16;
typedef struct TfLiteBFloat16 { uint16_t data; } TfLiteBFloat16;

/* ---- quantization ---------------------------------------------------------- */

typedef enum TfLiteQuantizationType
#ifdef __cplusplus
    : int
#endif
{ /* common.h:348-361 */
  kTfLiteNoQuantization = 0,
  kTfLiteAffineQuantization = 1,
  kTfLiteBlockwiseQuantization = 2,
  kTfLiteMultiAxisQuantization = 3,
} TfLiteQuantizationType;

typedef struct TfLiteQuantization { /* common.h:364-371 */
  TfLiteQuantizationType type;
  void* params; /* TfLiteAffineQuantization* or TfLiteBlockwiseQuantization* */
} TfLiteQuantization;

typedef struct TfLiteAffineQuantization { /* common.h:380-384 */
  TfLiteFloatArray* scale;
  TfLiteIntArray* zero_point;
  int32_t quantized_dimension;
} TfLiteAffineQuantization;

typedef struct TfLiteBlockwiseQuantization { /* common.h:390-398 */
  int32_t scale;      /* index of the fp16 scales tensor in context->tensors */
  int32_t zero_point; /* index of the zero-point tensor, -1 when absent */
  int32_t blocksize;
  int32_t quantized_dimension;
} TfLiteBlockwiseQuantization;

/* ---- tensors ------------------------------------------------------------------ */

typedef union TfLitePtrUnion { /* common.h:413-436: every member is one pointer */
  int32_t* i32; uint32_t* u32; int64_t* i64; uint64_t* u64; float* f; TfLiteFloat16* f16;
  TfLiteBFloat16* bf16; double* f64; char* raw; const char* raw_const; uint8_t* uint8; bool* b;
  int16_t* i16; uint16_t* ui16; TfLiteComplex64* c64; TfLiteComplex128* c128; int8_t* int8;
  void* data;
} TfLitePtrUnion;

typedef enum TfLiteAllocationType { /* common.h:456-466 */
  kTfLiteMemNone = 0, kTfLiteMmapRo, kTfLiteArenaRw, kTfLiteArenaRwPersistent, kTfLiteDynamic,
  kTfLitePersistentRo, kTfLiteCustom, kTfLiteVariantObject, kTfLiteNonCpu,
} TfLiteAllocationType;

typedef int TfLiteBufferHandle;
enum { kTfLiteNullBufferHandle = -1 };

typedef struct TfLiteDimensionMetadata {
  TfLiteDimensionType format;
  int dense_size;
  TfLiteIntArray* array_segments;
  TfLiteIntArray* array_indices;
} TfLiteDimensionMetadata;

typedef struct TfLiteSparsity {
  TfLiteIntArray* traversal_order;
  TfLiteIntArray* block_map;
  TfLiteDimensionMetadata* dim_metadata;
  int dim_metadata_size;
} TfLiteSparsity;

typedef struct TfLiteTensor { /* common.h:565-636 */
  TfLiteType type;
  TfLitePtrUnion data;
  TfLiteIntArray* dims;
  TfLiteQuantizationParams params;
  TfLiteAllocationType allocation_type;
  size_t bytes;
  const void* allocation;
  const char* name;
  struct TfLiteDelegate* delegate;
  TfLiteBufferHandle buffer_handle;
  bool data_is_stale;
  bool is_variable;
  TfLiteQuantization quantization;
  TfLiteSparsity* sparsity;
  const TfLiteIntArray* dims_signature;
} TfLiteTensor;

typedef struct TfLiteNode { /* common.h:641-678 */
  TfLiteIntArray* inputs;
  TfLiteIntArray* outputs;
  TfLiteIntArray* intermediates;
  TfLiteIntArray* temporaries;
  void* user_data;
  void* builtin_data;
  const void* custom_initial_data;
  int custom_initial_data_size;
  struct TfLiteDelegate* delegate;
  bool might_have_side_effect;
} TfLiteNode;

typedef struct TfLiteEvalTensor TfLiteEvalTensor; /* only ever handled by pointer here */

typedef struct TfLiteDelegateParams { /* common.h:869-874 */
  struct TfLiteDelegate* delegate;
  TfLiteIntArray* nodes_to_replace;
  TfLiteIntArray* input_tensors;
  TfLiteIntArray* output_tensors;
} TfLiteDelegateParams;

/* ---- registration, context, delegate --------------------------------------------- */

typedef struct TfLiteRegistration { /* common.h:1218-1305 */
  void* (*init)(struct TfLiteContext* context, const char* buffer, size_t length);
  void (*free)(struct TfLiteContext* context, void* buffer);
  TfLiteStatus (*prepare)(struct TfLiteContext* context, TfLiteNode* node);
  TfLiteStatus (*invoke)(struct TfLiteContext* context, TfLiteNode* node);
  const char* (*profiling_string)(const struct TfLiteContext* context, const TfLiteNode* node);
  int32_t builtin_code;
  const char* custom_name;
  int version;
  TfLiteOperator* registration_external;
  struct TfLiteAsyncKernel* (*async_kernel)(struct TfLiteContext* context, TfLiteNode* node);
  uint64_t inplace_operator;
} TfLiteRegistration;

typedef struct TfLiteContext { /* common.h:905-1100 (non-Windows layout) */
  size_t tensors_size;
  TfLiteStatus (*GetExecutionPlan)(struct TfLiteContext* context, TfLiteIntArray** execution_plan);
  TfLiteTensor* tensors;
  void* impl_;
  TfLiteStatus (*ResizeTensor)(struct TfLiteContext*, TfLiteTensor* tensor,
                               TfLiteIntArray* new_size);
  void (*ReportError)(struct TfLiteContext*, const char* msg, ...);
  TfLiteStatus (*AddTensors)(struct TfLiteContext*, int tensors_to_add,
                             int* first_new_tensor_index);
  TfLiteStatus (*GetNodeAndRegistration)(struct TfLiteContext*, int node_index, TfLiteNode** node,
                                         struct TfLiteRegistration** registration);
  TfLiteStatus (*ReplaceNodeSubsetsWithDelegateKernels)(struct TfLiteContext*,
                                                        struct TfLiteRegistration registration,
                                                        const TfLiteIntArray* nodes_to_replace,
                                                        struct TfLiteDelegate* delegate);
  int recommended_num_threads;
  TfLiteExternalContext* (*GetExternalContext)(struct TfLiteContext*, TfLiteExternalContextType);
  void (*SetExternalContext)(struct TfLiteContext*, TfLiteExternalContextType,
                             TfLiteExternalContext*);
  bool allow_fp32_relax_to_fp16;
  void* profiler;
  void* (*AllocatePersistentBuffer)(struct TfLiteContext* ctx, size_t bytes);
  TfLiteStatus (*AllocateBufferForEval)(struct TfLiteContext* ctx, size_t bytes, void** ptr);
  TfLiteStatus (*RequestScratchBufferInArena)(struct TfLiteContext* ctx, size_t bytes,
                                              int* buffer_idx);
  void* (*GetScratchBuffer)(struct TfLiteContext* ctx, int buffer_idx);
  TfLiteStatus (*ResizeTensorExplicit)(struct TfLiteContext* ctx, TfLiteTensor* tensor, int dims,
                                       const int* shape);
  TfLiteStatus (*PreviewDelegatePartitioning)(struct TfLiteContext* context,
                                              const TfLiteIntArray* nodes_to_replace,
                                              TfLiteDelegateParams** partition_params_array,
                                              int* num_partitions);
  TfLiteTensor* (*GetTensor)(const struct TfLiteContext* context, int tensor_idx);
  TfLiteEvalTensor* (*GetEvalTensor)(const struct TfLiteContext* context, int tensor_idx);
  TfLiteStatus (*GetModelMetadata)(const struct TfLiteContext* context, const char* name,
                                   const char** ptr, size_t* bytes);
  TfLiteStatus (*AcquireSubgraphContext)(struct TfLiteContext* context, int subgraph_index,
                                         struct TfLiteContext** acquired_context);
  TfLiteStatus (*ReleaseSubgraphContext)(struct TfLiteContext* context, int subgraph_index);
} TfLiteContext;

typedef enum TfLiteDelegateFlags { /* common.h:1389-1440 */
  kTfLiteDelegateFlagsNone = 0,
  kTfLiteDelegateFlagsAllowDynamicTensors = 1,
  kTfLiteDelegateFlagsRequirePropagatedShapes = 2,
  kTfLiteDelegateFlagsPerOperatorProfiling = 4,
  kTfLiteDelegateFlagsHintFullyDelegatedToSingleDelegate = 8,
} TfLiteDelegateFlags;

typedef struct TfLiteDelegate { /* common.h:1442-1493 */
  void* data_;
  TfLiteStatus (*Prepare)(TfLiteContext* context, struct TfLiteDelegate* delegate);
  TfLiteStatus (*CopyFromBufferHandle)(TfLiteContext* context, struct TfLiteDelegate* delegate,
                                       TfLiteBufferHandle buffer_handle, TfLiteTensor* tensor);
  TfLiteStatus (*CopyToBufferHandle)(TfLiteContext* context, struct TfLiteDelegate* delegate,
                                     TfLiteBufferHandle buffer_handle, TfLiteTensor* tensor);
  void (*FreeBufferHandle)(TfLiteContext* context, struct TfLiteDelegate* delegate,
                           TfLiteBufferHandle* handle);
  int64_t flags;
  struct TfLiteOpaqueDelegateBuilder* opaque_delegate_builder;
} TfLiteDelegate;

/* ---- FULLY_CONNECTED builtin data ---------------------------------------------------- */

typedef enum { /* builtin_op_data.h:79-87 */
  kTfLiteActNone = 0, kTfLiteActRelu, kTfLiteActReluN1To1, kTfLiteActRelu6, kTfLiteActTanh,
  kTfLiteActSignBit, kTfLiteActSigmoid,
} TfLiteFusedActivation;

typedef enum { /* builtin_op_data.h:186-189 */
  kTfLiteFullyConnectedWeightsFormatDefault = 0,
  kTfLiteFullyConnectedWeightsFormatShuffled4x16Int8 = 1,
} TfLiteFullyConnectedWeightsFormat;

typedef struct { /* builtin_op_data.h:191-211 */
  TfLiteFusedActivation activation;
  TfLiteFullyConnectedWeightsFormat weights_format;
  bool keep_num_dims;
  bool asymmetric_quantize_inputs;
  TfLiteType quantized_bias_type;
} TfLiteFullyConnectedParams;

typedef struct { /* builtin_op_data.h:246-253 */
  bool adj_x;
  bool adj_y;
  bool asymmetric_quantize_inputs;
} TfLiteBatchMatMulParams;

enum { /* builtin_ops.h:37,39,81,156 */
  kTfLiteBuiltinEmbeddingLookup = 7,
  kTfLiteBuiltinFullyConnected = 9,
  kTfLiteBuiltinDelegate = 51,
  kTfLiteBuiltinBatchMatmul = 126,
};

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* LITERT_AMD_USE_TFLITE_HEADERS */

/* ---- plugin entry points (external_delegate_interface.h:65-74) -------------------------- */
#ifdef __cplusplus
extern "C" {
#endif

/* Creates the delegate from key/value string options; NULL on failure (the reason goes
 * to report_error when that is non-NULL). Options understood:
 *   device          GPU ordinal (default 0)
 *   quant_variant   portable | neon_v8 | neon_legacy: which build of the reference's
 *                   activation quantizer to reproduce (default portable)
 *   claim           comma list out of int8,hybrid,int4_blockwise,int4_per_channel,
 *                   embedding_lookup,batch_matmul (default: all) */
TfLiteDelegate* tflite_plugin_create_delegate(const char* const* options_keys,
                                              const char* const* options_values,
                                              size_t num_options,
                                              void (*report_error)(const char*));
void tflite_plugin_destroy_delegate(TfLiteDelegate* delegate);

#ifdef __cplusplus
}
#endif

#endif /* LITERT_AMD_TFLITE_ABI_H_ */

/* litert_amd_delegate.h — symbols exported by liblitert_amd_delegate.so, the TfLite external
 * delegate plugin of the MI355X (gfx950) FULLY_CONNECTED kernels.
 *
 * The first two are the reference's plugin interface
 * (tflite/delegates/external/external_delegate_interface.h:65-74): a loader such as
 * TfLiteExternalDelegateCreate dlopens the library and looks them up by name
 * (tflite/delegates/external/external_delegate.cc:39-60, 215-223). The library also exports
 * the LiteRT accelerator table `LiteRtAcceleratorImpl` (include/litert_accelerator_abi.h).
 * The litert_amd_* functions are this library's own additions: what an application that holds
 * the TfLiteDelegate can ask of it beyond the reference interface.
 */
#ifndef LITERT_AMD_DELEGATE_H_
#define LITERT_AMD_DELEGATE_H_

#include <stddef.h>
#include <stdint.h>

#include "tflite_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* tflite_plugin_create_delegate / tflite_plugin_destroy_delegate are declared, with the
 * options they understand, in tflite_abi.h beside the structs they use. */

/* Registers device memory (`bytes` bytes, allocated by the application on the delegate's
 * device) and returns a buffer handle to bind to an input or output tensor with
 * Interpreter::SetBufferHandle (tflite/core/subgraph.h:1043-1057); kTfLiteNullBufferHandle on
 * failure. Counterpart of StatefulNnApiDelegate::RegisterNnapiMemory
 * (tflite/delegates/nnapi/nnapi_delegate.cc:6645-6660). The kernels work on the registered
 * memory itself: it must be 16-byte aligned and at least as large as the tensor bound to it, and
 * an output must not be bound to memory that overlaps a bound input of the same partition. */
TfLiteBufferHandle litert_amd_register_device_buffer(TfLiteDelegate* delegate,
                                                     void* device_memory, size_t bytes);

/* Totals over the partition invokes between litert_amd_start_metrics and
 * litert_amd_stop_metrics; what the LiteRT accelerator table reports through
 * start_metrics_collection / stop_metrics_collection
 * (litert/c/internal/litert_accelerator_def.h:57-62). */
typedef struct litert_amd_metrics {
  int64_t partition_invokes;
  int64_t nodes_run;         /* FULLY_CONNECTED / EMBEDDING_LOOKUP nodes those invokes ran */
  int64_t bytes_uploaded;    /* host -> device */
  int64_t bytes_downloaded;  /* device -> host */
  double host_time_us;       /* wall time inside the partitions' invoke callbacks */
  double device_time_us;     /* per invoke: first enqueued command to last finished one (HIP
                              * events; collected from detail_level 1 on, 0 below) */
  /* host_time_us by phase of an invoke: host tensors gathered into page-locked memory; copies and
   * kernels enqueued; the wait for the device to finish; outputs scattered back to the tensors. */
  double host_gather_us, host_enqueue_us, host_wait_us, host_scatter_us;
} litert_amd_metrics;
/* Both return 0, or 1 when `delegate` is not one of this library's (or, for stop, when no
 * collection is running). start clears the totals. detail_level 0: counts, bytes and host times
 * (a few clock reads per invoke); 1 and above: device_time_us as well (two event records per
 * invoke, which lengthen the enqueue phase by a few microseconds). */
int litert_amd_start_metrics(TfLiteDelegate* delegate, int detail_level);
int litert_amd_stop_metrics(TfLiteDelegate* delegate, litert_amd_metrics* out);

/* Tooling hooks (no device needed for the first): the node-claim predicate on its own —
 * returns 0 = declined, 1 = int8, 2 = hybrid, 3 = int4 blockwise, 4 = int4 per-channel hybrid,
 * 5 = EMBEDDING_LOOKUP, 6 = hybrid BATCH_MATMUL, `reason` (may be NULL) receiving why a node was
 * declined — and a text
 * account of how a prepared partition (the user_data of its delegate-kernel node) will run;
 * returns the number of grouped launches, -1 on bad arguments. */
int litert_amd_classify_node(const TfLiteContext* ctx, const TfLiteNode* node,
                             const TfLiteRegistration* registration, char* reason,
                             size_t reason_size);
int litert_amd_describe_partition(const void* user_data, char* out, size_t out_size);

/* Tooling hooks around the accelerator table's stop_metrics_collection, for callers that cannot
 * build the runtime's C++ metrics object themselves: make one, read entry i (value as a
 * double, whatever its type), free it. */
struct LiteRtMetricsT;
struct LiteRtMetricsT* litert_amd_metrics_object_new(void);
void litert_amd_metrics_object_free(struct LiteRtMetricsT* metrics);
int litert_amd_metrics_object_size(struct LiteRtMetricsT* metrics);
const char* litert_amd_metrics_object_name(struct LiteRtMetricsT* metrics, int i);
double litert_amd_metrics_object_value(struct LiteRtMetricsT* metrics, int i);

#ifdef __cplusplus
}
#endif
#endif /* LITERT_AMD_DELEGATE_H_ */

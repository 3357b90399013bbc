// A minimal stand-in for the TFLite interpreter, for tests only: it owns tensors and
// FULLY_CONNECTED nodes, loads a delegate plugin the way
// tflite/delegates/external/external_delegate.cc does (dlopen + the two plugin entry
// points), services the TfLiteContext calls a delegate makes during Prepare
// (GetExecutionPlan, GetNodeAndRegistration, ReplaceNodeSubsetsWithDelegateKernels,
// ReportError) and then drives init / prepare / invoke / free of the delegate kernel in
// the order tflite/core/subgraph.cc does (:523-637 partition + init, :2497-2569 delegate
// application with rollback on failure, :1691-1775 invoke loop). Nodes the delegate
// leaves alone are run by a callback the test supplies (the "CPU kernels").
//
// Exposed as a C API for ctypes; see tests/fake_host.py.
#include <dlfcn.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "tflite_abi.h"

namespace {

TfLiteIntArray* MakeIntArray(const std::vector<int>& v) {
  auto* a = static_cast<TfLiteIntArray*>(std::malloc(sizeof(TfLiteIntArray) + sizeof(int) * v.size()));
  a->size = static_cast<int>(v.size());
  for (size_t i = 0; i < v.size(); ++i) a->data[i] = v[i];
  return a;
}

struct NodeRec {
  TfLiteNode node{};
  TfLiteRegistration reg{};
  TfLiteFullyConnectedParams fc{};
  TfLiteBatchMatMulParams bmm{};
  bool is_delegate_kernel = false;
  std::vector<int> replaced;  // original node indices, for delegate kernels
  TfLiteDelegateParams dparams{};
  bool initialised = false;
  ~NodeRec() {
    std::free(node.inputs);
    std::free(node.outputs);
    std::free(dparams.nodes_to_replace);
    std::free(dparams.input_tensors);
    std::free(dparams.output_tensors);
  }
};

typedef TfLiteDelegate* (*CreateFn)(const char* const*, const char* const*, size_t,
                                    void (*)(const char*));
typedef void (*DestroyFn)(TfLiteDelegate*);
typedef int (*CpuCallback)(int node_index);

struct Host {
  TfLiteContext ctx{};
  std::vector<TfLiteTensor> tensors;
  std::vector<std::unique_ptr<std::vector<char>>> buffers;  // one per tensor (may be empty)
  std::vector<std::unique_ptr<TfLiteAffineQuantization>> affine;
  std::vector<std::unique_ptr<TfLiteBlockwiseQuantization>> blockwise;
  std::vector<std::unique_ptr<NodeRec>> nodes;
  std::vector<int> plan;
  std::vector<int> original_plan;
  TfLiteIntArray* plan_array = nullptr;
  std::set<int> graph_outputs;
  void* dl = nullptr;
  CreateFn create = nullptr;
  DestroyFn destroy = nullptr;
  TfLiteDelegate* delegate = nullptr;
  CpuCallback cpu = nullptr;
  std::string errors;
  int replace_calls = 0;

  void Sync() {
    ctx.tensors = tensors.data();
    ctx.tensors_size = tensors.size();
  }
};

thread_local std::string g_plugin_error;
void PluginError(const char* msg) { g_plugin_error += msg; }

Host* FromCtx(TfLiteContext* ctx) { return static_cast<Host*>(ctx->impl_); }

void CtxReportError(TfLiteContext* ctx, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  Host* h = FromCtx(ctx);
  h->errors += buf;
  h->errors += "\n";
}

TfLiteStatus CtxGetExecutionPlan(TfLiteContext* ctx, TfLiteIntArray** plan) {
  Host* h = FromCtx(ctx);
  std::free(h->plan_array);  // the previous array dies with this call, as in the runtime
  h->plan_array = MakeIntArray(h->plan);
  *plan = h->plan_array;
  return kTfLiteOk;
}

TfLiteStatus CtxGetNodeAndRegistration(TfLiteContext* ctx, int node_index, TfLiteNode** node,
                                       TfLiteRegistration** reg) {
  Host* h = FromCtx(ctx);
  if (node_index < 0 || node_index >= static_cast<int>(h->nodes.size())) return kTfLiteError;
  *node = &h->nodes[node_index]->node;
  *reg = &h->nodes[node_index]->reg;
  return kTfLiteOk;
}

TfLiteStatus CtxReplaceNodeSubsets(TfLiteContext* ctx, TfLiteRegistration registration,
                                   const TfLiteIntArray* nodes_to_replace,
                                   TfLiteDelegate* delegate) {
  Host* h = FromCtx(ctx);
  ++h->replace_calls;
  std::set<int> claimed(nodes_to_replace->data, nodes_to_replace->data + nodes_to_replace->size);
  if (claimed.empty()) return kTfLiteOk;
  // Which tensors does each node outside a run consume? Needed for partition outputs.
  std::vector<int> new_plan;
  size_t i = 0;
  while (i < h->plan.size()) {
    if (!claimed.count(h->plan[i])) {
      new_plan.push_back(h->plan[i]);
      ++i;
      continue;
    }
    std::vector<int> run;
    while (i < h->plan.size() && claimed.count(h->plan[i])) run.push_back(h->plan[i++]);
    std::set<int> produced, run_set(run.begin(), run.end());
    std::vector<int> inputs, outputs;
    for (int n : run) {
      const TfLiteNode& node = h->nodes[n]->node;
      for (int k = 0; k < node.inputs->size; ++k) {
        const int t = node.inputs->data[k];
        if (t == kTfLiteOptionalTensor || produced.count(t)) continue;
        bool seen = false;
        for (int u : inputs) seen = seen || (u == t);
        if (!seen) inputs.push_back(t);
      }
      for (int k = 0; k < node.outputs->size; ++k) produced.insert(node.outputs->data[k]);
    }
    for (int t : produced) {
      bool used_outside = h->graph_outputs.count(t) > 0;
      bool used_at_all = false;
      for (int n : h->plan) {
        const TfLiteNode& node = h->nodes[n]->node;
        for (int k = 0; k < node.inputs->size; ++k) {
          if (node.inputs->data[k] != t) continue;
          used_at_all = true;
          if (!run_set.count(n)) used_outside = true;
        }
      }
      if (used_outside || !used_at_all) outputs.push_back(t);
    }
    auto rec = std::make_unique<NodeRec>();
    rec->is_delegate_kernel = true;
    rec->replaced = run;
    rec->reg = registration;
    rec->dparams.delegate = delegate;
    rec->dparams.nodes_to_replace = MakeIntArray(run);
    rec->dparams.input_tensors = MakeIntArray(inputs);
    rec->dparams.output_tensors = MakeIntArray(outputs);
    rec->node.inputs = MakeIntArray(inputs);
    rec->node.outputs = MakeIntArray(outputs);
    rec->node.builtin_data = &rec->dparams;
    rec->node.delegate = delegate;
    if (registration.init) {
      rec->node.user_data =
          registration.init(ctx, reinterpret_cast<const char*>(&rec->dparams), 0);
      if (rec->node.user_data == reinterpret_cast<void*>(-1)) {
        h->errors += "delegate kernel init failed\n";
        return kTfLiteError;
      }
      rec->initialised = true;
    }
    for (int t : outputs) h->tensors[t].delegate = delegate;
    h->nodes.push_back(std::move(rec));
    new_plan.push_back(static_cast<int>(h->nodes.size()) - 1);
  }
  h->plan = new_plan;
  return kTfLiteOk;
}


// Subgraph::EnsureTensorDataIsReadable (tflite/core/subgraph.cc:876-889).
TfLiteStatus EnsureReadable(Host* h, int tensor_index) {
  TfLiteTensor* t = &h->tensors[tensor_index];
  TfLiteStatus status = kTfLiteOk;
  if (t->data_is_stale) {
    if (!t->delegate || t->buffer_handle == kTfLiteNullBufferHandle ||
        !t->delegate->CopyFromBufferHandle) {
      h->errors += "stale tensor without a delegate buffer handle\n";
      return kTfLiteError;
    }
    status = t->delegate->CopyFromBufferHandle(&h->ctx, t->delegate, t->buffer_handle, t);
    t->data_is_stale = false;
  }
  return status;
}

void FreeDelegateKernels(Host* h) {
  for (auto& n : h->nodes) {
    if (n->is_delegate_kernel && n->initialised && n->reg.free) {
      n->reg.free(&h->ctx, n->node.user_data);
      n->initialised = false;
    }
  }
}

}  // namespace

extern "C" {

void* fh_create() {
  auto* h = new Host();
  h->ctx.impl_ = h;
  h->ctx.GetExecutionPlan = CtxGetExecutionPlan;
  h->ctx.GetNodeAndRegistration = CtxGetNodeAndRegistration;
  h->ctx.ReplaceNodeSubsetsWithDelegateKernels = CtxReplaceNodeSubsets;
  h->ctx.ReportError = CtxReportError;
  h->ctx.recommended_num_threads = 1;
  return h;
}

void fh_destroy(void* hp) {
  auto* h = static_cast<Host*>(hp);
  FreeDelegateKernels(h);
  for (auto& t : h->tensors) {  // Subgraph::~Subgraph (subgraph.cc:310-316)
    if (t.buffer_handle != kTfLiteNullBufferHandle && t.delegate && t.delegate->FreeBufferHandle) {
      t.delegate->FreeBufferHandle(&h->ctx, t.delegate, &t.buffer_handle);
    }
  }
  if (h->delegate && h->destroy) h->destroy(h->delegate);
  for (auto& t : h->tensors) std::free(t.dims);
  for (auto& a : h->affine) {
    std::free(a->scale);
    std::free(a->zero_point);
  }
  std::free(h->plan_array);
  if (h->dl) dlclose(h->dl);
  delete h;
}

// data may be NULL (zero-filled buffer of `bytes`). allocation_type as TfLiteAllocationType.
int fh_add_tensor(void* hp, int type, int ndims, const int* dims, int allocation_type,
                  const void* data, size_t bytes, float scale, int zero_point) {
  auto* h = static_cast<Host*>(hp);
  TfLiteTensor t{};
  t.type = static_cast<TfLiteType>(type);
  t.dims = MakeIntArray(std::vector<int>(dims, dims + ndims));
  t.params.scale = scale;
  t.params.zero_point = zero_point;
  t.allocation_type = static_cast<TfLiteAllocationType>(allocation_type);
  t.bytes = bytes;
  t.buffer_handle = kTfLiteNullBufferHandle;
  auto buf = std::make_unique<std::vector<char>>(bytes ? bytes : 1);
  if (data && bytes) std::memcpy(buf->data(), data, bytes);
  t.data.raw = bytes ? buf->data() : nullptr;
  h->tensors.push_back(t);
  h->buffers.push_back(std::move(buf));
  h->Sync();
  return static_cast<int>(h->tensors.size()) - 1;
}

int fh_set_affine_quantization(void* hp, int tensor, int n, const float* scales,
                               const int* zero_points, int quantized_dimension) {
  auto* h = static_cast<Host*>(hp);
  auto q = std::make_unique<TfLiteAffineQuantization>();
  q->scale = static_cast<TfLiteFloatArray*>(std::malloc(sizeof(TfLiteFloatArray) + sizeof(float) * n));
  q->scale->size = n;
  std::memcpy(q->scale->data, scales, sizeof(float) * n);
  q->zero_point = MakeIntArray(std::vector<int>(zero_points, zero_points + n));
  q->quantized_dimension = quantized_dimension;
  TfLiteTensor& t = h->tensors[tensor];
  t.quantization.type = kTfLiteAffineQuantization;
  t.quantization.params = q.get();
  t.params.scale = scales[0];
  t.params.zero_point = zero_points[0];
  h->affine.push_back(std::move(q));
  return 0;
}

int fh_set_blockwise_quantization(void* hp, int tensor, int scale_tensor, int zero_point_tensor,
                                  int blocksize, int quantized_dimension) {
  auto* h = static_cast<Host*>(hp);
  auto q = std::make_unique<TfLiteBlockwiseQuantization>();
  q->scale = scale_tensor;
  q->zero_point = zero_point_tensor;
  q->blocksize = blocksize;
  q->quantized_dimension = quantized_dimension;
  TfLiteTensor& t = h->tensors[tensor];
  t.quantization.type = kTfLiteBlockwiseQuantization;
  t.quantization.params = q.get();
  h->blockwise.push_back(std::move(q));
  return 0;
}

// bias < 0 with three_inputs != 0 gives the optional-tensor form (index -1).
int fh_add_fc_node(void* hp, int input, int filter, int bias, int three_inputs, int output,
                   int activation, int keep_num_dims, int asymmetric_quantize_inputs,
                   int weights_format, int version) {
  auto* h = static_cast<Host*>(hp);
  auto rec = std::make_unique<NodeRec>();
  std::vector<int> in = {input, filter};
  if (three_inputs) in.push_back(bias < 0 ? kTfLiteOptionalTensor : bias);
  rec->node.inputs = MakeIntArray(in);
  rec->node.outputs = MakeIntArray({output});
  rec->fc.activation = static_cast<TfLiteFusedActivation>(activation);
  rec->fc.weights_format = static_cast<TfLiteFullyConnectedWeightsFormat>(weights_format);
  rec->fc.keep_num_dims = keep_num_dims != 0;
  rec->fc.asymmetric_quantize_inputs = asymmetric_quantize_inputs != 0;
  rec->fc.quantized_bias_type = kTfLiteNoType;
  rec->node.builtin_data = &rec->fc;
  rec->reg.builtin_code = kTfLiteBuiltinFullyConnected;
  rec->reg.version = version;
  h->nodes.push_back(std::move(rec));
  h->plan.push_back(static_cast<int>(h->nodes.size()) - 1);
  return static_cast<int>(h->nodes.size()) - 1;
}

// BATCH_MATMUL (builtin code 126, TfLiteBatchMatMulParams).
int fh_add_batch_matmul_node(void* hp, int lhs, int rhs, int output, int adj_x, int adj_y,
                             int asymmetric_quantize_inputs, int version) {
  auto* h = static_cast<Host*>(hp);
  auto rec = std::make_unique<NodeRec>();
  rec->node.inputs = MakeIntArray({lhs, rhs});
  rec->node.outputs = MakeIntArray({output});
  rec->bmm.adj_x = adj_x != 0;
  rec->bmm.adj_y = adj_y != 0;
  rec->bmm.asymmetric_quantize_inputs = asymmetric_quantize_inputs != 0;
  rec->node.builtin_data = &rec->bmm;
  rec->reg.builtin_code = kTfLiteBuiltinBatchMatmul;
  rec->reg.version = version;
  h->nodes.push_back(std::move(rec));
  h->plan.push_back(static_cast<int>(h->nodes.size()) - 1);
  return static_cast<int>(h->nodes.size()) - 1;
}

// Any other operator (the delegate must leave it alone).
int fh_add_other_node(void* hp, int builtin_code, int input, int output) {
  auto* h = static_cast<Host*>(hp);
  auto rec = std::make_unique<NodeRec>();
  rec->node.inputs = MakeIntArray({input});
  rec->node.outputs = MakeIntArray({output});
  rec->reg.builtin_code = builtin_code;
  rec->reg.version = 1;
  h->nodes.push_back(std::move(rec));
  h->plan.push_back(static_cast<int>(h->nodes.size()) - 1);
  return static_cast<int>(h->nodes.size()) - 1;
}

// EMBEDDING_LOOKUP (builtin code 7): inputs {lookup, table}, no builtin options.
int fh_add_embedding_lookup_node(void* hp, int lookup, int value, int output) {
  auto* h = static_cast<Host*>(hp);
  auto rec = std::make_unique<NodeRec>();
  rec->node.inputs = MakeIntArray({lookup, value});
  rec->node.outputs = MakeIntArray({output});
  rec->reg.builtin_code = 7;
  rec->reg.version = 1;
  h->nodes.push_back(std::move(rec));
  h->plan.push_back(static_cast<int>(h->nodes.size()) - 1);
  return static_cast<int>(h->nodes.size()) - 1;
}

void fh_mark_graph_output(void* hp, int tensor) { static_cast<Host*>(hp)->graph_outputs.insert(tensor); }
void fh_set_cpu_callback(void* hp, CpuCallback cb) { static_cast<Host*>(hp)->cpu = cb; }

// dlopen + tflite_plugin_create_delegate. Returns 0, or 1 with the reason in fh_errors().
int fh_load_delegate(void* hp, const char* path, const char* const* keys,
                     const char* const* values, size_t n) {
  auto* h = static_cast<Host*>(hp);
  h->dl = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!h->dl) {
    h->errors += std::string("dlopen: ") + dlerror() + "\n";
    return 1;
  }
  h->create = reinterpret_cast<CreateFn>(dlsym(h->dl, "tflite_plugin_create_delegate"));
  h->destroy = reinterpret_cast<DestroyFn>(dlsym(h->dl, "tflite_plugin_destroy_delegate"));
  if (!h->create || !h->destroy) {
    h->errors += "plugin entry points missing\n";
    return 1;
  }
  g_plugin_error.clear();
  h->delegate = h->create(keys, values, n, PluginError);
  if (!h->delegate) {
    h->errors += "create_delegate returned NULL: " + g_plugin_error + "\n";
    return 1;
  }
  return 0;
}

// Interpreter::ModifyGraphWithDelegate: on failure the original plan is restored and
// kTfLiteDelegateError returned (tflite/core/subgraph.cc:2508-2517).
int fh_modify_graph_with_delegate(void* hp) {
  auto* h = static_cast<Host*>(hp);
  if (!h->delegate) return kTfLiteError;
  h->original_plan = h->plan;
  const size_t nodes_before = h->nodes.size();
  const TfLiteStatus st = h->delegate->Prepare(&h->ctx, h->delegate);
  if (st != kTfLiteOk) {
    FreeDelegateKernels(h);
    h->plan = h->original_plan;
    h->nodes.resize(nodes_before);
    for (auto& t : h->tensors) t.delegate = nullptr;
    return kTfLiteDelegateError;
  }
  return kTfLiteOk;
}

int fh_allocate_tensors(void* hp) {
  auto* h = static_cast<Host*>(hp);
  for (int n : h->plan) {
    NodeRec& rec = *h->nodes[n];
    if (rec.is_delegate_kernel && rec.reg.prepare) {
      const TfLiteStatus st = rec.reg.prepare(&h->ctx, &rec.node);
      if (st != kTfLiteOk) return st;
    }
  }
  return kTfLiteOk;
}

int fh_invoke(void* hp) {
  auto* h = static_cast<Host*>(hp);
  for (int n : h->plan) {
    NodeRec& rec = *h->nodes[n];
    // Inputs another party left in its own memory are fetched first (subgraph.cc:1724-1734).
    for (int i = 0; i < rec.node.inputs->size; ++i) {
      const int t = rec.node.inputs->data[i];
      if (t == kTfLiteOptionalTensor) continue;
      TfLiteTensor& tensor = h->tensors[t];
      if (tensor.delegate && tensor.delegate != rec.node.delegate && tensor.data_is_stale) {
        if (EnsureReadable(h, t) != kTfLiteOk) return kTfLiteError;
      }
    }
    if (rec.is_delegate_kernel) {
      const TfLiteStatus st = rec.reg.invoke(&h->ctx, &rec.node);
      if (st != kTfLiteOk) return st;
    } else {
      if (!h->cpu) {
        h->errors += "node left on the CPU but no CPU callback set\n";
        return kTfLiteError;
      }
      if (h->cpu(n) != 0) return kTfLiteError;
    }
  }
  return kTfLiteOk;
}

// Interpreter::SetBufferHandle with the loaded delegate (subgraph.cc:2784-2800).
int fh_set_buffer_handle(void* hp, int tensor, int handle) {
  auto* h = static_cast<Host*>(hp);
  TfLiteTensor& t = h->tensors[tensor];
  if (!h->delegate || (t.delegate && t.delegate != h->delegate)) return kTfLiteError;
  t.delegate = h->delegate;
  if (t.buffer_handle != kTfLiteNullBufferHandle && h->delegate->FreeBufferHandle) {
    h->delegate->FreeBufferHandle(&h->ctx, h->delegate, &t.buffer_handle);
  }
  t.buffer_handle = handle;
  return kTfLiteOk;
}
void fh_set_data_is_stale(void* hp, int tensor, int stale) {
  static_cast<Host*>(hp)->tensors[tensor].data_is_stale = stale != 0;
}
int fh_data_is_stale(void* hp, int tensor) {
  return static_cast<Host*>(hp)->tensors[tensor].data_is_stale ? 1 : 0;
}
int fh_buffer_handle(void* hp, int tensor) { return static_cast<Host*>(hp)->tensors[tensor].buffer_handle; }
int fh_ensure_tensor_data_is_readable(void* hp, int tensor) {
  return EnsureReadable(static_cast<Host*>(hp), tensor);
}
void* fh_delegate(void* hp) { return static_cast<Host*>(hp)->delegate; }
// TfLiteDelegate::CopyToBufferHandle on the tensor's own handle.
int fh_copy_to_buffer_handle(void* hp, int tensor) {
  auto* h = static_cast<Host*>(hp);
  TfLiteTensor& t = h->tensors[tensor];
  if (!t.delegate || !t.delegate->CopyToBufferHandle) return kTfLiteError;
  return t.delegate->CopyToBufferHandle(&h->ctx, t.delegate, t.buffer_handle, &t);
}

void* fh_tensor_data(void* hp, int tensor) { return static_cast<Host*>(hp)->tensors[tensor].data.raw; }
size_t fh_tensor_bytes(void* hp, int tensor) { return static_cast<Host*>(hp)->tensors[tensor].bytes; }

// Gives the tensor a fresh buffer at a new address (contents preserved), as the arena
// may between invokes.
void fh_move_tensor_data(void* hp, int tensor) {
  auto* h = static_cast<Host*>(hp);
  auto fresh = std::make_unique<std::vector<char>>(*h->buffers[tensor]);
  h->tensors[tensor].data.raw = h->tensors[tensor].bytes ? fresh->data() : nullptr;
  std::memset(h->buffers[tensor]->data(), 0x5A, h->buffers[tensor]->size());  // poison the old one
  h->buffers.push_back(std::move(h->buffers[tensor]));                        // keep it alive
  h->buffers[tensor] = std::move(fresh);
}

void fh_resize_tensor(void* hp, int tensor, int ndims, const int* dims, size_t bytes) {
  auto* h = static_cast<Host*>(hp);
  TfLiteTensor& t = h->tensors[tensor];
  std::free(t.dims);
  t.dims = MakeIntArray(std::vector<int>(dims, dims + ndims));
  t.bytes = bytes;
  h->buffers[tensor] = std::make_unique<std::vector<char>>(bytes ? bytes : 1);
  t.data.raw = bytes ? h->buffers[tensor]->data() : nullptr;
}

int fh_plan_size(void* hp) { return static_cast<int>(static_cast<Host*>(hp)->plan.size()); }
int fh_plan_node(void* hp, int i) { return static_cast<Host*>(hp)->plan[i]; }
int fh_node_is_delegate_kernel(void* hp, int node) {
  return static_cast<Host*>(hp)->nodes[node]->is_delegate_kernel ? 1 : 0;
}
int fh_node_num_replaced(void* hp, int node) {
  return static_cast<int>(static_cast<Host*>(hp)->nodes[node]->replaced.size());
}
int fh_node_replaced(void* hp, int node, int i) { return static_cast<Host*>(hp)->nodes[node]->replaced[i]; }
int fh_node_num_inputs(void* hp, int node) { return static_cast<Host*>(hp)->nodes[node]->node.inputs->size; }
int fh_node_input(void* hp, int node, int i) { return static_cast<Host*>(hp)->nodes[node]->node.inputs->data[i]; }
int fh_node_num_outputs(void* hp, int node) { return static_cast<Host*>(hp)->nodes[node]->node.outputs->size; }
int fh_node_output(void* hp, int node, int i) { return static_cast<Host*>(hp)->nodes[node]->node.outputs->data[i]; }
int fh_tensor_has_delegate(void* hp, int tensor) {
  return static_cast<Host*>(hp)->tensors[tensor].delegate != nullptr;
}
void* fh_node_user_data(void* hp, int node) { return static_cast<Host*>(hp)->nodes[node]->node.user_data; }
// What the node's registration reports to a profiler (profile_summarizer.cc:84-88 calls it
// with the interpreter's context and the node); nullptr when the registration has none.
const char* fh_node_profiling_string(void* hp, int node) {
  auto* h = static_cast<Host*>(hp);
  const auto& rec = h->nodes[node];
  if (!rec->reg.profiling_string) return nullptr;
  return rec->reg.profiling_string(&h->ctx, &rec->node);
}
int fh_replace_calls(void* hp) { return static_cast<Host*>(hp)->replace_calls; }
const char* fh_errors(void* hp) { return static_cast<Host*>(hp)->errors.c_str(); }
void fh_clear_errors(void* hp) { static_cast<Host*>(hp)->errors.clear(); }

// Runs the plugin's claim predicate on one node without a device (the plugin exports it
// for exactly this). Needs only dlopen, not create_delegate.
int fh_classify(void* hp, const char* plugin_path, int node, char* reason, size_t reason_size) {
  auto* h = static_cast<Host*>(hp);
  void* dl = dlopen(plugin_path, RTLD_NOW | RTLD_LOCAL);
  if (!dl) {
    h->errors += std::string("dlopen: ") + dlerror() + "\n";
    return -1;
  }
  typedef int (*ClassifyFn)(const TfLiteContext*, const TfLiteNode*, const TfLiteRegistration*,
                            char*, size_t);
  auto fn = reinterpret_cast<ClassifyFn>(dlsym(dl, "litert_amd_classify_node"));
  if (!fn) return -1;
  const int kind = fn(&h->ctx, &h->nodes[node]->node, &h->nodes[node]->reg, reason, reason_size);
  dlclose(dl);
  return kind;
}

}  // extern "C"

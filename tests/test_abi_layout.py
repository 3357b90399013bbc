"""Layout check of include/tflite_abi.h against the reference's own C headers: every struct
the delegate touches must have the same size and member offsets, every enum value the same
number. Runs only where the reference tree is mounted (it is compiled, not copied)."""
import os
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"

STRUCTS = {
    "TfLiteQuantizationParams": ["scale", "zero_point"],
    "TfLiteQuantization": ["type", "params"],
    "TfLiteAffineQuantization": ["scale", "zero_point", "quantized_dimension"],
    "TfLiteBlockwiseQuantization": ["scale", "zero_point", "blocksize", "quantized_dimension"],
    "TfLiteIntArray": ["size", "data"],
    "TfLiteFloatArray": ["size", "data"],
    "TfLiteTensor": ["type", "data", "dims", "params", "allocation_type", "bytes", "allocation",
                     "name", "delegate", "buffer_handle", "data_is_stale", "is_variable",
                     "quantization", "sparsity", "dims_signature"],
    "TfLiteNode": ["inputs", "outputs", "intermediates", "temporaries", "user_data", "builtin_data",
                   "custom_initial_data", "custom_initial_data_size", "delegate",
                   "might_have_side_effect"],
    "TfLiteDelegateParams": ["delegate", "nodes_to_replace", "input_tensors", "output_tensors"],
    "TfLiteRegistration": ["init", "free", "prepare", "invoke", "profiling_string", "builtin_code",
                           "custom_name", "version", "registration_external", "async_kernel",
                           "inplace_operator"],
    "TfLiteContext": ["tensors_size", "GetExecutionPlan", "tensors", "impl_", "ResizeTensor",
                      "ReportError", "AddTensors", "GetNodeAndRegistration",
                      "ReplaceNodeSubsetsWithDelegateKernels", "recommended_num_threads",
                      "GetExternalContext", "SetExternalContext", "allow_fp32_relax_to_fp16",
                      "profiler", "AllocatePersistentBuffer", "AllocateBufferForEval",
                      "RequestScratchBufferInArena", "GetScratchBuffer", "ResizeTensorExplicit",
                      "PreviewDelegatePartitioning", "GetTensor", "GetEvalTensor",
                      "GetModelMetadata", "AcquireSubgraphContext", "ReleaseSubgraphContext"],
    "TfLiteDelegate": ["data_", "Prepare", "CopyFromBufferHandle", "CopyToBufferHandle",
                       "FreeBufferHandle", "flags", "opaque_delegate_builder"],
    "TfLiteFullyConnectedParams": ["activation", "weights_format", "keep_num_dims",
                                   "asymmetric_quantize_inputs", "quantized_bias_type"],
    "TfLiteSparsity": ["traversal_order", "block_map", "dim_metadata", "dim_metadata_size"],
}
ENUMS = ["kTfLiteOk", "kTfLiteError", "kTfLiteDelegateError", "kTfLiteApplicationError",
         "kTfLiteFloat32", "kTfLiteInt32", "kTfLiteUInt8", "kTfLiteInt64", "kTfLiteInt16",
         "kTfLiteInt8", "kTfLiteFloat16", "kTfLiteInt4", "kTfLiteInt2", "kTfLiteNoQuantization",
         "kTfLiteAffineQuantization", "kTfLiteBlockwiseQuantization", "kTfLiteMmapRo",
         "kTfLiteArenaRw", "kTfLiteArenaRwPersistent", "kTfLiteDynamic", "kTfLitePersistentRo",
         "kTfLiteCustom", "kTfLiteActNone", "kTfLiteActRelu", "kTfLiteActReluN1To1",
         "kTfLiteActRelu6", "kTfLiteActTanh", "kTfLiteActSignBit", "kTfLiteActSigmoid",
         "kTfLiteFullyConnectedWeightsFormatDefault",
         "kTfLiteFullyConnectedWeightsFormatShuffled4x16Int8", "kTfLiteBuiltinFullyConnected",
         "kTfLiteBuiltinDelegate", "kTfLiteDelegateFlagsNone",
         "kTfLiteDelegateFlagsAllowDynamicTensors", "kTfLiteOptionalTensor",
         "kTfLiteNullBufferHandle"]


@pytest.mark.skipif(not os.path.exists(os.path.join(REF, "tflite/core/c/common.h")),
                    reason="reference tree not mounted")
def test_abi_layout_matches_reference_headers():
    lines = ["#include <cstddef>", "#include <cstdint>", "#include <stdbool.h>",
             '#include "tflite/core/c/common.h"', '#include "tflite/core/c/builtin_op_data.h"',
             '#include "tflite/builtin_ops.h"',
             "namespace mine {", '#include "tflite_abi.h"', "}"]
    for name, members in STRUCTS.items():
        lines.append("static_assert(sizeof(::%s) == sizeof(mine::%s), \"sizeof %s\");"
                     % (name, name, name))
        for m in members:
            lines.append("static_assert(offsetof(::%s, %s) == offsetof(mine::%s, %s), \"%s.%s\");"
                         % (name, m, name, m, name, m))
    for e in ENUMS:
        if e == "kTfLiteOptionalTensor":
            continue  # a macro in both headers: same token, checked by value below
        lines.append("static_assert(static_cast<long>(::%s) == static_cast<long>(mine::%s), \"%s\");"
                     % (e, e, e))
    lines.append("static_assert(kTfLiteOptionalTensor == -1, \"optional tensor index\");")
    lines.append("int main() { return 0; }")
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "abi_check.cc")
        open(src, "w").write("\n".join(lines) + "\n")
        r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wno-invalid-offsetof",
                            "-I" + REF, "-I" + os.path.join(ROOT, "include"), src],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-4000:]

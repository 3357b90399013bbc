"""Builds the native libraries of litert_amd for gfx950 with hipcc, in-tree.

    python -m litert_amd.build            # everything
    python -m litert_amd.build --only fc  # just the kernel library

Outputs land in litert_amd/lib/ (git-ignored; they travel to the GPU box with the tree).
"""
import argparse
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.environ.get("LITERT_AMD_LIB_DIR", os.path.join(HERE, "lib"))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: several float steps reproduce the reference's unfused
# multiply-then-add; packed-fp32 ops are disabled (they have misbehaved on this pool).
COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall",
          "-Wno-unused-function", "-I" + os.path.join(ROOT, "include")]
# Kernel-argument preloading (gfx940 and later): the leading scalar arguments of a kernel
# arrive in registers with the wavefront instead of through a first round of scalar loads.
COMMON += ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
COMMON += os.environ.get("LITERT_AMD_EXTRA_HIPCC_FLAGS", "").split()

FC_SOURCES = ["capi.hip", "quantize.hip", "fc_int8_gemv.hip", "fc_int8_packed_gemv.hip", "fc_int8_rows_gemv.hip", "fc_int8_packed_gemm.hip",
              "fc_int8_gemm_mfma.hip", "fc_int4_blockwise.hip", "fc_int4_packed.hip", "fc_int4_per_channel_gemv.hip",
              "embedding_lookup.hip", "fc_int4_blockwise_gemm.hip"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


# Per-file additions. The blockwise int4 GEMM reads every MFMA result with the vector ALU right
# away (one MFMA per quantization block), so its results should land in ordinary vector
# registers: with the default choice of accumulation registers each of them costs a copy
# instruction first (a quarter of the kernel's vector work).
FILE_FLAGS = {"fc_int4_blockwise_gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def build_fc():
    os.makedirs(LIB, exist_ok=True)
    objs = []
    procs = []
    for src in FC_SOURCES:
        obj = os.path.join(LIB, src.replace(".hip", ".o"))
        cmd = [HIPCC] + COMMON + FILE_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd)))
        objs.append(obj)
    for src, p in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed on " + src)
    out = os.path.join(LIB, "liblitert_amd_fc.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs)
    return out


def build_delegate():
    src_dir = os.path.join(CSRC, "delegate")
    if not os.path.isdir(src_dir):
        return None
    srcs = sorted(os.path.join(src_dir, f) for f in os.listdir(src_dir) if f.endswith(".cc"))
    if not srcs:
        return None
    out = os.path.join(LIB, "liblitert_amd_delegate.so")
    _run([HIPCC, "-x", "hip"] + COMMON + ["-shared", "-o", out] + srcs +
         ["-L" + LIB, "-llitert_amd_fc", "-Wl,-rpath,$ORIGIN"])
    return out


def build_bench_probes():
    """The benchmark's measurement aids: a library of their own, not linked into the others."""
    os.makedirs(LIB, exist_ok=True)
    out = os.path.join(LIB, "liblitert_amd_bench_probes.so")
    _run([HIPCC] + COMMON + ["-shared", "-o", out, os.path.join(HERE, "bench_probes", "probes.hip")])
    return out


def build_all():
    outs = [build_fc(), build_bench_probes()]
    d = build_delegate()
    if d:
        outs.append(d)
    return outs


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", choices=["fc", "delegate", "probes"])
    args = ap.parse_args()
    if args.only == "fc":
        build_fc()
    elif args.only == "delegate":
        build_delegate()
    elif args.only == "probes":
        build_bench_probes()
    else:
        build_all()
    sys.exit(0)

"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer (CPU only; the reference's
own sanitizer build is ci/build_litert_runtime_cmake_asan.sh:56-73): the oracle, the stand-in
host and the delegate plugin's host side are rebuilt with -fsanitize=address,undefined and the
CPU tests that exercise them (the oracle's known-answer tests, the delegate's claim / option /
partition tests) run again against those builds in a child process. Any sanitizer report fails
the test. GPU code is not instrumented."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SUITES = ["tests/test_oracle_kat.py", "tests/test_oracle_blockwise.py",
          "tests/test_oracle_int4_per_channel.py", "tests/test_delegate_cpu.py",
          "tests/test_litert_accelerator.py"]


def _libasan():
    out = subprocess.run(["g++", "-print-file-name=libasan.so"], capture_output=True, text=True)
    path = out.stdout.strip()
    return os.path.realpath(path) if os.path.isabs(path) and os.path.exists(path) else None


def test_cpu_suites_pass_under_asan_and_ubsan():
    asan = _libasan()
    if asan is None:
        pytest.skip("g++ has no libasan.so here")
    if not os.path.exists(os.path.join(ROOT, "litert_amd", "lib", "liblitert_amd_fc.so")):
        pytest.skip("the kernel library is not built (the delegate links against it)")
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "san"])
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "litert_amd", "standin_host"),
                           "san"])
    env = dict(os.environ)
    env["LITERT_AMD_SANITIZED"] = "1"
    # The runtime must be in the process before the instrumented libraries are loaded by
    # ctypes; whatever the environment already preloads stays in the list.
    env["LD_PRELOAD"] = ":".join(x for x in (asan, env.get("LD_PRELOAD", "")) if x)
    # Python itself is not leak-clean; link order is checked off because other preloads may exist.
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:abort_on_error=0"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    run = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p",
                          "no:cacheprovider"] + SUITES, cwd=ROOT, env=env, capture_output=True,
                         text=True, timeout=900)
    text = run.stdout + run.stderr
    assert "AddressSanitizer" not in text and "runtime error:" not in text, text[-4000:]
    assert run.returncode == 0, text[-4000:]
    assert " passed" in text

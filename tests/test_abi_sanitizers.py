"""The host side of libarctic_mi355x under AddressSanitizer and UBSan: ``tests/native/abi_host_fuzz.cpp`` calls
every entry point of the C ABI with seeded random sizes, pitches, type codes and pointers.  It is built from the
library's own sources with the sanitizers on the host pass only and runs where there is no GPU: a call is turned
away or fails at the launch, and either way returns a code and a message and trips no sanitizer."""
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "arcticinference_amd", "csrc")


@pytest.fixture(scope="module")
def fuzz_binary(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    out = str(tmp_path_factory.mktemp("abi_host_fuzz") / "abi_host_fuzz")
    kernels = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    cmd = [hipcc, "--offload-arch=gfx950", "-parallel-jobs=8", "-O1", "-g", "-std=c++17",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-o", out,
           os.path.join(ROOT, "tests", "native", "abi_host_fuzz.cpp"), *kernels,
           "-x", "hip", os.path.join(CSRC, "error.cpp")]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=os.path.dirname(out))
    assert proc.returncode == 0, proc.stderr[-4000:]
    return out


@pytest.mark.parametrize("seed", [1, 2])
def test_random_arguments_are_clean_under_asan_and_ubsan(fuzz_binary, seed):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([fuzz_binary, str(seed), "20000"], capture_output=True, text=True, env=env, timeout=300)
    text = proc.stdout + proc.stderr
    assert proc.returncode == 0, text[-4000:]
    if proc.stdout.startswith("skipped"):
        pytest.skip("a GPU is present: fake device pointers must not reach a kernel")
    assert proc.stdout.startswith("ok "), text[-4000:]
    launched = int(proc.stdout.split("message,")[1].split()[0])
    assert launched > 500, "the fuzzer should get past the argument checks in a fair share of its calls: " + proc.stdout

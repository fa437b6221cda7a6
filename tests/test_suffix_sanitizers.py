"""The suffix tree's C++ under AddressSanitizer and UndefinedBehaviorSanitizer: ``tests/native/suffix_stress.cpp``
(seeded random appends, extends, removals and drafts through the C ABI, the tree's integrity check after every
batch) is compiled together with ``csrc/suffix_tree.cpp`` by g++ with both sanitizers and run over a few seeds.
Host code only; nothing here touches a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def stress_binary(tmp_path_factory):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("g++ not found")
    out = str(tmp_path_factory.mktemp("suffix_stress") / "suffix_stress")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-static-libasan", "-I", os.path.join(ROOT, "include"), "-o", out,
           os.path.join(ROOT, "tests", "native", "suffix_stress.cpp"),
           os.path.join(ROOT, "arcticinference_amd", "csrc", "suffix_tree.cpp")]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0 and "asan" in proc.stderr.lower() and "cannot find" in proc.stderr.lower():
        pytest.skip("the sanitizer runtimes are not installed: " + proc.stderr.strip().splitlines()[-1])
    assert proc.returncode == 0, proc.stderr
    return out


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_operations_are_clean_under_asan_and_ubsan(stress_binary, seed):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([stress_binary, str(seed), "1500"], capture_output=True, text=True, env=env, timeout=300)
    assert proc.returncode == 0 and proc.stdout.strip() == "ok", (proc.stdout + proc.stderr)[-4000:]

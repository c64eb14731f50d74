"""The native host code under AddressSanitizer and UndefinedBehaviorSanitizer, on the CPU: the cache
core, the generation bookkeeping and the kernels' plain C++ references are compiled together with a
C++ driver (tests/native/sanitize_host.cpp: random cache traffic with the books checked after every
move, step assembly, refused arguments, generations with stop tokens that run ahead, planning) and
run without Python or ctypes in between.  The reference gets the same assurance from its language
(crates/burn-lm-llama/src/nn/attention/cache.rs:56-149, generation/context.rs:116-171)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "burn-lm_amd", "csrc")


def test_host_core_generation_and_references_are_clean_under_the_sanitizers(tmp_path):
    cxx = shutil.which(os.environ.get("CXX", "g++")) or shutil.which("c++")
    if cxx is None:
        pytest.skip("no C++ compiler")
    host = os.path.join(CSRC, "host")
    sources = [os.path.join(ROOT, "tests", "native", "sanitize_host.cpp"), os.path.join(CSRC, "ref", "reference.cpp")]
    sources += sorted(os.path.join(host, f) for f in os.listdir(host) if f.endswith(".cpp"))
    exe = str(tmp_path / "sanitize_host")
    flags = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer"]
    # the sanitizer's runtime linked in: a library that the environment preloads must not come before it
    build = subprocess.run([cxx, *flags, "-static-libasan", "-I", host, *sources, "-o", exe], capture_output=True, text=True)
    if build.returncode != 0 and "static-libasan" in build.stderr:
        build = subprocess.run([cxx, *flags, "-I", host, *sources, "-o", exe], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode == 0, (run.stdout + run.stderr)[-6000:]
    assert "native host code: clean" in run.stdout

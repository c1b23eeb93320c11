"""The engine's host library under AddressSanitizer and UndefinedBehaviorSanitizer: built with
them into a temporary folder, loaded in a child process in place of the ordinary build, and
driven by the cache, step-plan and generation-loop tests (none of which needs a GPU)."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
sys.path.insert(0, {root!r})
import tq_kv_amd.csrc.build as build
build.find_host_library = lambda: {lib!r}
build.ensure_host_built = lambda *a, **k: {lib!r}
import pytest
rc = pytest.main(["-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] + {tests!r})
loaded = [line.split()[-1] for line in open("/proc/self/maps") if "tqengine" in line]
assert loaded and all(p == {lib!r} for p in loaded), loaded
sys.exit(rc)
"""


def test_host_library_is_clean_under_address_and_ub_sanitizers(tmp_path):
    cxx = shutil.which("g++")
    if cxx is None:
        pytest.skip("no g++")
    runtimes = [subprocess.run([cxx, "-print-file-name=" + n], capture_output=True, text=True).stdout.strip()
                for n in ("libasan.so", "libubsan.so")]
    if not all(os.path.isabs(p) and os.path.exists(p) for p in runtimes):
        pytest.skip("this g++ has no sanitizer runtimes")
    lib = str(tmp_path / "libtqengine_sanitized.so")
    src = os.path.join(ROOT, "tq_kv_amd", "csrc", "host_engine.cpp")
    built = subprocess.run([cxx, "-O1", "-g", "-fPIC", "-std=c++17", "-shared", "-Wall", "-fsanitize=address,undefined",
                            "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", src, "-o", lib], capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    tests = [os.path.join(ROOT, "tests", n) for n in ("test_cache.py", "test_step_plan.py", "test_generate_loop.py")]
    env = dict(os.environ, LD_PRELOAD=" ".join(runtimes), ASAN_OPTIONS="detect_leaks=0:abort_on_error=1")
    child = subprocess.run([sys.executable, "-c", CHILD.format(root=ROOT, lib=lib, tests=tests)], capture_output=True, text=True, env=env,
                           timeout=600)
    assert child.returncode == 0, child.stdout[-3000:] + child.stderr[-3000:]
    assert "passed" in child.stdout and "ERROR: AddressSanitizer" not in child.stderr and "runtime error" not in child.stderr

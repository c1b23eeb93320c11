"""The engine library under AddressSanitizer and UndefinedBehaviorSanitizer: built with them into a
temporary folder, loaded in a child process in place of the ordinary build, and driven by the tests
that need no GPU: configuration, weights and their errors (models in host memory), the cache, the
step's arrays, the generation loop over stand-in engines and samplers, and whole steps and generation of models on
the null device (every line of the engine that is not a kernel)."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
sys.path.insert(0, {root!r})
import pytest
rc = pytest.main(["-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] + {tests!r})
loaded = [line.split()[-1] for line in open("/proc/self/maps") if "tqengine" in line]
assert loaded and all(p == {lib!r} for p in loaded), loaded
sys.exit(rc)
"""


def test_host_library_is_clean_under_address_and_ub_sanitizers(tmp_path):
    from tq_kv_amd.csrc import build
    cxx = shutil.which("g++")
    if cxx is None:
        pytest.skip("no g++")
    runtimes = [subprocess.run([cxx, "-print-file-name=" + n], capture_output=True, text=True).stdout.strip()
                for n in ("libasan.so", "libubsan.so")]
    if not all(os.path.isabs(p) and os.path.exists(p) for p in runtimes):
        pytest.skip("this g++ has no sanitizer runtimes")
    build.ensure_built(verbose=False)             # the kernel library (not sanitized) answers the engine's questions about sizes
    lib = str(tmp_path / "libtqengine_sanitized.so")
    os.environ.setdefault("CXX", cxx)
    build.compile_host(lib, extra_flags=["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"])
    tests = [os.path.join(ROOT, "tests", n) for n in ("test_cache.py", "test_step_plan.py", "test_generate_loop.py", "test_config.py",
                                                      "test_weights.py", "test_dry_run.py")]
    env = dict(os.environ, LD_PRELOAD=" ".join(runtimes), ASAN_OPTIONS="detect_leaks=0:abort_on_error=1",
               TQ_KERNEL_LIBRARY=build.find_library(), TQ_ENGINE_LIBRARY=lib)
    child = subprocess.run([sys.executable, "-c", CHILD.format(root=ROOT, lib=lib, tests=tests)], capture_output=True, text=True, env=env,
                           timeout=900)
    assert child.returncode == 0, child.stdout[-3000:] + child.stderr[-3000:]
    assert "passed" in child.stdout and "ERROR: AddressSanitizer" not in child.stderr and "runtime error" not in child.stderr

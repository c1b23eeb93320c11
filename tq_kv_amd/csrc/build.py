"""Building the gfx950 kernel library with hipcc, in the source tree.

`build()` compiles every source beside this file into one shared library next to
them.  `ensure_built()` is what loaders call: it builds only if there is no library
that matches the sources (the library's name carries a hash of the sources), and
prints a line now and then while hipcc runs, because a first build takes a while.
If the source tree cannot be written, the library goes to a per-user folder under
the system's temporary directory.
"""
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["host.cpp", "elementwise.hip", "gemm_generic.hip", "attention_generic.hip", "sampling.hip",
           "attention_decode.hip", "attention_prefill.hip", "skinny_fused.hip", "mid_product.hip", "random_init.hip", "utility.hip", "probe.hip"]
HEADERS = ["common.h", "tq_kernels.h", "tq_no_alloc.h"]
# the engine: host code only (config, weights, parts, model, cache, step, loop), built with the host compiler into a
# library of its own that reaches the GPU through the HIP runtime, hipBLASLt and the kernel library above
HOST_SOURCES = ["host_engine.cpp"] + ["engine/" + n for n in (
    "api.cpp", "config.cpp", "core.cpp", "engine.cpp", "generate.cpp", "json.cpp", "linear.cpp", "model.cpp", "parts_builtin.cpp",
    "plugin.cpp", "qwen2.cpp", "spec.cpp", "step.cpp", "store.cpp", "trace.cpp", "weights.cpp")]
HOST_HEADERS = ["tq_engine.h"] + ["engine/" + n for n in (
    "config.h", "core.h", "engine.h", "generate.h", "json.h", "kernels.h", "linear.h", "model.h", "parts.h", "plugin.h", "spec.h",
    "step.h", "store.h", "trace.h", "weights.h")]
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
# no contraction of a multiplication with the addition after it: the random weights' recipe needs each rounded on its own
HOST_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-Wall", "-ffp-contract=off", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROCM, "include")]
HOST_LINK = ["-shared", "-L" + os.path.join(ROCM, "lib"), "-Wl,-rpath," + os.path.join(ROCM, "lib"), "-lamdhip64", "-lhipblaslt", "-ldl", "-lpthread"]
ARCH = "gfx950"
# Packed float32 instructions are switched off for all device code.
HIPCC_FLAGS = ["-O3", "-fPIC", "-std=c++17", "--offload-arch=" + ARCH,
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-result", "-Wno-unknown-attributes"]


class BuildError(RuntimeError):
    pass


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found: the HIP kernels cannot be built (looked in $HIPCC, PATH, /opt/rocm/bin)")


def source_hash():
    h = hashlib.sha256()
    for name in sorted(SOURCES + HEADERS):
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:12]


def library_name():
    return "libtqkernels_%s.so" % source_hash()


def host_source_hash():
    h = hashlib.sha256()
    for name in sorted(HOST_SOURCES + HOST_HEADERS):
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(HOST_FLAGS + HOST_LINK).encode())
    return h.hexdigest()[:12]


def host_library_name():
    return "libtqengine_%s.so" % host_source_hash()


def _writable(folder):
    try:
        os.makedirs(folder, exist_ok=True)
        probe = tempfile.NamedTemporaryFile(dir=folder, prefix=".probe", delete=True)
        probe.close()
        return True
    except OSError:
        return False


def _fallback_dir():
    return os.path.join(tempfile.gettempdir(), "tq_kv_amd_build_%d" % os.getuid())


def find_library():
    """Path of a built library that matches the sources, or None."""
    name = library_name()
    for folder in (HERE, _fallback_dir()):
        path = os.path.join(folder, name)
        if os.path.exists(path):
            return path
    return None


def find_host_library():
    """Path of a built engine library that matches the sources, or None.  TQ_ENGINE_LIBRARY names another build of it outright (a
    sanitizer build, for instance)."""
    if os.environ.get("TQ_ENGINE_LIBRARY"):
        return os.environ["TQ_ENGINE_LIBRARY"]
    name = host_library_name()
    for folder in (HERE, _fallback_dir()):
        path = os.path.join(folder, name)
        if os.path.exists(path):
            return path
    return None


def _host_compiler():
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"), "/opt/rocm/llvm/bin/clang++"):
        if cand and (os.path.exists(cand) or shutil.which(cand)):
            return cand
    raise BuildError("no C++ compiler found for the engine's host library (looked in $CXX, g++, c++, clang++)")


def build_host(force=True, verbose=True):
    """Compile the engine's host library (seconds; needs no GPU toolchain).  Returns its path."""
    existing = find_host_library()
    if existing and not force:
        return existing
    out_dir = HERE if _writable(HERE) else _fallback_dir()
    if not _writable(out_dir):
        raise BuildError("cannot write the engine library to %s or %s" % (HERE, out_dir))
    target = os.path.join(out_dir, host_library_name())
    tmp = target + ".tmp%d" % os.getpid()
    compile_host(tmp, verbose=verbose)
    os.replace(tmp, target)
    for name in os.listdir(out_dir):
        if name.startswith("libtqengine_") and name.endswith(".so") and name != os.path.basename(target):
            try:
                os.remove(os.path.join(out_dir, name))
            except OSError:
                pass
    if verbose:
        print("[tq_kv_amd build] built %s" % target, file=sys.stderr, flush=True)
    return target


def compile_host(target, extra_flags=(), obj_dir=None, verbose=False):
    """Compile the engine's sources (in parallel) and link them into `target`.  extra_flags: more compiler and linker
    flags (a sanitizer build).  Objects go to obj_dir (default: a folder beside the target that is removed afterwards)."""
    cxx = _host_compiler()
    own = obj_dir is None
    if own:
        obj_dir = tempfile.mkdtemp(prefix="tq_host_obj_", dir=os.path.dirname(os.path.abspath(target)))
    os.makedirs(obj_dir, exist_ok=True)
    errors, objects, threads = [], [], []
    gate = threading.Semaphore(max(1, min(8, os.cpu_count() or 1)))

    def compile_one(src, obj):
        with gate:
            proc = subprocess.run([cxx] + HOST_FLAGS + list(extra_flags) + ["-I", HERE, "-c", os.path.join(HERE, src), "-o", obj],
                                  stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            errors.append("the host compiler failed on %s:\n%s" % (src, proc.stdout))

    try:
        for src in HOST_SOURCES:
            obj = os.path.join(obj_dir, src.replace("/", "_").rsplit(".", 1)[0] + ".o")
            objects.append(obj)
            th = threading.Thread(target=compile_one, args=(src, obj))
            th.start()
            threads.append(th)
        for th in threads:
            th.join()
        if errors:
            raise BuildError(errors[0])
        proc = subprocess.run([cxx] + list(extra_flags) + objects + HOST_LINK + ["-o", target], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                              text=True)
        if proc.returncode != 0:
            raise BuildError("linking the engine library failed:\n%s" % proc.stdout)
    finally:
        if own:
            shutil.rmtree(obj_dir, ignore_errors=True)
    return target


def ensure_host_built(verbose=False):
    return find_host_library() or build_host(force=True, verbose=verbose)


def _run_with_heartbeat(cmd, what, log):
    done = threading.Event()
    start = time.time()

    def beat():
        while not done.wait(15.0):
            log("[tq_kv_amd build] still compiling %s (%.0f s)" % (what, time.time() - start))
    th = threading.Thread(target=beat, daemon=True)
    th.start()
    try:
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    finally:
        done.set()
    if proc.returncode != 0:
        raise BuildError("hipcc failed on %s:\n%s" % (what, proc.stdout))
    return proc.stdout


def build(force=True, verbose=True):
    """Compile all sources for gfx950 and link the shared library.  Returns its path."""
    def log(msg):
        if verbose:
            print(msg, file=sys.stderr, flush=True)

    existing = find_library()
    if existing and not force:
        return existing
    build_host(force=force, verbose=verbose)
    hipcc = _hipcc()
    out_dir = HERE if _writable(HERE) else _fallback_dir()
    if not _writable(out_dir):
        raise BuildError("cannot write the kernel library to %s or %s" % (HERE, out_dir))
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    log("[tq_kv_amd build] compiling %d sources for %s into %s" % (len(SOURCES), ARCH, out_dir))

    errors = []
    objects = []
    threads = []

    def compile_one(src, obj):
        try:
            _run_with_heartbeat([hipcc] + HIPCC_FLAGS + ["-I", HERE, "-c", os.path.join(HERE, src), "-o", obj], src, log)
            log("[tq_kv_amd build] compiled %s" % src)
        except BuildError as e:
            errors.append(e)

    for src in SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        objects.append(obj)
        th = threading.Thread(target=compile_one, args=(src, obj))
        th.start()
        threads.append(th)
    for th in threads:
        th.join()
    if errors:
        raise errors[0]

    target = os.path.join(out_dir, library_name())
    tmp = target + ".tmp%d" % os.getpid()
    _run_with_heartbeat([hipcc, "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", tmp] + objects, "link", log)
    os.replace(tmp, target)
    # older libraries of other source versions are of no use any more
    for name in os.listdir(out_dir):
        if name.startswith("libtqkernels_") and name.endswith(".so") and name != os.path.basename(target):
            try:
                os.remove(os.path.join(out_dir, name))
            except OSError:
                pass
    log("[tq_kv_amd build] built %s" % target)
    return target


def ensure_built(verbose=True):
    return find_library() or build(force=True, verbose=verbose)


if __name__ == "__main__":
    print(build(force=True))

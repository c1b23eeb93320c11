"""A C program with no Python in its process: compiled here against csrc/tq_engine.h, it loads a
model folder written by `tq random-weights`, runs one step by hand and generates greedily; what it
prints is compared with the plain implementation."""
import os
import shutil
import subprocess
import sys

import pytest

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_c_program_generates_the_plain_implementations_tokens(name, tmp_path):
    from tq_kv_amd import native
    cc = shutil.which("cc") or shutil.which("gcc")
    if cc is None:
        pytest.skip("no C compiler")
    cfg, seed = helpers.CONFIGS[name]
    shape = tmp_path / "shape.json"
    import json
    shape.write_text(json.dumps(cfg))
    folder = str(tmp_path / "model")
    made = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tq"), "random-weights", str(shape), folder, "--seed", str(seed),
                           "--store", "float32"], capture_output=True, text=True)
    assert made.returncode == 0, made.stderr
    lib = native.library_path()
    exe = str(tmp_path / "generate")
    built = subprocess.run([cc, "-std=c99", "-Wall", "-Werror", os.path.join(ROOT, "examples", "generate.c"), "-I", os.path.join(ROOT, "tq_kv_amd", "csrc"),
                            lib, "-Wl,-rpath," + os.path.dirname(lib), "-o", exe], capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 60 + n) for n in (5, 11, 17, 70)]
    env = {k: v for k, v in os.environ.items() if not k.startswith("PYTHON")}
    run = subprocess.run([exe, folder, "float32", "8"] + [",".join(str(t) for t in p) for p in prompts], capture_output=True, text=True, env=env,
                         timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    linked = subprocess.run(["ldd", exe], capture_output=True, text=True).stdout
    assert "libpython" not in linked and "libtorch" not in linked
    pcfg, w = helpers.read_folder(folder)
    lines = run.stdout.strip().splitlines()
    want = [plain.generate_greedy(w, pcfg, p, 8) for p in prompts]
    assert lines[0] == "step: %d" % want[0][0]
    for i, tokens in enumerate(want):
        assert lines[1 + i] == "%d: %s" % (i, " ".join(str(t) for t in tokens))
    # a folder that is not there: a message and a status, no crash
    bad = subprocess.run([exe, str(tmp_path / "nothing"), "float32", "2", "1,2"], capture_output=True, text=True, env=env, timeout=120)
    assert bad.returncode == 1 and "Cannot read config.json" in bad.stderr

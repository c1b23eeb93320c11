"""The command line: the reference's option names and defaults where it has them
(src/main.rs:46-139), and a run through `tq generate` on the GPU."""
import json
import os
import subprocess
import sys

import pytest

from tq_kv_amd.cli import build_parser, format_chatml

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")


def test_generate_options_are_the_references():
    a = build_parser().parse_args(["generate", "tiny:a", "--prompt-ids", "1,2,3"])
    # -n/--max-tokens 512, -t/--temperature 0.7, --top-p 0.9, --top-k 40, --repeat-penalty 1.1 (src/main.rs:56-69)
    assert (a.max_tokens, a.temperature, a.top_p, a.top_k, a.repeat_penalty) == (512, 0.7, 0.9, 40, 1.1)
    a = build_parser().parse_args(["generate", "m", "-n", "7", "-t", "0", "--top-k", "0", "--top-p", "1", "--repeat-penalty", "1",
                                   "--prompt-ids", "5 6", "--prompt-ids", "7"])
    assert (a.max_tokens, a.temperature, a.top_k, a.prompt_ids) == (7, 0.0, 0, ["5 6", "7"])
    b = build_parser().parse_args(["bench", "qwen2.5:7b", "--json"])
    assert b.tokens == 100 and b.json                       # -n/--tokens 100, --json (src/main.rs:124-133)
    assert build_parser().parse_args(["--fp32", "generate", "m"]).fp32


def test_chat_template_is_chatml():
    # src/chat.rs:98-104
    assert format_chatml("S", "U") == "<|im_start|>system\nS<|im_end|>\n<|im_start|>user\nU<|im_end|>\n<|im_start|>assistant\n"


def test_list_and_no_command():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tq"), "list"], capture_output=True, text=True)
    assert out.returncode == 0 and "qwen2.5:7b" in out.stdout and "tiny:b" in out.stdout
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tq")], capture_output=True, text=True)
    assert out.returncode == 0 and "tq generate" in out.stderr


@pytest.mark.gpu
def test_tq_generate_runs_and_is_greedy_reproducible():
    cmd = [sys.executable, os.path.join(ROOT, "bin", "tq"), "--fp32", "generate", "tiny:b", "--prompt-ids", "1,2,3",
           "--prompt-ids", "9 8 7 6 5", "-n", "6", "-t", "0", "--repeat-penalty", "1.0", "--json"]
    a = subprocess.run(cmd, capture_output=True, text=True)
    assert a.returncode == 0, a.stderr
    res = json.loads(a.stdout.strip().splitlines()[-1])
    assert [len(o) for o in res["outputs"]] == [6, 6] and res["tokens"] == 12
    b = subprocess.run(cmd, capture_output=True, text=True)
    assert json.loads(b.stdout.strip().splitlines()[-1])["outputs"] == res["outputs"]
    c = subprocess.run(cmd[:-1] + ["--eos", str(res["outputs"][0][2])], capture_output=True, text=True)
    assert c.returncode == 0 and c.stdout.splitlines()[0].split(": ")[1].split() == [str(t) for t in res["outputs"][0][:2]]

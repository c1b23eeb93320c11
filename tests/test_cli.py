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


@pytest.mark.gpu
def test_tq_generate_with_packed_weights_only_emits_the_same_tokens():
    # steps of up to 128 rows run the same kernels with and without the weights' rows
    cmd = [sys.executable, os.path.join(ROOT, "bin", "tq"), "generate", "tiny:b", "--prompt-ids", "1,2,3",
           "--prompt-ids", "9 8 7 6 5 4 3 2", "-n", "8", "-t", "0", "--repeat-penalty", "1.0", "--json"]
    a = subprocess.run(cmd, capture_output=True, text=True)
    b = subprocess.run(cmd + ["--packed-weights-only"], capture_output=True, text=True)
    assert a.returncode == 0 and b.returncode == 0, a.stderr + b.stderr
    outs = [json.loads(r.stdout.strip().splitlines()[-1])["outputs"] for r in (a, b)]
    assert outs[0] == outs[1] and [len(o) for o in outs[0]] == [8, 8]


@pytest.mark.gpu
def test_tq_generate_on_a_folder_written_by_tq_random_weights_emits_the_plain_tokens(tmp_path):
    """`tq random-weights` writes a folder, `tq generate <folder>` loads it and generates; the
    tokens it prints are the plain implementation's greedy tokens for the same folder, and a stop
    id that only generation_config.json names ends a request without being printed."""
    import helpers
    import plain_qwen2 as plain
    tq = [sys.executable, os.path.join(ROOT, "bin", "tq")]
    cfg_path = tmp_path / "shape.json"
    cfg_path.write_text(json.dumps(helpers.TINY_B))
    folder = str(tmp_path / "model")
    w = subprocess.run(tq + ["random-weights", str(cfg_path), folder, "--seed", "5", "--store", "float32"],
                       capture_output=True, text=True)
    assert w.returncode == 0 and os.path.exists(os.path.join(folder, "model.safetensors")), w.stderr
    cfg, weights = helpers.read_folder(folder)
    prompts = [[1, 2, 3], [9, 8, 7, 6, 5, 300, 12]]
    want = [plain.generate_greedy(weights, cfg, p, 7) for p in prompts]
    cmd = tq + ["--fp32", "generate", folder, "--prompt-ids", "1,2,3", "--prompt-ids", "9 8 7 6 5 300 12", "-n", "7", "-t", "0",
                "--repeat-penalty", "1.0", "--json"]
    a = subprocess.run(cmd, capture_output=True, text=True)
    assert a.returncode == 0, a.stderr
    assert json.loads(a.stdout.strip().splitlines()[-1])["outputs"] == want
    # the same through the text output, one line per request
    b = subprocess.run(cmd[:-1], capture_output=True, text=True)
    assert [line.split(": ")[1].split() for line in b.stdout.strip().splitlines()] == [[str(t) for t in o] for o in want]
    # a stop token named by generation_config.json alone
    stop = want[1][3]
    with open(os.path.join(folder, "generation_config.json"), "w") as f:
        json.dump({"eos_token_id": [stop]}, f)
    c = subprocess.run(cmd, capture_output=True, text=True)
    assert c.returncode == 0, c.stderr
    got = json.loads(c.stdout.strip().splitlines()[-1])["outputs"]
    assert got == [plain.generate_greedy(weights, cfg, p, 7, eos_ids=(stop,)) for p in prompts] and len(got[1]) <= 3


@pytest.mark.gpu
def test_tq_generate_takes_text_where_the_folder_holds_a_tokenizer(tmp_path):
    """`tq generate --prompt TEXT`: the folder's tokenizer.json turns the text into ids (no special tokens added, as
    src/engine.rs:342-345) and the answer back into text; with -s the text is wrapped in the reference's chat template
    first.  The ids that reach the model are checked through what it generates: the plain implementation's tokens."""
    import helpers
    import plain_qwen2 as plain
    from tokenizers import Tokenizer, models, pre_tokenizers
    words = ["<unk>", "<|im_start|>", "<|im_end|>"] + ["w%d" % i for i in range(40)] + ["system", "user", "assistant", "hello", "there"]
    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tq = [sys.executable, os.path.join(ROOT, "bin", "tq")]
    cfg_path = tmp_path / "shape.json"
    cfg_path.write_text(json.dumps(helpers.TINY_A))
    folder = str(tmp_path / "model")
    assert subprocess.run(tq + ["random-weights", str(cfg_path), folder, "--seed", "3", "--store", "float32"], capture_output=True).returncode == 0
    tok.save(os.path.join(folder, "tokenizer.json"))
    cfg, weights = helpers.read_folder(folder)
    text = "hello there w3 w17 w5"
    ids = tok.encode(text, add_special_tokens=False).ids
    assert ids == [words.index(w) for w in text.split()]
    want = plain.generate_greedy(weights, cfg, ids, 6, eos_ids=(2,))            # <|im_end|> is one of the reference's stop strings
    run = subprocess.run(tq + ["--fp32", "generate", folder, "--prompt", text, "-n", "6", "-t", "0", "--repeat-penalty", "1.0"],
                         capture_output=True, text=True)
    assert run.returncode == 0, run.stderr
    assert run.stdout.strip() == tok.decode(want, skip_special_tokens=True) and "Prompt tokens: 5" in run.stderr
    as_json = subprocess.run(tq + ["--fp32", "generate", folder, "--prompt", text, "-n", "6", "-t", "0", "--repeat-penalty", "1.0", "--json"],
                             capture_output=True, text=True)
    assert json.loads(as_json.stdout.strip().splitlines()[-1])["outputs"] == [want]
    # without a tokenizer.json the text cannot be taken
    os.remove(os.path.join(folder, "tokenizer.json"))
    bad = subprocess.run(tq + ["generate", folder, "--prompt", text], capture_output=True, text=True)
    assert bad.returncode != 0 and "tokenizer.json" in bad.stderr

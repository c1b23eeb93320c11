"""bin/trace_run as a user runs it: a child process fed steps on standard input.  The
same requests whole, with the last 32 tokens one by one, and in batches of unequal
lengths one after another, in float32 and bfloat16, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import gpu_common as G

pytestmark = pytest.mark.gpu
ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")


class Replay:
    def __init__(self, folder, dtype, out, max_tokens):
        self.out = out
        self.proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                                      "--out", out, "--max-tokens", str(max_tokens)],
                                     stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.n = 0

    def step(self, entries, end=()):
        rec = {"step": self.n, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w in entries], "end": list(end)}
        self.proc.stdin.write(json.dumps(rec) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline().strip()
        assert line == "done %d" % self.n, "trace_run said %r" % line
        path = os.path.join(self.out, "%d.f32" % self.n)
        self.n += 1
        if not any(w for _, _, w in entries):
            assert not os.path.exists(path)
            return None
        return torch.from_numpy(np.fromfile(path, dtype="<f4"))

    def finish(self):
        self.proc.stdin.close()
        assert self.proc.wait(timeout=60) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_trace_run_three_ways(name, dtype, tmp_path):
    vocab = G.plain_model(name, True)[0]["vocab_size"]
    reqs = dict(zip("abcde", G.prompts(name, [40, 7, 64, 33, 90 if name == "B" else 100], seed=900)))
    ref = {k: G.plain_logits(name, v, True) for k, v in reqs.items()}
    r = Replay(G.folder(name, True), dtype, str(tmp_path / "out"), max_tokens=64 * 6)
    # 1. each request alone and whole
    for k, toks in reqs.items():
        got = r.step([(k + "1", toks, list(range(len(toks))))], end=[k + "1"])
        G.close(got.view(-1, vocab), ref[k], dtype, "whole " + k)
    # 2. the last 32 tokens one by one (the logits of the prompt part are not asked for)
    for k, toks in reqs.items():
        cut = max(1, len(toks) - 32)
        assert r.step([(k + "2", toks[:cut], [])]) is None
        rows = [r.step([(k + "2", [toks[t]], [0])], end=[k + "2"] if t == len(toks) - 1 else []) for t in range(cut, len(toks))]
        G.close(torch.stack(rows), ref[k][cut:], dtype, "one by one " + k)
    # 3. batches of unequal lengths, one after another; the cache (6 pages) only holds them
    #    because ended requests give their pages back
    for batch in (["a", "b", "c"], ["d", "e", "b"], ["c", "a", "d"]):
        tails = {k: min(len(reqs[k]) - 1, 3 + 4 * i) for i, k in enumerate(batch)}
        heads = {k: len(reqs[k]) - tails[k] for k in batch}
        got = r.step([(k + "3", reqs[k][:heads[k]], [heads[k] - 1]) for k in batch]).view(-1, vocab)
        for i, k in enumerate(batch):
            G.close(got[i], ref[k][heads[k] - 1], dtype, "batch prompt " + k)
        pos = dict(heads)
        live = list(batch)
        while live:
            ending = [k + "3" for k in live if pos[k] + 1 == len(reqs[k])]
            got = r.step([(k + "3", [reqs[k][pos[k]]], [0]) for k in live], end=ending).view(-1, vocab)
            for i, k in enumerate(live):
                G.close(got[i], ref[k][pos[k]], dtype, "batch decode %s at %d" % (k, pos[k]))
                pos[k] += 1
            live = [k for k in live if pos[k] < len(reqs[k])]
    r.finish()

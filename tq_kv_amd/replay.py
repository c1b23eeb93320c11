"""Trace replay: feed given token ids through a model step by step and write logits.

The reference's nearest program is its perplexity loop, which feeds given tokens one
at a time and reads the logits of every step (src/engine.rs:467-528).  This one reads
steps from standard input, one JSON object a line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

runs each through the engine's step function (the same model, cache and kernels that
generation uses; nothing here computes), writes the wanted logits of step s as
little-endian float32 [wanted, vocab] to <out>/<s>.f32, and prints "done <s>".
It samples nothing.
"""
import argparse
import json
import os
import sys

import numpy as np


def main(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"],
                    help="bfloat16: the kernels and precisions of serving; float32: everything in true 32-bit")
    ap.add_argument("--out", required=True, help="folder the logits are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each request counted up to a multiple of 64")
    args = ap.parse_args(argv)

    from . import kernels, native
    kernels.library()                       # builds the kernels and the engine on a first call, with progress lines
    native.library()
    from .cache.store import PAGE
    from .engine import Engine, Model

    os.makedirs(args.out, exist_ok=True)
    model = Model.from_dir(args.model, dtype=args.dtype, device="cuda")
    max_tokens = max(PAGE, (args.max_tokens + PAGE - 1) // PAGE * PAGE)
    engine = Engine(model, max_tokens=max_tokens, max_slots=max_tokens // PAGE)
    slots = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        items = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if rid not in slots:
                slots[rid] = engine.open()
            items.append((slots[rid], e["tokens"], e.get("want", [])))
        if items:
            logits = engine.step(items)
            if logits.shape[0] > 0:
                arr = logits.detach().cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, "%s.f32.tmp" % step)
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, "%s.f32" % step))
            else:
                import torch
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            if rid in slots:
                engine.close(slots.pop(rid))
        sys.stdout.write("done %s\n" % step)
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())

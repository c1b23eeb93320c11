"""The `tq` command, in the manner of the reference's (src/main.rs:23-214): subcommands,
option names and defaults as there where they exist.

    tq generate <model> ...   generate tokens for one or more prompts
    tq bench <model> ...      tokens per second of one request (src/main.rs:926-1151)
    tq replay ...             trace replay (see tq_kv_amd/replay.py)
    tq list                   the shapes that can be run with random weights
    tq random-weights ...     write a model folder with seeded random weights

<model> is a folder with config.json and *.safetensors, or the name of a shape of the
catalog ("qwen2.5:7b", "tiny:a"), which is run with seeded random weights.  The
reference's `chat` takes text and prints text; here prompts are token ids, and text
only if the model folder holds a tokenizer.json.
"""
import argparse
import json
import os
import sys
import time

DEFAULT_SYSTEM_PROMPT = "You are a helpful assistant. Answer the user's questions clearly and concisely."


def format_chatml(system_prompt, user_message):
    """The reference's template for Qwen models (src/chat.rs:98-104)."""
    return ("<|im_start|>system\n%s<|im_end|>\n<|im_start|>user\n%s<|im_end|>\n<|im_start|>assistant\n"
            % (system_prompt, user_message))


def _add_sampling(p, max_tokens):
    p.add_argument("-n", "--max-tokens", type=int, default=max_tokens, help="Max tokens per response")
    p.add_argument("-t", "--temperature", type=float, default=0.7, help="Temperature (0.0 - 2.0); 0 is greedy")
    p.add_argument("--top-p", type=float, default=0.9, help="Top-p sampling")
    p.add_argument("--top-k", type=int, default=40, help="Top-k sampling (0: off)")
    p.add_argument("--repeat-penalty", type=float, default=1.1, help="Repeat penalty (1.0: off)")
    p.add_argument("--seed", type=int, default=0, help="Seed of the sampling streams")


def _add_model(p):
    p.add_argument("model", help="Model folder, or name of a shape to run with random weights (see `tq list`)")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--weights-seed", type=int, default=0, help="Seed of the random weights of a shape")
    p.add_argument("--allow-extra-tensors", action="store_true",
                   help="Tensors in the folder that the model does not use are a warning, not an error")
    p.add_argument("--packed-weights-only", action="store_true",
                   help="Keep only the copy of the bfloat16 weights that the decoding kernels read (half the weight memory; "
                        "a prompt's products get the rows back from it for their own length: a seventh more time for 2048 tokens)")
    p.add_argument("--max-cache-tokens", type=int, default=0,
                   help="Positions the cache holds for all live requests together (0: what the prompts need)")


def build_parser():
    ap = argparse.ArgumentParser(prog="tq", description="tq for MI355X -- local LLM inference (Qwen2 dense decoder)")
    ap.add_argument("--fp32", action="store_true", help="Run everything in true 32-bit (same as --dtype float32)")
    ap.add_argument("--trace", action="store_true",
                    help="Named ranges (model, attn, attn-mlp, rms-norm, output) around the parts of every step, for a profiler's marker trace")
    sub = ap.add_subparsers(dest="command")
    g = sub.add_parser("generate", help="Generate tokens for prompts")
    _add_model(g)
    g.add_argument("--prompt-ids", action="append", default=[], help="A prompt as token ids, e.g. 1,2,3 (may be repeated)")
    g.add_argument("--prompt-file", help="A file with one prompt per line, as token ids")
    g.add_argument("--prompt", action="append", default=[], help="A prompt as text (needs tokenizer.json in the model folder)")
    g.add_argument("-s", "--system", default=None, help="System prompt: wrap text prompts in the chat template")
    g.add_argument("--eos", default=None, help="Stop token ids, e.g. 151645,151643 (default: eos_token_id of config.json and generation_config.json, stop strings of tokenizer.json)")
    g.add_argument("--json", action="store_true", help="Output results as JSON")
    _add_sampling(g, 512)
    b = sub.add_parser("bench", help="Run a generation benchmark")
    _add_model(b)
    b.add_argument("-n", "--tokens", type=int, default=100, help="Number of tokens to generate per run")
    b.add_argument("--prompt-len", type=int, default=32, help="Length of the random prompt")
    b.add_argument("--json", action="store_true", help="Output results as JSON")
    b.add_argument("--tune", action="store_true",
                   help="Let the matrix library try its kernels for the prompt's size first (takes some milliseconds a shape)")
    r = sub.add_parser("replay", help="Replay a trace of steps from standard input and write logits")
    r.add_argument("--model", required=True)
    r.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    r.add_argument("--out", required=True)
    r.add_argument("--max-tokens", type=int, required=True)
    rw = sub.add_parser("random-weights", help="Write a model folder (config.json, model.safetensors) with random weights")
    rw.add_argument("shape", help="Name of a shape (see `tq list`) or path of a config.json")
    rw.add_argument("out", help="Folder to write")
    rw.add_argument("--seed", type=int, default=0)
    rw.add_argument("--store", choices=["bfloat16", "float32"], default="bfloat16", help="dtype the tensors are stored in")
    ls = sub.add_parser("list", help="List the shapes of the catalog")
    ls.add_argument("-a", "--available", action="store_true", help="(accepted for likeness; all shapes are always listed)")
    return ap


def load_model(name, dtype, weights_seed, strict=True, packed_only=False):
    from .config import catalog
    from .engine import Model
    if packed_only:
        from .policy import POLICY
        POLICY["keep_rows"] = False
    if os.path.isdir(name):
        return Model.from_dir(name, dtype=dtype, strict=strict)
    if catalog.find(name) is None:
        raise SystemExit("Model '%s' not found: no such folder and no such shape. Available shapes: %s"
                         % (name, ", ".join("%s:%s" % e for e in catalog.entries())))
    return Model.random(name, seed=weights_seed, dtype=dtype)


def _ids(text):
    return [int(t) for t in text.replace(",", " ").split()]


def cmd_generate(args):
    from .cache.store import PAGE
    from .engine import Engine, generate
    from .sampling import GenerationParams
    prompts = [_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [_ids(line) for line in f if line.strip()]
    tokenizer = None
    if args.prompt:
        path = os.path.join(args.model, "tokenizer.json")
        if not os.path.exists(path):
            raise SystemExit("--prompt needs %s; give token ids with --prompt-ids instead" % path)
        from tokenizers import Tokenizer
        tokenizer = Tokenizer.from_file(path)
        for text in args.prompt:
            if args.system is not None:
                text = format_chatml(args.system or DEFAULT_SYSTEM_PROMPT, text)
            prompts.append(tokenizer.encode(text, add_special_tokens=False).ids)       # as src/engine.rs:342-345
    if not prompts:
        raise SystemExit("no prompt: give --prompt-ids, --prompt-file or --prompt")
    model = load_model(args.model, args.dtype, args.weights_seed, strict=not args.allow_extra_tensors,
                       packed_only=args.packed_weights_only)
    params = GenerationParams(max_tokens=args.max_tokens, temperature=args.temperature, top_p=args.top_p,
                              top_k=args.top_k, repeat_penalty=args.repeat_penalty, seed=args.seed)
    eos = _ids(args.eos) if args.eos is not None else list(model.stop_token_ids)
    # room for one batch of the generation loop (at most 64 requests at a time)
    rooms = sorted(((len(p) + args.max_tokens + PAGE - 1) // PAGE * PAGE for p in prompts), reverse=True)
    engine = Engine(model, max_tokens=args.max_cache_tokens or sum(rooms[:64]))
    print("Prompt tokens: %s" % ", ".join(str(len(p)) for p in prompts), file=sys.stderr)
    t0 = time.perf_counter()
    out = generate(engine, prompts, params, eos_ids=eos)
    dt = time.perf_counter() - t0
    if args.json:
        print(json.dumps({"outputs": out, "seconds": round(dt, 4), "tokens": sum(len(o) for o in out)}))
    else:
        for i, o in enumerate(out):
            if tokenizer is not None:
                print(tokenizer.decode(o, skip_special_tokens=True))
            else:
                print("%d: %s" % (i, " ".join(str(t) for t in o)))
    print("%d tokens in %.3f s (%.1f tok/s)" % (sum(len(o) for o in out), dt, sum(len(o) for o in out) / max(dt, 1e-9)),
          file=sys.stderr)
    return 0


def cmd_bench(args):
    """One request, greedy, tokens per second over the whole run including the prompt and
    time to the first token, as the reference's bench reports them (src/main.rs:1123-1143)."""
    import torch

    from .cache.store import PAGE
    from .engine import Engine, generate
    from .sampling import GenerationParams
    model = load_model(args.model, args.dtype, args.weights_seed, packed_only=args.packed_weights_only)
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, model.spec.vocab_size, (args.prompt_len,), generator=g).tolist()
    engine = Engine(model, max_tokens=args.max_cache_tokens or (args.prompt_len + args.tokens + 2 * PAGE) // PAGE * PAGE)
    params = GenerationParams(max_tokens=args.tokens, temperature=0.0, repeat_penalty=1.0)
    if args.tune:
        model.tune_library(len(prompt))
    generate(engine, [prompt], GenerationParams(max_tokens=4, temperature=0.0, repeat_penalty=1.0), eos_ids=())      # warm-up
    marks = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = generate(engine, [prompt], params, eos_ids=(), on_tokens=lambda pairs: marks.append(time.perf_counter()))
    torch.cuda.synchronize()
    total = time.perf_counter() - t0
    res = {"model": args.model, "dtype": args.dtype, "prompt_tokens": len(prompt), "tokens": len(out[0]),
           "total_s": round(total, 4), "ttft_s": round(marks[0] - t0, 4) if marks else None,
           "tok_per_s": round(len(out[0]) / total, 2),
           "decode_tok_per_s": round((len(out[0]) - 1) / (marks[-1] - marks[0]), 2) if len(marks) > 1 else None}
    if args.json:
        print(json.dumps(res))
    else:
        print("%(model)s [%(dtype)s]: %(tokens)d tokens in %(total_s).3f s = %(tok_per_s).1f tok/s, TTFT %(ttft_s).3f s, "
              "decode %(decode_tok_per_s)s tok/s" % res)
    return 0


def cmd_random_weights(args):
    import torch

    from .engine import Model
    shape = args.shape
    if os.path.isfile(shape):
        with open(shape) as f:
            shape = json.load(f)
    folder = Model.write_random_folder(args.out, shape, seed=args.seed,
                                       store_dtype=torch.bfloat16 if args.store == "bfloat16" else torch.float32)
    print("wrote %s" % folder)
    return 0


def cmd_list(args):
    from .config import catalog
    for name, tag in catalog.entries():
        raw = catalog.find("%s:%s" % (name, tag))
        print("%-16s layers=%-3d hidden=%-5d heads=%d/%d head_dim=%d inter=%d vocab=%d"
              % ("%s:%s" % (name, tag), raw["num_hidden_layers"], raw["hidden_size"], raw["num_attention_heads"],
                 raw.get("num_key_value_heads", raw["num_attention_heads"]),
                 raw.get("head_dim", raw["hidden_size"] // raw["num_attention_heads"]), raw["intermediate_size"],
                 raw["vocab_size"]))
    return 0


def main(argv=None):
    ap = build_parser()
    args = ap.parse_args(argv)
    if args.command is None:
        print("Use `tq generate <model>` or `tq bench <model>` or `tq --help`", file=sys.stderr)   # src/main.rs:209
        return 0
    if getattr(args, "fp32", False) and hasattr(args, "dtype"):
        args.dtype = "float32"
    if args.trace:
        from . import tracing
        tracing.enable()
    if args.command == "generate":
        return cmd_generate(args)
    if args.command == "bench":
        return cmd_bench(args)
    if args.command == "list":
        return cmd_list(args)
    if args.command == "random-weights":
        return cmd_random_weights(args)
    if args.command == "replay":
        from .replay import main as replay_main
        return replay_main(["--model", args.model, "--dtype", args.dtype, "--out", args.out, "--max-tokens", str(args.max_tokens)])
    return 2


if __name__ == "__main__":
    sys.exit(main())

"""Decode and prefill throughput of the Qwen2.5-7B shape with random bfloat16 weights on
one MI355X: `python bench.py [--gpus 1] [--steps K] [--warmup W]` prints one JSON line.

A step is one decode step of the whole batch through the generation loop (step
function, sampling, host round trip for the stop check).  The reference measures
tokens per second of one chat request including its prompt (src/main.rs:1123-1143);
here decoding is timed alone, the prompt pass is reported beside it, and the reference's
prompt-inclusive figure goes into `end_to_end_tok_per_s`.

Other workloads of the same bench, each one command and one line:
  --workload 1.5b-mixed   Qwen2.5-1.5B shape, 32 prompts of 16..1024 tokens, 128 sampled steps
  --workload 32b          Qwen2.5-32B shape, 16 prompts of 512 tokens, 256 greedy steps
  --prompt-len N          other contexts of the default workload (8192, 16384, ...)
"""
import argparse
import json
import sys
import time

PEAK = {"hbm_gbs": 8000.0, "bf16_flops": 2.5e15}     # MI355X: HBM3E 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s
# shape, batch, prompt length, steps, warm-up steps; mixed: unequal prompts, sampled; no_points: headline only
WORKLOADS = {
    "7b": dict(shape="qwen2.5:7b", batch=8, prompt_len=2048, steps=128, warmup=16),
    "1.5b-mixed": dict(shape="qwen2.5:1.5b", batch=32, prompt_len=1024, steps=128, warmup=16, mixed=True),
    "32b": dict(shape="qwen2.5:32b", batch=16, prompt_len=512, steps=256, warmup=8, no_points=True),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--prompt-len", type=int, default=None)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="7b",
                    help="a preset of shape, batch, prompt length, steps and sampling; the other options override it")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--shape", default=None)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1, 64 and 128 points")
    ap.add_argument("--no-tune", action="store_true", help="do not let the library pick its fastest kernel per product shape")
    ap.add_argument("--mixed", action="store_true",
                    help="another workload instead: --batch prompts of unequal lengths (uniform in 16..--prompt-len), sampled with "
                         "the default parameters (temperature 0.7, top-k 40, top-p 0.9, repeat penalty 1.1); prints its own line")
    args = ap.parse_args()
    preset = WORKLOADS[args.workload]
    for key, value in preset.items():
        if getattr(args, key) in (None, False):
            setattr(args, key, value)
    if args.gpus != 1:
        print("bench.py: this library runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    import torch

    from tq_kv_amd import Engine, GenerationParams, Model, generate
    from tq_kv_amd.config import catalog
    from tq_kv_amd import POLICY

    t_start = time.perf_counter()

    def note(msg):
        print("[bench %.0fs] %s" % (time.perf_counter() - t_start, msg), file=sys.stderr, flush=True)

    raw = dict(catalog.find(args.shape))
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    layers = raw["num_hidden_layers"]
    H, I, V = raw["hidden_size"], raw["intermediate_size"], raw["vocab_size"]
    nh, nkv, d = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"]
    ctx_len = raw["max_position_embeddings"]
    needed = args.prompt_len + args.steps + args.warmup + 2
    if needed > ctx_len:             # other contexts than the shape's own: the position tables grow with them
        ctx_len = raw["max_position_embeddings"] = (needed + 1023) // 1024 * 1024
    note("making random weights for %s (%d layers)" % (args.shape, layers))
    model = Model.random(raw, seed=0, dtype="bfloat16", device="cuda:0")
    total_new = args.steps + args.warmup + 2
    per_seq = (args.prompt_len + total_new + 63) // 64 * 64           # positions a sequence holds at the end
    # the other batch sizes, as far as their caches fit beside the weights (long contexts: not all do)
    free_bytes = torch.cuda.mem_get_info(0)[0]
    point_batches = [] if args.no_points else [b for b in (1, 64, 128)
                                               if b * per_seq * layers * 2 * nkv * d * 2 < 0.8 * free_bytes]
    max_batch = max([args.batch] + point_batches)
    engine = Engine(model, max_tokens=max_batch * per_seq)
    gen = torch.Generator().manual_seed(0)

    def prompts(n):
        return torch.randint(0, V, (n, args.prompt_len), generator=gen).tolist()

    if args.mixed:
        return mixed_workload(args, model, engine, raw, note)

    # -- prefill of one prompt --------------------------------------------------------------
    if not args.no_tune:
        # products of more rows than the own kernels take are the library's: let it try its kernels once for the
        # shapes of the measured prompt pass
        note("library tuning for %d rows" % args.prompt_len)
        model.tune_library(args.prompt_len)
    p = prompts(1)[0]
    times = []
    note("prefill of %d tokens" % args.prompt_len)
    for i in range(8):
        slot = engine.open()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([(slot, p, [len(p) - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.close(slot)
    prefill_s = min(times[2:])

    T = args.prompt_len
    linear_params = layers * (H * (nh + 2 * nkv) * d + nh * d * H + 3 * H * I)
    prefill_flops = 2.0 * T * linear_params + layers * 4.0 * nh * d * (T * (T + 1) / 2) + 2.0 * H * V
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops / prefill_s / PEAK["bf16_flops"], 4)}

    # -- decoding ---------------------------------------------------------------------------
    def decode(batch, steps, warmup):
        """Tokens per second over `steps` decode steps of `batch` sequences after their prompts."""
        marks, calls = {}, [0]

        def on_tokens(pairs):
            # call i comes when the tokens of draw i are known; draw i+1 needs decode step i+1.
            # The loop keeps one step under way while it reads a draw, so the device is waited
            # for at the two ends of the timed steps only, and each wait ends just after a step.
            if calls[0] in (warmup, warmup + steps):
                torch.cuda.synchronize()
                marks[calls[0]] = time.perf_counter()
            calls[0] += 1
        params = GenerationParams(max_tokens=warmup + steps + 2, temperature=0.0, repeat_penalty=1.0)
        ps = prompts(batch)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = generate(engine, ps, params, eos_ids=(), on_tokens=on_tokens, max_batch=batch)
        torch.cuda.synchronize()
        whole = time.perf_counter() - t0
        assert all(len(o) == warmup + steps + 2 for o in out)
        seconds = marks[warmup + steps] - marks[warmup]
        return batch * steps / seconds, seconds / steps, sum(len(o) for o in out) / whole

    weight_bytes = 2.0 * (linear_params + H * V)                      # every weight the step uses, once

    def hbm(batch, steps, warmup, sec_per_step):
        """GB/s of a decode step: the weights once and the cache of the live requests, over its time."""
        mean_ctx = args.prompt_len + warmup + steps / 2.0
        kv_bytes = batch * mean_ctx * layers * 2 * nkv * d * 2.0
        return (weight_bytes + kv_bytes) / sec_per_step / 1e9

    note("decode at batch %d" % args.batch)
    tps, sec_per_step, end_to_end = decode(args.batch, args.steps, args.warmup)
    points = {}
    if not args.no_points:
        for batch, steps, warmup in ((1, min(args.steps, 64), 8), (64, min(args.steps, 32), 4), (128, min(args.steps, 16), 4)):
            if batch not in point_batches:
                continue
            note("decode at batch %d" % batch)
            b_tps, b_sec, _ = decode(batch, steps, warmup)
            gbs = hbm(batch, steps, warmup, b_sec)
            name = "decode_b%d" % batch
            points.update({name: round(b_tps, 1), name + "_ms": round(b_sec * 1e3, 4), name + "_gbs": round(gbs, 1),
                           name + "_frac": round(gbs / PEAK["hbm_gbs"], 4)})
    note("done")
    achieved = hbm(args.batch, args.steps, args.warmup, sec_per_step)
    line = {
        "metric": "decode tok/s @ batch %d, %s shape" % (args.batch, args.shape), "value": round(tps, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": args.shape, "global_batch": args.batch, "seq_len": ctx_len, "parallelism": "single-gpu",
                   "layers": layers, "layers_of_shape": full_layers, "hidden": H, "heads": nh, "kv_heads": nkv,
                   "head_dim": d, "intermediate": I, "vocab": V, "prompt_len": args.prompt_len,
                   "new_tokens": args.warmup + args.steps + 2, "weights": "random N(0,0.02)", "sampling": "greedy",
                   "library_tuning": not args.no_tune, "packed_weight_copy": bool(POLICY["packed"])},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK["hbm_gbs"], "unit": "GB/s",
                     "frac": round(achieved / PEAK["hbm_gbs"], 4)},
        "points": points,
        # the reference's figure: generated tokens over the whole run, prompt pass included (src/main.rs:1139-1143)
        "end_to_end_tok_per_s": round(end_to_end, 1),
    }
    print(json.dumps(line))
    return 0


def mixed_workload(args, model, engine, raw, note):
    """Prompts of unequal lengths in one batch, sampled: tokens per second of the decoding steps."""
    import torch

    from tq_kv_amd import GenerationParams, generate
    gen = torch.Generator().manual_seed(1)
    lens = torch.randint(16, args.prompt_len + 1, (args.batch,), generator=gen).tolist()
    prompts = [torch.randint(0, raw["vocab_size"], (n,), generator=gen).tolist() for n in lens]
    marks, calls = {}, [0]

    def on_tokens(pairs):
        if calls[0] in (args.warmup, args.warmup + args.steps):
            torch.cuda.synchronize()
            marks[calls[0]] = time.perf_counter()
        calls[0] += 1
    note("%d prompts of %d..%d tokens, %d sampled steps" % (args.batch, min(lens), max(lens), args.steps))
    params = GenerationParams(max_tokens=args.warmup + args.steps + 2)
    # untimed: one prompt of the longest length, so that the library's first call is not in the clock
    generate(engine, [prompts[lens.index(max(lens))]], GenerationParams(max_tokens=2), max_batch=1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = generate(engine, prompts, params, on_tokens=on_tokens, max_batch=args.batch)
    torch.cuda.synchronize()
    total = time.perf_counter() - t0
    seconds = marks[args.warmup + args.steps] - marks[args.warmup]
    print(json.dumps({"metric": "decode tok/s, %d prompts of unequal lengths, %s shape, sampled" % (args.batch, args.shape),
                      "value": round(args.batch * args.steps / seconds, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
                      "warmup": args.warmup, "ms_per_step": round(seconds / args.steps * 1e3, 4), "dtype": "bf16",
                      "data": "synthetic", "prompt_tokens": sum(lens), "generated_tokens": sum(len(o) for o in out),
                      "end_to_end_tok_per_s": round(sum(len(o) for o in out) / total, 1)}))
    return 0


if __name__ == "__main__":
    sys.exit(main())

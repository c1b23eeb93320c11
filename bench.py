"""Decode and prefill throughput with random bfloat16 weights on one MI355X:
`python bench.py [--gpus 1] [--steps K] [--warmup W]` prints one JSON line.

The headline is the Qwen2.5-7B shape: decoding at batch 8 after 2048-token prompts (`value`, tokens a
second; a step is one decode step of the whole batch through the generation loop: step function,
sampling, host round trip for the stop check), the prompt pass of 2048 tokens (`prefill`), and the decode
step's memory traffic against the HBM peak (`roofline`).  `points` holds decoding at batch 1, 64 and 128,
the same shape at 8192 tokens of context, and the two other workloads of the baseline: the Qwen2.5-1.5B
shape with 32 prompts of unequal lengths sampled at temperature 0.7 (`w15b_*`), and the Qwen2.5-32B shape
with 16 prompts of 512 tokens decoded greedily (`w32b_*`).  `probe` says what this GPU gives a kernel that
only reads memory and one that only feeds the matrix cores; every fraction is given against the published
peak and (`*_of_probe`) against the probe.

The reference measures tokens per second of one chat request including its prompt
(src/main.rs:1123-1143); here decoding is timed alone, the prompt pass is reported beside it, and the
reference's prompt-inclusive figure goes into `end_to_end_tok_per_s`.
"""
import argparse
import gc
import json
import statistics
import sys
import time

PEAK = {"hbm_gbs": 8000.0, "bf16_flops": 2.5e15}     # MI355X: HBM3E 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128, help="timed decode steps of the headline")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--shape", default="qwen2.5:7b")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--no-points", action="store_true", help="the headline alone: no other batch sizes, contexts or workloads")
    ap.add_argument("--no-workloads", action="store_true", help="skip the 1.5B and 32B workloads")
    ap.add_argument("--no-long", action="store_true", help="skip the points at 8192 tokens of context")
    ap.add_argument("--no-tune", action="store_true", help="do not let the matrix library try its kernels for the prompt's size")
    ap.add_argument("--no-probe", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    import torch

    from tq_kv_amd import POLICY, Engine, GenerationParams, Model, generate
    from tq_kv_amd import kernels as K
    from tq_kv_amd.config import catalog

    t_start = time.perf_counter()

    def note(msg):
        print("[bench %.0fs] %s" % (time.perf_counter() - t_start, msg), file=sys.stderr, flush=True)

    # -- what this GPU gives ----------------------------------------------------------------------
    probe = {}
    if not args.no_probe:
        note("probes: a streaming read of 4 GB, a loop of matrix-core products")
        buf = torch.empty(1 << 30, dtype=torch.float32, device="cuda:0")          # 4 GB: far beyond every cache
        buf.fill_(1.0)
        probe["hbm_read_gbs"] = round(K.probe_read(buf), 1)
        del buf
        torch.cuda.empty_cache()
        probe["mfma_bf16_pflops"] = round(K.probe_mfma(), 4)

    def of_probe(value, key):
        return round(value / probe[key], 4) if probe.get(key) else None

    def sizes(raw):
        return dict(L=raw["num_hidden_layers"], H=raw["hidden_size"], I=raw["intermediate_size"], V=raw["vocab_size"],
                    nh=raw["num_attention_heads"], nkv=raw["num_key_value_heads"], d=raw["head_dim"])

    def linear_params(z):
        return z["L"] * (z["H"] * (z["nh"] + 2 * z["nkv"]) * z["d"] + z["nh"] * z["d"] * z["H"] + 3 * z["H"] * z["I"])

    def weight_bytes(z):
        return 2.0 * (linear_params(z) + z["H"] * z["V"])                 # every weight a decode step uses, once

    def kv_bytes_per_token(z):
        return z["L"] * 2 * z["nkv"] * z["d"] * 2.0

    def prefill_flops(z, lens):
        attn = sum(z["L"] * 4.0 * z["nh"] * z["d"] * (n * (n + 1) / 2) for n in lens)
        return 2.0 * sum(lens) * linear_params(z) + attn + 2.0 * z["H"] * z["V"] * len(lens)

    def timed_prefill(engine, prompts, runs):
        """Seconds of the prompt pass of `prompts` (one step, the last place of each wanted), for each of `runs` runs."""
        times = []
        for _ in range(runs):
            slots = [engine.open() for _ in prompts]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.step([(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            for s in slots:
                engine.close(s)
        return times

    def decode(engine, prompts, steps, warmup, params=None):
        """Tokens per second over `steps` decode steps after the prompts, seconds per step, and generated tokens per
        second of the whole run (prompt pass included)."""
        marks, calls = {}, [0]

        def on_tokens(pairs):
            # call i comes when the tokens of draw i are known; draw i+1 needs decode step i+1.  The loop keeps one
            # step under way while it reads a draw, so the device is waited for at the two ends of the timed steps
            # only, and each wait ends just after a step.
            if calls[0] in (warmup, warmup + steps):
                torch.cuda.synchronize()
                marks[calls[0]] = time.perf_counter()
            calls[0] += 1
        params = params or GenerationParams(max_tokens=warmup + steps + 2, temperature=0.0, repeat_penalty=1.0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = generate(engine, prompts, params, eos_ids=(), on_tokens=on_tokens, max_batch=len(prompts))
        torch.cuda.synchronize()
        whole = time.perf_counter() - t0
        assert all(len(o) == warmup + steps + 2 for o in out)
        seconds = marks[warmup + steps] - marks[warmup]
        return len(prompts) * steps / seconds, seconds / steps, sum(len(o) for o in out) / whole

    def hbm(z, mean_tokens_held, sec_per_step):
        """GB/s of a decode step: the weights once and the cache of the live requests, over its time."""
        return (weight_bytes(z) + mean_tokens_held * kv_bytes_per_token(z)) / sec_per_step / 1e9

    def decode_point(name, z, b_tps, b_sec, mean_tokens_held):
        gbs = hbm(z, mean_tokens_held, b_sec)
        return {name: round(b_tps, 1), name + "_ms": round(b_sec * 1e3, 4), name + "_gbs": round(gbs, 1),
                name + "_frac": round(gbs / PEAK["hbm_gbs"], 4), name + "_frac_of_probe": of_probe(gbs, "hbm_read_gbs")}

    gen = torch.Generator().manual_seed(0)

    def random_prompts(vocab, lens):
        return [torch.randint(0, vocab, (n,), generator=gen).tolist() for n in lens]

    def release():
        gc.collect()
        torch.cuda.empty_cache()

    # -- the headline shape -------------------------------------------------------------------------
    raw = dict(catalog.find(args.shape))
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    z = sizes(raw)
    ctx_len = raw["max_position_embeddings"]
    long_ctx = 0 if (args.no_points or args.no_long) else 8192
    total_new = args.steps + args.warmup + 2
    if args.prompt_len + total_new > ctx_len:            # other contexts than the shape's own: the position tables grow with them
        ctx_len = (args.prompt_len + total_new + 1023) // 1024 * 1024
    raw["max_position_embeddings"] = max(ctx_len, (long_ctx + 64 + 1023) // 1024 * 1024 if long_ctx else 0)
    note("making random weights for %s (%d layers)" % (args.shape, z["L"]))
    model = Model.random(raw, seed=0, dtype="bfloat16", device="cuda:0")
    per_seq = (args.prompt_len + total_new + 63) // 64 * 64           # positions a sequence holds at the end
    free_bytes = torch.cuda.mem_get_info(0)[0]
    # the other batch sizes, as far as their caches fit beside the weights (long contexts: not all do)
    point_batches = [] if args.no_points else [b for b in (1, 64, 128) if b * per_seq * kv_bytes_per_token(z) < 0.8 * free_bytes]
    room = max([args.batch] + point_batches) * per_seq
    if long_ctx:
        room = max(room, 8 * (long_ctx + 128))
    engine = Engine(model, max_tokens=room)

    def prefill_point(T, runs):
        if not args.no_tune:
            # products of more rows than the own kernels take are the library's: let it try its kernels once for the
            # shapes of the measured prompt pass
            note("library tuning for %d rows" % T)
            model.tune_library(T)
        note("prefill of %d tokens" % T)
        times = timed_prefill(engine, random_prompts(z["V"], [T]), runs + 2)[2:]
        best, median = min(times), statistics.median(times)
        flops = prefill_flops(z, [T])
        return {"value": round(T / median, 1), "tokens": T, "ms": round(median * 1e3, 3), "frac": round(flops / median / PEAK["bf16_flops"], 4),
                "stat": "median of %d runs" % len(times), "ms_best": round(best * 1e3, 3), "value_best": round(T / best, 1),
                "frac_of_probe": of_probe(flops / median / 1e15, "mfma_bf16_pflops")}

    prefill = prefill_point(args.prompt_len, 7)

    note("decode at batch %d" % args.batch)
    tps, sec_per_step, end_to_end = decode(engine, random_prompts(z["V"], [args.prompt_len] * args.batch), args.steps, args.warmup)
    achieved = hbm(z, args.batch * (args.prompt_len + args.warmup + args.steps / 2.0), sec_per_step)
    points = {}
    for batch, steps, warmup in ((1, min(args.steps, 64), 8), (64, min(args.steps, 32), 4), (128, min(args.steps, 16), 4)):
        if batch not in point_batches:
            continue
        note("decode at batch %d" % batch)
        b_tps, b_sec, _ = decode(engine, random_prompts(z["V"], [args.prompt_len] * batch), steps, warmup)
        points.update(decode_point("decode_b%d" % batch, z, b_tps, b_sec, batch * (args.prompt_len + warmup + steps / 2.0)))
    if long_ctx:
        p = prefill_point(long_ctx, 3)
        points.update({"prefill_8k": p["value"], "prefill_8k_ms": p["ms"], "prefill_8k_frac": p["frac"], "prefill_8k_frac_of_probe": p["frac_of_probe"]})
        note("decode at batch 8 after prompts of %d tokens" % long_ctx)
        b_tps, b_sec, _ = decode(engine, random_prompts(z["V"], [long_ctx] * 8), 32, 4)
        points.update(decode_point("decode_b8_8k", z, b_tps, b_sec, 8 * (long_ctx + 4 + 16.0)))
    packed = bool(POLICY["packed"])
    engine = model = None
    release()

    # -- the baseline's other workloads ---------------------------------------------------------------
    workloads = {}
    if not (args.no_points or args.no_workloads):
        # Qwen2.5-1.5B shape: 32 prompts of unequal lengths (uniform in 16..1024), 128 decode steps at temperature 0.7
        raw15 = dict(catalog.find("qwen2.5:1.5b"))
        z15 = sizes(raw15)
        note("making random weights for qwen2.5:1.5b")
        model = Model.random(raw15, seed=0, dtype="bfloat16", device="cuda:0")
        lens = torch.randint(16, 1025, (32,), generator=torch.Generator().manual_seed(1)).tolist()
        engine = Engine(model, max_tokens=sum((n + 128 + 16 + 2 + 63) // 64 * 64 for n in lens))
        prompts = random_prompts(z15["V"], lens)

        def sampled(n):
            return GenerationParams(max_tokens=n, temperature=0.7, top_k=0, top_p=1.0, repeat_penalty=1.0, seed=0)
        if not args.no_tune:
            model.tune_library(sum(lens))
        decode(engine, prompts[:2], 2, 1, sampled(5))                  # untimed: the sampler's first calls
        note("1.5B shape: 32 prompts of %d..%d tokens, 128 steps at temperature 0.7" % (min(lens), max(lens)))
        first = statistics.median(timed_prefill(engine, prompts, 4)[1:])
        w_tps, w_sec, w_e2e = decode(engine, prompts, 128, 16, sampled(128 + 16 + 2))
        points.update(decode_point("w15b_decode", z15, w_tps, w_sec, sum(lens) + 32 * (16 + 64.0)))
        points.update({"w15b_prefill": round(sum(lens) / first, 1), "w15b_prefill_ms": round(first * 1e3, 3),
                       "w15b_prefill_frac": round(prefill_flops(z15, lens) / first / PEAK["bf16_flops"], 4), "w15b_end_to_end": round(w_e2e, 1)})
        workloads["w15b"] = {"model": "qwen2.5:1.5b", "layers": z15["L"], "hidden": z15["H"], "heads": z15["nh"], "kv_heads": z15["nkv"],
                             "head_dim": z15["d"], "intermediate": z15["I"], "vocab": z15["V"], "batch": 32,
                             "prompt_lens": "uniform in 16..1024 (seed 1), %d tokens in all" % sum(lens), "steps": 128, "warmup": 16,
                             "sampling": "temperature 0.7 (no top-k, no top-p, no repeat penalty)", "seq_len": raw15["max_position_embeddings"]}
        engine = model = None
        release()

        # Qwen2.5-32B shape: 16 prompts of 512 tokens, 256 greedy decode steps
        raw32 = dict(catalog.find("qwen2.5:32b"))
        z32 = sizes(raw32)
        note("making random weights for qwen2.5:32b (%.0f GB, and their packed copy)" % (weight_bytes(z32) / 1e9))
        model = Model.random(raw32, seed=0, dtype="bfloat16", device="cuda:0")
        engine = Engine(model, max_tokens=16 * ((512 + 256 + 8 + 2 + 63) // 64 * 64))
        prompts = random_prompts(z32["V"], [512] * 16)
        if not args.no_tune:
            model.tune_library(16 * 512)
        note("32B shape: 16 prompts of 512 tokens, 256 greedy steps")
        first = statistics.median(timed_prefill(engine, prompts, 4)[1:])
        w_tps, w_sec, w_e2e = decode(engine, prompts, 256, 8)
        points.update(decode_point("w32b_decode", z32, w_tps, w_sec, 16 * (512 + 8 + 128.0)))
        points.update({"w32b_prefill": round(16 * 512 / first, 1), "w32b_prefill_ms": round(first * 1e3, 3),
                       "w32b_prefill_frac": round(prefill_flops(z32, [512] * 16) / first / PEAK["bf16_flops"], 4), "w32b_end_to_end": round(w_e2e, 1)})
        workloads["w32b"] = {"model": "qwen2.5:32b", "layers": z32["L"], "hidden": z32["H"], "heads": z32["nh"], "kv_heads": z32["nkv"],
                             "head_dim": z32["d"], "intermediate": z32["I"], "vocab": z32["V"], "batch": 16, "prompt_len": 512,
                             "steps": 256, "warmup": 8, "sampling": "greedy", "seq_len": raw32["max_position_embeddings"]}
        engine = model = None
        release()
    note("done")
    line = {
        "metric": "decode tok/s @ batch %d, %s shape" % (args.batch, args.shape), "value": round(tps, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": args.shape, "global_batch": args.batch, "seq_len": ctx_len, "parallelism": "single-gpu",
                   "layers": z["L"], "layers_of_shape": full_layers, "hidden": z["H"], "heads": z["nh"], "kv_heads": z["nkv"],
                   "head_dim": z["d"], "intermediate": z["I"], "vocab": z["V"], "prompt_len": args.prompt_len,
                   "new_tokens": total_new, "weights": "random N(0,0.02)", "sampling": "greedy",
                   "library_tuning": not args.no_tune, "packed_weight_copy": packed, "position_table": raw["max_position_embeddings"]},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK["hbm_gbs"], "unit": "GB/s",
                     "frac": round(achieved / PEAK["hbm_gbs"], 4), "frac_of_probe": of_probe(achieved, "hbm_read_gbs")},
        "probe": probe,
        "points": points,
        "workloads": workloads,
        # the reference's figure: generated tokens over the whole run, prompt pass included (src/main.rs:1139-1143)
        "end_to_end_tok_per_s": round(end_to_end, 1),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

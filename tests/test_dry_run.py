"""The engine's host code without a GPU: a model in host memory steps on the "null device" (buffers are host memory,
kernel launches are skipped), so everything that is not a kernel runs: building the parts from the configuration, the
loader, the step's plan and uploads, the workspace's arenas, the order of the layers, the cache's reservations, the
sampler's bookkeeping and the generation loop with its run-ahead.  The numbers that come out mean nothing (no kernel
ran); what is checked is that every call does what it says with slots, pages, lengths and counts.  The same runs on
the sanitized build of the engine library (tests/test_host_sanitizers.py)."""
import pytest
import torch

import helpers
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import PAGE, CacheFull


@pytest.mark.parametrize("name", sorted(helpers.CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_and_generation_on_the_null_device(name, dtype):
    cfg, seed = helpers.CONFIGS[name]
    model = Model.random(cfg, seed=seed, dtype=dtype, device="cpu")
    assert not model.on_gpu
    engine = Engine(model, max_tokens=4 * PAGE, max_slots=5)
    vocab = cfg["vocab_size"]
    free0 = [g.pool.n_free for g in engine.cache.kv_groups]
    a, b, c = engine.open(), engine.open(), engine.open()
    prompts = {a: helpers.random_tokens(70, vocab, 1), b: helpers.random_tokens(3, vocab, 2), c: helpers.random_tokens(1, vocab, 3)}
    out = engine.step([(s, p, [0, len(p) - 1]) for s, p in prompts.items()])
    assert tuple(out.shape) == (6, vocab) and out.dtype == torch.float32
    assert [engine.length(s) for s in (a, b, c)] == [70, 3, 1]
    for step in range(3):                                   # one token each, the shortest request ends first
        live = [a, b, c][:3 - step]
        out = engine.step([(s, [step + 1], [0]) for s in live])
        assert tuple(out.shape) == (len(live), vocab)
        if len(live) > 1:
            engine.close(live[-1])
    assert engine.length(a) == 73
    # a step that does not fit gives back what it took
    held = [g.pool.n_held for g in engine.cache.kv_groups]
    d, e = engine.open(), engine.open()
    with pytest.raises(CacheFull):
        engine.step([(s, helpers.random_tokens(min(2 * PAGE, cfg["max_position_embeddings"]), vocab, 4), [0]) for s in (d, e)])
    assert [g.pool.n_held for g in engine.cache.kv_groups] == held and engine.length(d) == engine.length(e) == 0
    engine.close(d), engine.close(e), engine.close(a)
    assert [g.pool.n_free for g in engine.cache.kv_groups] == free0
    engine.cache.check()
    # the loop: unequal prompts, more requests than a batch takes, a stop token (token 0 is all a null device draws)
    requests = [helpers.random_tokens(n, vocab, 10 + n) for n in (5, 1, 17, 2, 9, 30, 4)]
    params = GenerationParams(max_tokens=4, temperature=0.0, repeat_penalty=1.0)
    got = generate(engine, requests, params, eos_ids=(), max_batch=3)
    assert got == [[0] * 4] * len(requests)
    assert generate(engine, requests, params, eos_ids=(0,), max_batch=3) == [[]] * len(requests)
    sampled = GenerationParams(max_tokens=3, temperature=0.8, top_k=5, top_p=0.9, repeat_penalty=1.1, seed=7)
    assert [len(o) for o in generate(engine, requests[:4], sampled, eos_ids=())] == [3] * 4
    assert [g.pool.n_free for g in engine.cache.kv_groups] == free0
    engine.cache.check()

"""The engine against the plain implementation on the GPU, in float32 and bfloat16:
whole requests, the last 32 tokens one by one, batches of unequal lengths whose
shorter requests end earlier (batch after batch, slots used again), long decoding,
the first tokens of a sequence, generation through the entry point."""
import pytest
import torch

import gpu_common as G
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
CASES = [("A", False), ("A", True), ("B", False), ("B", True), ("C", False), ("C", True)]
LENS = {"A": [5, 11, 17, 64, 65, 100], "B": [1, 7, 20, 33, 64, 90], "C": [70, 129, 333, 600]}


def all_places(p):
    return list(range(len(p)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", CASES)
def test_each_request_alone_and_whole(name, sharp, dtype):
    eng = G.engine(name, dtype, sharp)
    for p in G.prompts(name, LENS[name]):
        s = eng.open()
        out = eng.step([(s, p, all_places(p))])
        eng.close(s)
        G.close(out, G.plain_logits(name, p, sharp), dtype, "%s len %d" % (name, len(p)))
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", CASES)
def test_last_32_tokens_one_by_one(name, sharp, dtype):
    eng = G.engine(name, dtype, sharp)
    for p in G.prompts(name, LENS[name], seed=200):
        ref = G.plain_logits(name, p, sharp)
        k = max(1, len(p) - 32)
        s = eng.open()
        outs = [eng.step([(s, p[:k], all_places(p[:k]))])]
        for t in range(k, len(p)):
            outs.append(eng.step([(s, [p[t]], [0])]))
            assert eng.length(s) == t + 1
        eng.close(s)
        G.close(torch.cat(outs), ref, dtype, "%s len %d" % (name, len(p)))


def run_batch(eng, reqs, tails):
    """reqs: token lists; tails[i]: how many of request i's last tokens are fed one by one.
    Prompts in one step, then one token each; a request that has no more tokens ends and
    gives its slot back while the others go on.  Returns the logits of every place."""
    slots = [eng.open() for _ in reqs]
    heads = [len(r) - t for r, t in zip(reqs, tails)]
    got = [[] for _ in reqs]
    out = eng.step([(s, r[:h], list(range(h))) for s, r, h in zip(slots, reqs, heads)])
    off = 0
    for i, h in enumerate(heads):
        got[i].append(out[off:off + h])
        off += h
    pos = list(heads)
    live = [i for i in range(len(reqs)) if pos[i] < len(reqs[i])]
    for i in range(len(reqs)):
        if i not in live:
            eng.close(slots[i])
    while live:
        out = eng.step([(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
        for j, i in enumerate(live):
            got[i].append(out[j:j + 1])
            pos[i] += 1
        for i in [i for i in live if pos[i] >= len(reqs[i])]:
            eng.close(slots[i])
        live = [i for i in live if pos[i] < len(reqs[i])]
    return [torch.cat(g) for g in got], slots


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", CASES)
def test_unequal_batches_one_after_another(name, sharp, dtype):
    eng = G.engine(name, dtype, sharp)
    lens = LENS[name]
    used = []
    for round_ in range(3):
        reqs = G.prompts(name, lens[round_:] + lens[:round_], seed=300 + 10 * round_)
        tails = [min(len(r) - 1, (3 + 5 * i + round_) % 13) for i, r in enumerate(reqs)]
        G.poison_free_pages(eng)
        outs, slots = run_batch(eng, reqs, tails)
        used.append(sorted(slots))
        for r, o in zip(reqs, outs):
            G.close(o, G.plain_logits(name, r, sharp), dtype, "%s round %d len %d" % (name, round_, len(r)))
        eng.cache.check()
        assert eng.cache.slots.n_held == 0 and all(g.pool.n_held == 0 for g in eng.cache.kv_groups)
    assert used[0] == used[1] == used[2]                 # the same slots, again and again


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,seed", [("A", 1), ("B", 2), ("B", 3), ("C", 4)])
def test_batches_of_random_sizes_shrink_through_every_kind_of_step(name, seed, dtype):
    """Up to 44 requests start together with unequal prompts and tails of unequal lengths, so the
    steps run from many rows down to one: through the library's products (prompts), the kernels
    for 17 to 64 rows, the folded few-row kernels, and every change from one to the next."""
    import random
    rng = random.Random(seed)
    sharp = name != "A"
    eng = G.engine(name, dtype, sharp)
    top = {"A": 100, "B": 80, "C": 120}[name]
    for round_ in range(2):
        n = rng.choice([18, 33, 44]) if round_ == 0 else rng.randint(2, 30)
        lens = [rng.randint(2, top) for _ in range(n)]
        reqs = G.prompts(name, lens, seed=900 + 17 * seed + round_)
        tails = [rng.randint(0, min(len(r) - 1, 24)) for r in reqs]
        G.poison_free_pages(eng)
        outs, _ = run_batch(eng, reqs, tails)
        for i, (r, o) in enumerate(zip(reqs, outs)):
            G.close(o, G.plain_logits(name, r, sharp), dtype, "%s seed %d round %d request %d (len %d, tail %d)"
                    % (name, seed, round_, i, len(r), tails[i]))
        eng.cache.check()
        assert eng.cache.slots.n_held == 0


PIECES = {"B": [2, 7, 31, 33], "C": [2, 7, 63, 64, 65, 129]}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_prompts_fed_in_pieces(name, dtype):
    """A prompt fed in pieces of 2, 7, 63, 64, 65, ... tokens (each piece a step of several tokens
    behind what the cache already holds, the window crossing piece edges), beside a second
    request that takes part in some steps only and a third that is decoded one token at a time
    meanwhile; every place of every request against the plain implementation."""
    eng = G.engine(name, dtype, True)
    top = {"B": 96, "C": 640}[name]
    for piece in PIECES[name]:
        long, other, slow = G.prompts(name, [top - 6, min(top, 3 * piece + 1), top // 3], seed=1300 + piece)
        s_long, s_other, s_slow = eng.open(), eng.open(), eng.open()
        got = {"long": [], "other": [], "slow": []}
        at_long = at_other = at_slow = 0
        step = 0
        while at_long < len(long) or at_other < len(other) or at_slow < len(slow):
            items, names = [], []
            if at_long < len(long):
                toks = long[at_long:at_long + piece]
                items.append((s_long, toks, all_places(toks))), names.append(("long", len(toks)))
                at_long += len(toks)
            if at_other < len(other) and step % 2 == 1:                  # left out of every other step
                toks = other[at_other:at_other + piece + 1]
                items.append((s_other, toks, all_places(toks))), names.append(("other", len(toks)))
                at_other += len(toks)
            if at_slow < len(slow):
                items.append((s_slow, [slow[at_slow]], [0])), names.append(("slow", 1))
                at_slow += 1
            if items:
                out = eng.step(items)
                off = 0
                for who, n in names:
                    got[who].append(out[off:off + n])
                    off += n
            step += 1
        for s in (s_long, s_other, s_slow):
            eng.close(s)
        for who, toks in (("long", long), ("other", other), ("slow", slow)):
            G.close(torch.cat(got[who]), G.plain_logits(name, toks, True), dtype, "%s pieces of %d, request %s" % (name, piece, who))
    eng.cache.check()


@pytest.mark.parametrize("name,sharp", CASES)
@pytest.mark.parametrize("mode", ["decode", "piece"])
def test_a_foreign_page_in_the_cache_is_noticed(name, sharp, mode):
    """The comparisons above can fail: with one page of one sequence's cache (keys and values of
    its first 64 positions, in the layers that see everything) replaced by another sequence's,
    the bfloat16 comparison with the plain implementation raises, for the sharpened and the
    plain random model alike, in one-token steps and in a prompt piece; the other sequence of
    the batch, whose cache is whole, still passes."""
    eng = G.engine(name, "bfloat16", sharp)
    n = {"A": 100, "B": 90, "C": 600}[name]
    p, other = G.prompts(name, [n, n], seed=1400)
    ref, ref_other = G.plain_logits(name, p, sharp), G.plain_logits(name, other, sharp)
    k = n - 8
    for spoil in (False, True):
        s, s2 = eng.open(), eng.open()
        eng.step([(s, p[:k], []), (s2, other[:k], [])])
        if spoil:
            g = next(g for g in eng.cache.kv_groups if g.need.window is None)
            a, b = g.pages[s][0], g.pages[s2][0]
            g.keys[:, a], g.values[:, a] = g.keys[:, b].clone(), g.values[:, b].clone()
        if mode == "decode":
            outs = [eng.step([(s, [p[t]], [0]), (s2, [other[t]], [0])]) for t in range(k, n)]
            got, got_other = torch.cat([o[:1] for o in outs]), torch.cat([o[1:] for o in outs])
        else:
            out = eng.step([(s, p[k:], list(range(8))), (s2, other[k:], list(range(8)))])
            got, got_other = out[:8], out[8:]
        eng.close(s), eng.close(s2)
        G.close(got_other, ref_other[k:], "bfloat16", "the untouched sequence")
        if spoil:
            with pytest.raises(AssertionError):
                G.close(got, ref[k:], "bfloat16")
        else:
            G.close(got, ref[k:], "bfloat16", "the clean run")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype):
    # 70 prompt tokens, then 400 single steps: across pages and far beyond the window
    eng = G.engine("C", dtype, True)
    p = G.prompts("C", [470], seed=400)[0]
    ref = G.plain_logits("C", p, True)
    s = eng.open()
    outs = [eng.step([(s, p[:70], all_places(p[:70]))])]
    for t in range(70, len(p)):
        outs.append(eng.step([(s, [p[t]], [0])]))
    win = next(g for g in eng.cache.kv_groups if g.need.window)
    assert win.pool.n_held <= 3                           # the window of 100 never needs more than 3 pages
    eng.close(s)
    G.close(torch.cat(outs), ref, dtype, "long decode")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_of_a_sequence(name, dtype):
    eng = G.engine(name, dtype, True)
    p = G.prompts(name, [6], seed=500)[0]
    ref = G.plain_logits(name, p, True)
    s = eng.open()
    outs = [eng.step([(s, [tok], [0])]) for tok in p]      # from the very first token on, one at a time
    eng.close(s)
    G.close(torch.cat(outs), ref, dtype, "first tokens")
    s = eng.open()
    out = eng.step([(s, p[:1], [0])])                      # a prompt of one token
    eng.close(s)
    G.close(out, ref[:1], dtype, "prompt of one")


def test_wanted_places_and_their_order():
    eng = G.engine("A", "float32")
    a, b = G.prompts("A", [9, 14], seed=600)
    sa, sb = eng.open(), eng.open()
    out = eng.step([(sa, a, [8, 0]), (sb, b, []), ])
    assert out.shape == (2, 256)
    ref = G.plain_logits("A", a)
    G.close(out, ref[[8, 0]], "float32")
    out = eng.step([(sb, [3], [0]), (sa, [4], [])])
    G.close(out, G.plain_logits("A", b + [3])[-1:], "float32")
    eng.close(sa), eng.close(sb)


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("B", "bfloat16"), ("C", "float32"), ("C", "bfloat16")])
def test_few_wanted_places_in_any_order_equal_all_places(name, dtype):
    # where a step wants fewer places than it has tokens, the last layer computes only those
    # (its keys and values still go to the cache for all tokens): wanted places out of order, twice,
    # in neighbouring runs, at a window's edge, in several sequences, and none at all; then
    # decoding goes on from the cache that such steps left
    eng = G.engine(name, dtype, True)
    ps = G.prompts(name, [90, 70, 9, 33], seed=1200)
    wants = [[89, 0, 1, 2, 77, 77, 64, 63], [], [8], [5, 4, 3]]
    slots = [eng.open() for _ in ps]
    full = eng.step([(s, p, all_places(p)) for s, p in zip(slots, ps)])
    for s in slots:
        eng.close(s)
    slots = [eng.open() for _ in ps]
    few = eng.step([(s, p, w) for s, p, w in zip(slots, ps, wants)])
    offsets = [0, 90, 160, 169]
    rows = [o + j for o, w in zip(offsets, wants) for j in w]
    assert few.shape[0] == len(rows)
    if dtype == "float32":
        assert torch.equal(few, full[rows])
    else:
        G.close(few, full[rows].cpu(), dtype)
    nxt = eng.step([(s, [7], [0]) for s in slots])
    for i, p in enumerate(ps):
        G.close(nxt[i:i + 1], G.plain_logits(name, p + [7], True)[-1:], dtype)
    for s in slots:
        eng.close(s)
    eng.cache.check()


def test_float32_results_do_not_depend_on_the_cut_at_all():
    # in float32 every kernel sums in an order that depends on the position only
    eng = G.engine("C", "float32", True)
    p, q = G.prompts("C", [200, 90], seed=700)
    s = eng.open()
    whole = eng.step([(s, p, all_places(p))])
    eng.close(s)
    s, s2 = eng.open(), eng.open()
    parts = [eng.step([(s2, q, []), (s, p[:37], all_places(p[:37]))])]
    parts.append(eng.step([(s, p[37:150], list(range(113)))]))
    for t in range(150, 200):
        parts.append(eng.step([(s, [p[t]], [0]), (s2, [q[t - 150]], [])]))
    eng.close(s), eng.close(s2)
    assert torch.equal(torch.cat(parts), whole)


def test_step_refuses_what_it_cannot_run():
    from tq_kv_amd import StepError
    from tq_kv_amd.cache import CacheFull
    eng = G.engine("A", "float32")
    s = eng.open()
    with pytest.raises(StepError, match="vocabulary"):
        eng.step([(s, [1, 256], [0])])
    with pytest.raises(StepError, match="Empty prompt"):
        eng.step([(s, [], [])])
    with pytest.raises(StepError, match="positions"):
        eng.step([(s, [1] * 129, [0])])
    with pytest.raises(StepError, match="twice"):
        eng.step([(s, [1], [0]), (s, [2], [0])])
    with pytest.raises(IndexError):
        eng.step([(s, [1, 2], [2])])
    # nothing of a refused step stays behind: no position, no page
    assert eng.length(s) == 0 and all(g.pool.n_held == 0 for g in eng.cache.kv_groups)
    eng.close(s)
    from tq_kv_amd import Engine
    small = Engine(eng.model, max_tokens=128)
    a, b = small.open(), small.open()
    small.step([(a, [1] * 64, [])])
    with pytest.raises(CacheFull):
        small.step([(a, [1], []), (b, [1] * 65, [])])
    assert small.length(a) == 64 and small.length(b) == 0
    small.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_tokens_given_on_the_device_equal_tokens_given_by_the_host(dtype):
    from tq_kv_amd import StepError
    # one-token steps whose tokens the host does not know (chosen by a kernel just before)
    eng = G.engine("A", dtype, True)
    reqs = G.prompts("A", [9, 4, 13], seed=1100)
    for device_side in (False, True, True):           # the second device-side round replays the graph
        slots = [eng.open() for _ in reqs]
        eng.step([(s, r[:-3], []) for s, r in zip(slots, reqs)])
        outs = []
        for k in range(3, 0, -1):
            toks = [r[-k] for r in reqs]
            if device_side:
                dev = torch.tensor(toks, dtype=torch.int32, device=eng.model.device)
                outs.append(eng.step([(s, [0], [0]) for s in slots], device_tokens=dev))
            else:
                outs.append(eng.step([(s, [t], [0]) for s, t in zip(slots, toks)]))
        if device_side:
            for a, b in zip(outs, want):
                assert torch.equal(a, b)
        else:
            want = outs
        for s in slots:
            eng.close(s)
    with pytest.raises(StepError, match="one token per sequence"):
        s = eng.open()
        eng.step([(s, [1, 2], [1])], device_tokens=torch.zeros(1, dtype=torch.int32, device=eng.model.device))
    eng.close(s)
    with pytest.raises(StepError, match="int32"):
        s = eng.open()
        eng.step([(s, [1], [0])], device_tokens=torch.zeros(2, dtype=torch.int32, device=eng.model.device))
    eng.close(s)


# ---- generation through the entry point -------------------------------------------------------
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_float32_equals_plain(name):
    from tq_kv_amd import GenerationParams, generate
    eng = G.engine(name, "float32", True)
    cfg, w = G.plain_model(name, True)
    ps = G.prompts(name, [5, 11, 17] if name == "A" else [1, 7, 20, 33], seed=800)
    n_new = 8 if name == "A" else 10
    out = generate(eng, ps, GenerationParams(max_tokens=n_new, temperature=0.0, repeat_penalty=1.0))
    for p, o in zip(ps, out):
        assert o == plain.generate_greedy(w, cfg, p, n_new)
    # prompts fed in pieces of at most 7 tokens (pieces of which nothing is wanted among them)
    assert generate(eng, ps, GenerationParams(max_tokens=n_new, temperature=0.0, repeat_penalty=1.0), max_step_tokens=7) == out
    # stop tokens: ending one request early leaves the others as they were
    stop = out[1][2]
    out2 = generate(eng, ps, GenerationParams(max_tokens=n_new, temperature=0.0, repeat_penalty=1.0), eos_ids=[stop])
    for p, o in zip(ps, out2):
        assert o == plain.generate_greedy(w, cfg, p, n_new, eos_ids=(stop,))
    assert len(out2[1]) <= 2
    eng.cache.check()
    assert eng.cache.slots.n_held == 0


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_bfloat16_picks_a_best_token_each_time(name):
    # bfloat16 logits differ a little from the plain ones, so a near-tie may go the other
    # way; what must hold is that every chosen token is (nearly) the plain implementation's
    # best one given the tokens chosen so far
    from tq_kv_amd import GenerationParams, generate
    eng = G.engine(name, "bfloat16", True)
    ps = G.prompts(name, [5, 11, 17], seed=810)
    out = generate(eng, ps, GenerationParams(max_tokens=8, temperature=0.0, repeat_penalty=1.0))
    for p, o in zip(ps, out):
        assert len(o) == 8
        ref = G.plain_logits(name, p + o, True)
        for i, tok in enumerate(o):
            row = ref[len(p) - 1 + i]
            assert row[tok] >= row.max() - 2 * G.BF16_SPREAD * row.std().item()


@pytest.mark.parametrize("name", ["A", "B"])
def test_sampled_generation_float32_equals_plain(name):
    from tq_kv_amd import GenerationParams, generate
    eng = G.engine(name, "float32", True)
    cfg, w = G.plain_model(name, True)
    ps = G.prompts(name, [1, 7, 20, 33], seed=820)
    for kw in (dict(temperature=0.8, top_k=0, top_p=1.0, repeat_penalty=1.0),
               dict(temperature=0.8, top_k=40, top_p=0.9, repeat_penalty=1.1),
               dict(temperature=0.0, top_k=0, top_p=1.0, repeat_penalty=1.3)):
        out = generate(eng, ps, GenerationParams(max_tokens=10, seed=5, **kw))
        for r, (p, o) in enumerate(zip(ps, out)):
            want = plain.generate(w, cfg, p, 10, temperature=kw["temperature"], top_k=kw["top_k"], top_p=kw["top_p"],
                                  penalty=kw["repeat_penalty"], seed=5, request=r)
            assert o == want, (kw, r)
    # what a request draws does not depend on its batch: alone, as request 2 of the run
    alone = generate(eng, ps, GenerationParams(max_tokens=10, seed=5, temperature=0.8, top_k=0, top_p=1.0,
                                               repeat_penalty=1.0), max_batch=1)
    together = generate(eng, ps, GenerationParams(max_tokens=10, seed=5, temperature=0.8, top_k=0, top_p=1.0,
                                                  repeat_penalty=1.0), max_batch=4)
    assert alone == together


@pytest.fixture(params=["own", "library", "rows"])
def products_of_17_to_128_rows(request):
    """The kernel for 17 to 128 rows (the default), the library's products in its place, and
    weights without a packed copy (then the few-row kernels read the rows and 17 rows on the library)."""
    from tq_kv_amd import POLICY
    old = dict(POLICY.items())
    if request.param == "library":
        POLICY["mid"] = False
    if request.param == "rows":
        POLICY["packed"] = False
    yield request.param
    POLICY.update(old)


@pytest.mark.parametrize("n_seqs", [40, 100])
@pytest.mark.parametrize("dtype", DTYPES)
def test_many_sequences_decode_through_replayed_graphs(dtype, products_of_17_to_128_rows, n_seqs):
    # 40 or 100 sequences: more rows than the few-row products take, so the captured step holds the
    # products for 17 to 128 rows (4 and 8 groups of 16 rows); every replay is checked (with other
    # work between the replays)
    if dtype == "float32" and products_of_17_to_128_rows != "own":
        pytest.skip("the switches are for bfloat16 products")
    if products_of_17_to_128_rows == "own":
        eng = G.engine("B", dtype, True)
    else:       # weights loaded and graphs captured under the switched policy
        from tq_kv_amd import Engine, Model
        eng = Engine(Model.from_dir(G.folder("B", True), dtype=dtype), max_tokens=8192)
    reqs = G.prompts("B", [3 + (7 * i) % 50 for i in range(n_seqs)], seed=1000)
    slots = [eng.open() for _ in reqs]
    heads = [len(r) - 6 for r in reqs]
    heads = [max(1, h) for h in heads]
    eng.step([(s, r[:h], []) for s, r, h in zip(slots, reqs, heads)])
    pos = list(heads)
    refs = [G.plain_logits("B", r, True) for r in reqs]
    n_graphs = len(eng.graphs)
    for step in range(6):
        live = [i for i in range(len(reqs)) if pos[i] < len(reqs[i])]
        if not live:
            break
        out = eng.step([(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
        torch.zeros(1000, device=out.device).add_(1.0)           # unrelated work between replays
        for j, i in enumerate(live):
            G.close(out[j], refs[i][pos[i]], dtype, "seq %d at %d (step %d)" % (i, pos[i], step))
            pos[i] += 1
    assert len(eng.graphs) > n_graphs
    for s in slots:
        eng.close(s)
    eng.cache.check()


# ---- decoding steps of more sequences than the graphs and the own products take ---------------------
@pytest.mark.parametrize("n_seqs", [128, 129, 200])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", [("B", True), ("D", False)])
def test_decode_steps_of_a_hundred_and_more_sequences(name, sharp, dtype, n_seqs):
    """Steps of exactly 128 sequences (the last that is captured as a graph and runs the own products), of 129 and of
    200 (eager, the library's products, the decoding attention kernel with more than 128 rows), and on the way down
    the steps either side of every change of kernels: 128 and 127, 17 and 16.  Sequences of unequal lengths; every
    row of every step against the plain implementation."""
    eng = G.engine(name, dtype, sharp, max_tokens=64 * 256)
    lens = [1 + (5 * i) % 13 for i in range(n_seqs)]
    reqs = G.prompts(name, [n + 9 for n in lens], seed=3000)
    refs = [G.plain_logits(name, r, sharp) for r in reqs]
    slots = [eng.open() for _ in reqs]
    out = eng.step([(s, r[:n], [n - 1]) for s, r, n in zip(slots, reqs, lens)])
    for i in range(n_seqs):
        G.close(out[i], refs[i][lens[i] - 1], dtype, "seq %d, last place of its prompt" % i)
    pos = list(lens)
    live = list(range(n_seqs))
    for count in [n_seqs, 128, 127, 64, 17, 16, 1]:
        while len(live) > count:                 # the sequences in the middle of the batch end first
            eng.close(slots[live.pop(len(live) // 2)])
        out = eng.step([(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
        for j, i in enumerate(live):
            G.close(out[j], refs[i][pos[i]], dtype, "seq %d at %d in a step of %d" % (i, pos[i], len(live)))
            pos[i] += 1
    assert len(eng.graphs) >= 6                    # the steps of up to 128 sequences went through captured graphs
    for i in live:
        eng.close(slots[i])
    eng.cache.check()
    assert eng.cache.slots.n_held == 0

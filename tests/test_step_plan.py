"""The arrays of a step as the engine's host library lays them out (tqe_plan_step), without a
GPU: against a plain construction of the same arrays, for random batches."""
import random

import numpy as np
import pytest
import torch

from tq_kv_amd import native
from tq_kv_amd.cache import PAGE, Cache, CacheFull
from tq_kv_amd.engine.context import StepContext
from tq_kv_amd.parts.spec import KVNeed


def plain_arrays(items, want):
    lens = [len(t) for _, _, t in items]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tok_seq = np.repeat(np.arange(len(items)), lens)
    tok_pos = np.concatenate([np.arange(start, start + n) for (_, start, _), n in zip(items, lens)])
    rows = [int(cu[i]) + j for i, w in enumerate(want) for j in w]
    last = sorted(set(rows))
    all_decode = all(n == 1 for n in lens)
    prune = not all_decode and len(last) < sum(lens)
    return dict(tokens=np.concatenate([t for _, _, t in items]), tok_seq=tok_seq, tok_pos=tok_pos,
                seq_slot=[s for s, _, _ in items], seq_start=[s for _, s, _ in items], seq_new=lens, cu=cu, want_rows=rows,
                last_rows=last if prune else [], want_in_last=[last.index(r) for r in rows] if prune else [],
                last_seq=[int(tok_seq[r]) for r in last] if prune else [], last_pos=[int(tok_pos[r]) for r in last] if prune else []), \
        dict(n_tokens=sum(lens), n_last=len(last), all_decode=all_decode, prune_last=prune, max_new=max(lens),
             max_end=max(s + n for (_, s, _), n in zip(items, lens)))


def test_step_arrays_equal_a_plain_construction():
    rng = random.Random(3)
    cache = Cache([KVNeed(2, 16, None), KVNeed(2, 16, 100)], [None, None], PAGE * 64, 8, torch.float32, "cpu")
    slots = [cache.acquire() for _ in range(6)]
    for round_ in range(40):
        chosen = rng.sample(slots, rng.randint(1, len(slots)))
        decode = rng.random() < 0.4
        items, want = [], []
        for s in chosen:
            n = 1 if decode else rng.choice([1, 2, 7, 64, 65, 130])
            if cache.length(s) + n > 1000:
                cache.release(s)
                slots[slots.index(s)] = s = cache.acquire()
            items.append((s, cache.length(s), [rng.randrange(1000) for _ in range(n)]))
            want.append([rng.randrange(n) for _ in range(rng.choice([0, 1, 1, 3]))] if rng.random() < 0.8 else list(range(n)))
        sizes = [(s, len(t)) for s, _, t in items]
        cache.reserve(sizes)
        step = rng.choice([1, 8])
        ctx = StepContext(items, want, cache, None, None, step, into=object())
        arrays, facts = plain_arrays(items, want)
        for name, value in arrays.items():
            assert getattr(ctx.host, name).tolist() == [int(v) for v in value], (round_, name)
        for name, value in facts.items():
            assert getattr(ctx, name) == value, (round_, name)
        for g, table in zip(cache.kv_groups, ctx.host_tables):
            want_table = cache.page_table(g, [s for s, _, _ in items])
            width = (want_table.shape[1] + step - 1) // step * step
            assert table.shape == (len(items), width)
            assert table[:, :want_table.shape[1]].tolist() == want_table.tolist() and (table[:, want_table.shape[1]:] == -1).all()
        assert ctx.shape_key() == (facts["n_tokens"], len(items), len(arrays["want_rows"]), tuple(t.shape[1] for t in ctx.host_tables))
        cache.commit(sizes)
        cache.check()
    with pytest.raises(IndexError, match="wanted place 2"):
        StepContext([(slots[0], 0, [1, 2])], [[2]], cache, None, None, 1, into=object())


def test_the_native_cache_reports_what_goes_wrong():
    c = native.NativeCache(2, [(3, 0)])
    a, b = c.acquire(), c.acquire()
    assert (a, b) == (0, 1) and c.counts(-1) == (0, 2)
    with pytest.raises(CacheFull, match="0 free of 2"):
        c.acquire()
    c.release(a)
    with pytest.raises(AssertionError, match="slot 0 given back but not held"):
        c.release(a)
    with pytest.raises(AssertionError, match="slot 0 is not held"):
        c.reserve([(a, 1)])
    assert c.acquire() == a                       # what came back last goes out first
    c.reserve([(a, PAGE + 1)])
    first = c.pages(0, a)
    assert len(set(first)) == 2 and all(0 <= p < 3 for p in first) and c.pages(0, b) is None and c.counts(0) == (1, 3)
    with pytest.raises(CacheFull, match="2 more pages"):
        c.reserve([(b, 2 * PAGE)])
    assert c.pages(0, b) is None and c.counts(0) == (1, 3)        # nothing was taken
    c.commit([(a, PAGE + 1)])
    assert c.length(a) == PAGE + 1
    c.check()
    with pytest.raises(native.EngineLibraryError, match="no slot 7"):
        c.length(7)


def test_the_library_refuses_steps_that_cannot_run():
    c = native.NativeCache(3, [(8, 0)])
    a, b = c.acquire(), c.acquire()
    i32 = lambda *v: np.asarray(v, dtype=np.int32)
    c.check_step(i32(a, b), i32(2, 1), i32(0, 99, 5), 100, 128)
    c.check_step(i32(a), i32(1), None, 100, 128)               # tokens the host does not know
    for slots, n_new, tokens, vocab, positions, what in [
            (i32(), i32(), i32(), 100, 128, "at least one sequence"),
            (i32(a, a), i32(1, 1), i32(1, 2), 100, 128, "slot 0 appears twice"),
            (i32(a, b), i32(1, 0), i32(1), 100, 128, "Empty prompt"),
            (i32(a, b), i32(2, 1), i32(1, 2, 100), 100, 128, "token id 100 is outside the vocabulary of 100"),
            (i32(a), i32(1), i32(-1), 100, 128, "token id -1"),
            (i32(a), i32(129), i32(*([1] * 129)), 100, 128, "would reach 129 positions, the model has 128")]:
        with pytest.raises(native.StepError, match=what):
            c.check_step(slots, n_new, tokens, vocab, positions)
    with pytest.raises(AssertionError, match="slot 2 is not held"):
        c.check_step(i32(2), i32(1), i32(1), 100, 128)
    c.reserve([(a, 100)]), c.commit([(a, 100)])
    c.check_step(i32(a), i32(28), None, 100, 128)
    with pytest.raises(native.StepError, match="would reach 129 positions"):
        c.check_step(i32(a), i32(29), None, 100, 128)


def test_runs_of_pages_lie_an_odd_number_of_pages_apart():
    # equally long prompts would otherwise get runs of pages a power of two apart in memory
    for run in (32, 31, 16, 2):
        c = native.NativeCache(8, [(8 * 40, 0)])
        slots = [c.acquire() for _ in range(6)]
        c.reserve([(s, run * PAGE) for s in slots])
        c.commit([(s, run * PAGE) for s in slots])
        firsts = [c.pages(0, s)[0] for s in slots]
        for s in slots:
            pages = c.pages(0, s)
            assert pages == list(range(pages[0], pages[0] + run))          # a run of neighbours
        assert all((b - a) % 2 == 1 and b - a <= run + 2 for a, b in zip(firsts, firsts[1:])), (run, firsts)
        # single pages, as decoding takes them, pass nothing over; what was passed over is still free
        c.reserve([(s, 1) for s in slots])
        tails = [c.pages(0, s)[-1] for s in slots]
        assert tails == list(range(tails[0], tails[0] + 6))
        free, n = c.counts(0)
        assert free == 8 * 40 - 6 * (run + 1) and n == 8 * 40
        c.check()
    # a pool that has exactly what is needed gives it all
    c = native.NativeCache(2, [(64, 0)])
    a, b = c.acquire(), c.acquire()
    c.reserve([(a, 32 * PAGE), (b, 32 * PAGE)])
    assert sorted(c.pages(0, a) + c.pages(0, b)) == list(range(64))
    c.check()


def test_the_library_refuses_negative_counts_and_changes_nothing():
    """What no caller of the engine can send but a C caller might: negative numbers of wanted places or of new
    positions.  Each is a status and a message (no exception escapes the library), and nothing was changed."""
    c = native.NativeCache(3, [(8, 0)])
    a, b = c.acquire(), c.acquire()
    i32 = lambda *v: np.asarray(v, dtype=np.int32)
    with pytest.raises(native.EngineLibraryError, match="wants -1 places"):
        native.plan_step(c, i32(a), i32(0), i32(1), i32(5), i32(-1), i32(), 1)
    with pytest.raises(native.EngineLibraryError, match="-3 new positions"):
        c.reserve([(a, 2), (b, -3)])
    assert c.pages(0, a) is None and c.counts(0) == (8, 8)
    c.reserve([(a, 70), (b, 1)])
    with pytest.raises(native.EngineLibraryError, match="-1000000000 new positions"):
        c.commit([(a, 70), (b, -10 ** 9)])
    assert c.length(a) == 0 and c.length(b) == 0                   # commit is all or nothing: a was not committed either
    with pytest.raises(AssertionError, match="slot 2 is not held"):
        c.commit([(a, 70), (2, 1)])
    assert c.length(a) == 0
    with pytest.raises(AssertionError, match="were not reserved"):
        c.commit([(a, 200)])
    c.commit([(a, 70), (b, 1)])
    assert (c.length(a), c.length(b)) == (70, 1)
    # a reservation that is given back: the pages beyond what the lengths need are free again
    c.reserve([(a, 100), (b, 64)])
    assert c.counts(0)[0] == 8 - 3 - 2
    c.trim([a, b])
    assert c.counts(0)[0] == 8 - 2 - 1 and len(c.pages(0, a)) == 2 and len(c.pages(0, b)) == 1
    c.check()


def test_pages_that_were_passed_over_come_back_into_use_on_an_engine_that_is_never_idle():
    """Requests that overlap for ever: some sequence is always live, so the pool is never wholly free.  The pages that
    were passed over to space the runs must not pile up at the end of the free list for good: after many rounds a new
    prompt still gets a run of neighbouring pages."""
    c = native.NativeCache(4, [(6 * 40, 0)])
    live = [c.acquire()]
    c.reserve([(live[0], 32 * PAGE)]), c.commit([(live[0], 32 * PAGE)])
    for round_ in range(200):
        s = c.acquire()
        c.reserve([(s, 32 * PAGE)]), c.commit([(s, 32 * PAGE)])
        pages = c.pages(0, s)
        assert pages == list(range(pages[0], pages[0] + 32)), (round_, pages)          # a run of neighbours every time
        live.append(s)
        c.release(live.pop(0))                                                      # the older one ends: never idle
        c.check()
    assert c.counts(0)[0] == 6 * 40 - 32

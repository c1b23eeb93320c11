"""The generation loop's decisions, with a stand-in engine and sampler (no GPU): which
tokens are fed, emitted and stopped on, when slots come back, how requests are cut into
batches."""
import pytest

from tq_kv_amd import GenerationError, GenerationParams, generate
from tq_kv_amd.engine.generate import plan_batches


class FakeEngine:
    """Its "logits" for a sequence are just (slot, tokens seen so far); it records steps."""
    max_positions = 10000

    def __init__(self, max_tokens=64 * 64, n_slots=8):
        self.max_tokens = max_tokens
        self.free = list(range(n_slots - 1, -1, -1))
        self.seen = {}
        self.steps = []
        self.closed = []

    def open(self):
        s = self.free.pop()
        self.seen[s] = []
        return s

    def close(self, slot):
        assert slot in self.seen, "slot closed twice"
        del self.seen[slot]
        self.closed.append(slot)
        self.free.append(slot)

    def step(self, items):
        self.steps.append([(s, list(t)) for s, t, _ in items])
        out = []
        for s, toks, want in items:
            self.seen[s].extend(toks)
            assert want in ([len(toks) - 1], [])
            if want:
                out.append(list(self.seen[s]))
        return out


class ScriptSampler:
    """Draws for request r the next token of scripts[r], whatever the logits."""

    def __init__(self, scripts, request_ids):
        self.scripts = [list(scripts[r]) for r in request_ids]
        self.calls = []

    def sample(self, logits, rows):
        assert len(logits) == len(rows)
        self.calls.append(list(rows))
        return [self.scripts[r].pop(0) for r in rows]


def run(prompts, scripts, max_tokens, eos=(), **kw):
    eng = kw.pop("engine", None) or FakeEngine()
    events = []
    out = generate(eng, prompts, GenerationParams(max_tokens=max_tokens, temperature=0.0), eos_ids=eos,
                   on_tokens=events.append, make_sampler=lambda p, ids: ScriptSampler(scripts, ids), **kw)
    return out, eng, events


def test_one_request_prompt_then_one_token_each():
    out, eng, events = run([[5, 6, 7]], [[10, 11, 12, 13]], 3)
    assert out == [[10, 11, 12]]
    # the prompt whole, then each emitted token but the last is fed (src/engine.rs:364-397)
    assert eng.steps == [[(0, [5, 6, 7])], [(0, [10])], [(0, [11])]]
    assert events == [[(0, 10)], [(0, 11)], [(0, 12)]]
    assert eng.seen == {} and eng.closed == [0]


def test_stop_token_ends_without_being_emitted():
    out, eng, _ = run([[1, 2]], [[10, 11, 99, 12]], 8, eos=(99,))
    assert out == [[10, 11]] and eng.steps[-1] == [(0, [11])]
    out, eng, _ = run([[1, 2]], [[99]], 8, eos=(99,))
    assert out == [[]] and len(eng.steps) == 1


def test_zero_max_tokens_emits_nothing():
    out, eng, _ = run([[1, 2]], [[10]], 0)
    assert out == [[]] and eng.seen == {}


def test_shorter_requests_leave_the_batch_and_free_their_slot():
    scripts = [[10, 99], [20, 21, 22, 23, 24], [30, 31, 99]]
    out, eng, events = run([[1], [2, 2], [3, 3, 3]], scripts, 4, eos=(99,))
    assert out == [[10], [20, 21, 22, 23], [30, 31]]
    assert eng.steps[0] == [(0, [1]), (1, [2, 2]), (2, [3, 3, 3])]
    assert eng.steps[1] == [(0, [10]), (1, [20]), (2, [30])]
    assert eng.steps[2] == [(1, [21]), (2, [31])]
    assert eng.steps[3] == [(1, [22])] and len(eng.steps) == 4
    assert eng.closed == [0, 2, 1] and eng.seen == {}
    assert events[0] == [(0, 10), (1, 20), (2, 30)] and events[-1] == [(1, 23)]


def test_batches_follow_one_another_and_reuse_slots():
    prompts = [[1] * 10, [2] * 10, [3] * 10, [4] * 10, [5] * 10]
    scripts = [[10 + i] * 5 for i in range(5)]
    out, eng, _ = run(prompts, scripts, 2, max_batch=2)
    assert out == [[10, 10], [11, 11], [12, 12], [13, 13], [14, 14]]
    firsts = [s for s in eng.steps if len(s[0][1]) == 10]
    assert [len(s) for s in firsts] == [2, 2, 1]
    assert {slot for s in eng.steps for slot, _ in s} == {0, 1}       # the same two slots serve all five
    assert eng.seen == {}


def test_long_prompts_are_fed_in_several_steps():
    from tq_kv_amd.engine.generate import _prompt_steps
    assert _prompt_steps([3, 4, 2], 100) == [[(0, 0, 3), (1, 0, 4), (2, 0, 2)]]
    assert _prompt_steps([3, 4, 2], 5) == [[(0, 0, 3), (1, 0, 2)], [(1, 2, 4), (2, 0, 2)]]
    assert _prompt_steps([7], 3) == [[(0, 0, 3)], [(0, 3, 6)], [(0, 6, 7)]]
    out, eng, _ = run([[1, 2, 3], [4, 5, 6, 7], [8, 9]], [[10, 11], [20, 21], [30, 31]], 2, max_step_tokens=5)
    assert out == [[10, 11], [20, 21], [30, 31]]
    assert eng.steps[0] == [(0, [1, 2, 3]), (1, [4, 5])] and eng.steps[1] == [(1, [6, 7]), (2, [8, 9])]
    assert eng.steps[2] == [(0, [10]), (1, [20]), (2, [30])] and len(eng.steps) == 3


def test_plan_batches_by_cache_room():
    # room of a request: prompt + max_new - 1 positions in whole pages of 64
    assert plan_batches([10, 10, 10], 5, 64 * 2, 8) == [[0, 1], [2]]
    assert plan_batches([64, 1], 2, 64 * 3, 8) == [[0, 1]]            # 65 -> 128, 2 -> 64
    assert plan_batches([60, 60, 60, 60], 5, 64 * 64, 3) == [[0, 1, 2], [3]]
    with pytest.raises(GenerationError, match="cache positions"):
        plan_batches([200], 5, 64 * 2, 8)


def test_errors():
    with pytest.raises(GenerationError, match="Empty prompt"):
        run([[]], [[1]], 3)
    eng = FakeEngine()
    eng.max_positions = 12
    with pytest.raises(GenerationError, match="positions"):
        run([[1] * 10], [[1] * 9], 4, engine=eng)


def test_slots_come_back_when_a_step_fails():
    class Boom(FakeEngine):
        def step(self, items):
            if len(self.steps) == 2:
                raise RuntimeError("boom")
            return super().step(items)
    eng = Boom()
    with pytest.raises(RuntimeError):
        run([[1], [2]], [[10] * 9, [20] * 9], 6, engine=eng)
    assert eng.seen == {} and sorted(eng.free) == list(range(8))


def test_params_have_the_reference_defaults():
    p = GenerationParams()
    assert (p.max_tokens, p.temperature, p.top_p, p.top_k, p.repeat_penalty, p.seed) == (512, 0.7, 0.9, 40, 1.1, 0)
    assert GenerationParams(temperature=0.0).greedy and not p.greedy
    with pytest.raises(ValueError):
        GenerationParams(top_p=0.0)
    assert "temperature=0.7" in repr(p)


# ---- running ahead: the next step is started before the draw has been read ---------------------
class AheadEngine(FakeEngine):
    """Takes a step's tokens "from the device": here a list that is only looked at when the
    step is recorded, as a device would."""
    takes_device_tokens = True

    def step(self, items, device_tokens=None, borrow=False):
        if device_tokens is not None:
            assert all(t == [0] for _, t, _ in items) and len(device_tokens) == len(items)
            items = [(s, [tok], w) for (s, _, w), tok in zip(items, device_tokens)]
        return FakeEngine.step(self, items)


class AheadSampler(ScriptSampler):
    class Draw:
        def __init__(self, tokens, log):
            self.tokens, self.log = tokens, log

        def read(self):
            self.log.append("read")
            return self.tokens

    def __init__(self, scripts, request_ids, log):
        ScriptSampler.__init__(self, scripts, request_ids)
        self.log = log

    def draw(self, logits, rows):
        self.log.append("draw")
        return self.Draw(ScriptSampler.sample(self, logits, rows), self.log)

    def pick(self, drawn, places):
        return [drawn.tokens[i] for i in places]


def run_ahead(prompts, scripts, max_tokens, eos=(), **kw):
    eng, log, events = AheadEngine(), [], []
    out = generate(eng, prompts, GenerationParams(max_tokens=max_tokens, temperature=0.0), eos_ids=eos,
                   on_tokens=events.append, make_sampler=lambda p, ids: AheadSampler(scripts, ids, log), **kw)
    return out, eng, events, log


CASES = [
    ([[5, 6, 7]], [[10, 11, 12, 13, 14, 15]], 3, ()),
    ([[5, 6, 7]], [[10, 11, 12, 13, 14, 15]], 1, ()),
    ([[5, 6, 7]], [[10, 11, 12, 13, 14, 15]], 0, ()),
    ([[1, 2]], [[10, 11, 99, 12, 13, 14]], 8, (99,)),
    ([[1, 2]], [[99, 1, 2, 3]], 8, (99,)),
    ([[1], [2, 2], [3, 3, 3]], [[10, 99, 7, 7], [20, 21, 22, 23, 24, 25], [30, 31, 99, 7, 7]], 4, (99,)),
    ([[1], [2, 2], [3, 3, 3]], [[10, 11, 12, 13, 99, 5, 5], [20, 99, 5, 5], [99, 5, 5]], 6, (99,)),
    ([[1] * 10, [2] * 10, [3] * 10, [4] * 10, [5] * 10], [[10 + i] * 9 for i in range(5)], 5, ()),
]


@pytest.mark.parametrize("prompts,scripts,max_tokens,eos", CASES)
def test_running_ahead_emits_the_same(prompts, scripts, max_tokens, eos):
    kw = {"max_batch": 2} if len(prompts) == 5 else {}
    want, plain_eng, want_events = run(prompts, scripts, max_tokens, eos, **kw)
    out, eng, events, _ = run_ahead(prompts, scripts, max_tokens, eos, **kw)
    assert out == want and events == want_events
    assert eng.seen == {} and sorted(eng.closed) == sorted(plain_eng.closed)        # every slot back, once
    # every step of the plain run is there, for the same slots and tokens; beyond them only rows of
    # requests whose stop token had not been read yet
    for plain_step, step in zip(plain_eng.steps, eng.steps):
        assert [x for x in step if x in plain_step] == plain_step


def test_running_ahead_starts_the_next_step_before_reading_the_draw():
    out, eng, _, log = run_ahead([[1, 2]], [[10, 11, 12, 13, 14]], 4)
    assert out == [[10, 11, 12, 13]]
    assert eng.steps == [[(0, [1, 2])], [(0, [10])], [(0, [11])], [(0, [12])]]
    # after the first decoding step there are always two draws under way when one is read
    assert log == ["draw", "draw", "read", "draw", "read", "read"]


def test_running_ahead_wastes_one_row_on_a_stop_token():
    out, eng, _, _ = run_ahead([[1], [2]], [[10, 11, 99, 5, 5], [20, 21, 22, 23, 24]], 5, eos=(99,))
    assert out == [[10, 11], [20, 21, 22, 23, 24]]
    # request 0's stop token 99 was fed once, because the step was started before it was read
    assert eng.steps[3] == [(0, [99]), (1, [22])] and eng.steps[4] == [(1, [23])]
    assert eng.seen == {}


def test_stop_tokens_default_to_those_the_model_names():
    class Named(FakeEngine):
        class model:
            stop_token_ids = (99,)
    make = lambda p, ids: ScriptSampler([[10, 99, 12]], ids)
    params = GenerationParams(max_tokens=8, temperature=0.0)
    assert generate(Named(), [[1]], params, make_sampler=make) == [[10]]
    assert generate(Named(), [[1]], params, eos_ids=(), make_sampler=lambda p, ids: ScriptSampler([[10, 99, 12] + [1] * 8], ids))[0][:3] == [10, 99, 12]
    assert generate(FakeEngine(), [[1]], GenerationParams(max_tokens=3, temperature=0.0), make_sampler=make) == [[10, 99, 12]]


def test_the_librarys_decisions_about_a_drawn_token():
    from tq_kv_amd import native
    p = native.BatchProgress(3, 3, {7, 9, 2 ** 40})        # three tokens each at most; 7 and 9 stop (an id no token can be is left out)
    assert [p.goes_on(r) for r in range(3)] == [True, True, True]
    assert p.accept(0, 5) == native.TOKEN_FEED and p.emitted(0) == 1 and p.goes_on(0)
    assert p.accept(0, 6) == native.TOKEN_FEED and p.emitted(0) == 2 and not p.goes_on(0)     # its next token will be its last
    assert p.accept(0, 8) == native.TOKEN_LAST and p.emitted(0) == 3 and p.ended(0)
    assert p.accept(0, 8) == native.TOKEN_DROPPED and p.emitted(0) == 3                        # a step that ran ahead for nothing
    assert p.accept(1, 9) == native.TOKEN_STOP and p.emitted(1) == 0 and p.ended(1) and not p.goes_on(1)
    assert p.accept(1, 5) == native.TOKEN_DROPPED
    assert p.accept(2, 2 ** 40) == native.TOKEN_FEED and not p.ended(2)
    with pytest.raises(native.EngineLibraryError, match="no request 3"):
        p.accept(3, 1)
    none_wanted = native.BatchProgress(1, 0, ())
    assert not none_wanted.goes_on(0) and none_wanted.accept(0, 5) == native.TOKEN_STOP and none_wanted.emitted(0) == 0
    one = native.BatchProgress(1, 1, ())
    assert not one.goes_on(0) and one.accept(0, 5) == native.TOKEN_LAST


def test_the_librarys_batches_and_prompt_steps():
    from tq_kv_amd import native
    from tq_kv_amd.cache import CacheFull
    assert native.plan_batches([], 5, 64, 4) == []
    assert native.plan_batches([1], 1, 64, 4) == [[0]]
    assert native.plan_batches([64, 64, 64], 1, 128, 8) == [[0, 1], [2]]            # 64 + 0 more positions: one page each
    assert native.plan_batches([64, 64, 64], 2, 128, 8) == [[0], [1], [2]]          # 65 positions: two pages each
    assert native.plan_batches([5] * 5, 3, 10 ** 12, 2) == [[0, 1], [2, 3], [4]]
    with pytest.raises(CacheFull, match="request 1 needs 192 cache positions, the engine has 128"):
        native.plan_batches([10, 129], 5, 128, 8)
    assert native.prompt_steps([], 8) == []
    assert native.prompt_steps([3, 4, 2], 5) == [[(0, 0, 3), (1, 0, 2)], [(1, 2, 4), (2, 0, 2)]]
    assert native.prompt_steps([10], 10) == [[(0, 0, 10)]]
    assert native.prompt_steps([2, 2, 2, 2], 4) == [[(0, 0, 2), (1, 0, 2)], [(2, 0, 2), (3, 0, 2)]]

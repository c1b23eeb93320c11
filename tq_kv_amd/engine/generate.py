"""The generation loop above the step function (csrc/engine/generate.cpp behind tqe_generate).

One request in the reference (src/engine.rs:364-438): the prompt whole, a first draw, then while
fewer than max_tokens tokens have been emitted: stop if the drawn token is a stop token (it is not
emitted), emit it, feed it, draw the next.  Here many requests run as batches that start together:
their prompts in one step, then one token each per step; a request that ends leaves the batch and
gives its slot back at once, the others go on unchanged; when a batch is done the next one starts,
until every request has been served.

The loop only decides; it computes nothing, and it is written against two small interfaces (an
engine: open, close, step; a sampler: sample).  With an Engine of this package and no sampler of
the caller's, `generate` runs it on the device sampler inside the library; with stand-ins (any
object with `open()`, `close(slot)`, `step(items)`, `max_tokens` and `max_positions`; any
`make_sampler(params, request_ids)` whose result has `sample(logits, rows)`) the same loop calls
back into Python, so its decisions can be tested without a GPU.
"""
import ctypes

import numpy as np

from .. import native
from ..native import CacheFull, GenerationError
from ..sampling.params import GenerationParams


def plan_batches(prompt_lens, max_new, max_tokens, max_batch, holds_pages=True):
    """Cut the requests, in order, into batches that fit the cache: at most max_batch
    requests and at most max_tokens positions (whole pages each; not counted where the
    engine's cache holds no pages: holds_pages False).  Returns lists of request indices."""
    try:
        return native.plan_batches(prompt_lens, max_new, max_tokens, max_batch, holds_pages)
    except CacheFull as e:
        raise GenerationError(str(e))


def _prompt_steps(lens, max_step_tokens):
    """Cut prompts of the given lengths into steps of at most max_step_tokens tokens.
    Returns steps, each a list of (index, begin, end); a prompt's pieces come in order."""
    return native.prompt_steps(lens, max_step_tokens)


def _c_params(params):
    return native.tqe_generation_params(int(params.max_tokens), float(params.temperature), float(params.top_p), int(params.top_k),
                                        float(params.repeat_penalty), int(params.seed) & 0xFFFFFFFFFFFFFFFF)


def generate(engine, prompts, params=None, eos_ids=None, on_tokens=None, max_batch=64, make_sampler=None,
             max_step_tokens=8192):
    """prompts: token-id lists.  Returns for each prompt the emitted token ids.

    eos_ids: stop tokens (default: those the engine's model names, Model.stop_token_ids; give ()
    for none).  on_tokens(pairs): called after every step with the (request index, token) pairs
    emitted by it.  make_sampler(params, request_ids): the sampler of a batch (default: the
    device sampler).  max_step_tokens: most tokens one step runs; a batch's prompts are fed in as
    many steps as that takes (whole prompts together while they fit, a longer prompt in pieces),
    which bounds the step's working memory."""
    from .engine import Engine
    params = params or GenerationParams()
    lib = native.library()
    prompts = [list(p) for p in prompts]
    n = len(prompts)
    lens = np.asarray([len(p) for p in prompts], dtype=np.int32)
    flat = np.asarray([t for p in prompts for t in p], dtype=np.int64).clip(-1, 2 ** 31 - 1).astype(np.int32)
    if len(flat) == 0:
        flat = np.zeros(1, dtype=np.int32)
    out_tokens = np.zeros(max(1, n * max(1, params.max_tokens)), dtype=np.int32)
    out_counts = np.zeros(max(1, n), dtype=np.int32)
    cp = _c_params(params)
    real = isinstance(engine, Engine) and make_sampler is None
    if eos_ids is None:
        eos_ids = getattr(getattr(engine, "model", None), "stop_token_ids", ())
    # a stop id is a token id: nothing negative, nothing beyond the library's int32
    eos = np.asarray(sorted(set(int(t) for t in eos_ids if 0 <= int(t) < 2 ** 31)), dtype=np.int32)

    def told(user, count, reqs, toks):
        try:
            on_tokens([(int(reqs[i]), int(toks[i])) for i in range(count)])
        except BaseException as e:      # noqa: B902
            native._pending_exception.append(e)
    cb = native.ON_TOKENS(told) if on_tokens is not None else ctypes.cast(None, native.ON_TOKENS)

    if real:
        status = lib.tqe_generate(engine.handle, n, native._ptr(lens), native._ptr(flat), ctypes.byref(cp), native._ptr(eos) if len(eos) else None,
                                  len(eos), int(max_batch), int(max_step_tokens), cb, None, native._ptr(out_tokens), native._ptr(out_counts),
                                  engine._stream())
    else:
        status = _generate_with(lib, engine, make_sampler, params, cp, n, lens, flat, eos, max_batch, max_step_tokens, cb, out_tokens, out_counts)
    if native._pending_exception:
        native._raise(status or native.ERR_PART)
    native.check(status)
    width = max(1, params.max_tokens)
    return [out_tokens[i * width:i * width + int(out_counts[i])].tolist() for i in range(n)]


def _generate_with(lib, engine, make_sampler, params, cp, n, lens, flat, eos, max_batch, max_step_tokens, cb, out_tokens, out_counts):
    """The library's loop over an engine and a sampler that live in Python."""
    state = {"logits": None, "sampler": None}
    error = native.CString()
    if make_sampler is None:
        from ..sampling.sampler import Sampler

        def make_sampler(p, request_ids):
            return Sampler(p, request_ids, engine.model.device)

    def guard(fn):
        def wrapped(*args):
            try:
                return fn(*args) or 0
            except BaseException as e:      # noqa: B902
                native._pending_exception.append(e)
                error.set(("%s: %s" % (type(e).__name__, e)).encode("utf-8", "replace"))
                return native.ERR_PART
        return wrapped

    @guard
    def c_open(user, slot_out):
        slot_out[0] = int(engine.open())

    @guard
    def c_close(user, slot):
        engine.close(int(slot))

    @guard
    def c_step(user, n_seqs, slots, n_new, tokens, want_last):
        items, at = [], 0
        for i in range(n_seqs):
            k = int(n_new[i])
            items.append((int(slots[i]), [int(tokens[at + j]) for j in range(k)], [k - 1] if want_last[i] else []))
            at += k
        state["logits"] = engine.step(items)

    @guard
    def c_batch(user, count, request_ids):
        state["sampler"] = make_sampler(params, [int(request_ids[i]) for i in range(count)])

    @guard
    def c_sample(user, n_rows, rows, out):
        toks = state["sampler"].sample(state["logits"], [int(rows[i]) for i in range(n_rows)])
        if len(toks) != n_rows:
            raise ValueError("the sampler gave %d tokens for %d rows" % (len(toks), n_rows))
        for i, t in enumerate(toks):
            t = int(t)
            out[i] = t if -2 ** 31 <= t < 2 ** 31 else -1        # no token id is negative: such a token stops nothing and is fed as it is

    def c_error(user):
        return error.address

    # running ahead: only where the engine takes a step's tokens from the device and the sampler can draw without waiting
    draws = {}
    borrow = {"borrow": True} if getattr(engine, "use_graphs", False) else {}

    @guard
    def c_draw(user, n_rows, rows, draw_out):
        draw_out[0] = state["next_draw"] = state.get("next_draw", 0) + 1
        draws[draw_out[0]] = state["sampler"].draw(state["logits"], [int(rows[i]) for i in range(n_rows)])

    @guard
    def c_ahead(user, n_seqs, slots, draw, places):
        tokens = state["sampler"].pick(draws[draw], [int(places[i]) for i in range(n_seqs)])
        state["logits"] = engine.step([(int(slots[i]), [0], [0]) for i in range(n_seqs)], device_tokens=tokens, **borrow)

    @guard
    def c_read(user, draw, count, out):
        toks = draws.pop(draw).read()
        if len(toks) != count:
            raise ValueError("a draw gave %d tokens for %d rows" % (len(toks), count))
        for i, t in enumerate(toks):
            t = int(t)
            out[i] = t if -2 ** 31 <= t < 2 ** 31 else -1

    probe = make_sampler(params, [0]) if bool(getattr(engine, "takes_device_tokens", False)) else None
    ahead = probe is not None and hasattr(probe, "draw") and hasattr(probe, "pick")
    none = lambda kind: ctypes.cast(None, kind)
    cbs = native.tqe_loop_callbacks(
        native.LOOP_OPEN(c_open), native.LOOP_CLOSE(c_close), native.LOOP_STEP(c_step), native.LOOP_BATCH(c_batch), native.LOOP_SAMPLE(c_sample),
        native.PART_ERROR(c_error), int(engine.max_tokens), int(engine.max_positions), int(getattr(engine, "max_slots", max_batch)),
        1 if getattr(engine, "holds_pages", True) else 0,
        native.LOOP_DRAW(c_draw) if ahead else none(native.LOOP_DRAW), native.LOOP_AHEAD(c_ahead) if ahead else none(native.LOOP_AHEAD),
        native.LOOP_READ(c_read) if ahead else none(native.LOOP_READ))
    return lib.tqe_generate_with(ctypes.byref(cbs), None, n, native._ptr(lens), native._ptr(flat), ctypes.byref(cp),
                                 native._ptr(eos) if len(eos) else None, len(eos), int(max_batch), int(max_step_tokens), cb, None,
                                 native._ptr(out_tokens), native._ptr(out_counts))

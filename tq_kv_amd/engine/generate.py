"""The generation loop above the step function.

One request in the reference (src/engine.rs:364-438): the prompt whole, a first draw,
then while fewer than max_tokens tokens have been emitted: stop if the drawn token is
a stop token (it is not emitted), emit it, feed it, draw the next.  Here many
requests run as batches that start together: their prompts in one step, then one
token each per step; a request that ends leaves the batch and gives its slot back at
once, the others go on unchanged; when a batch is done the next one starts, until
every request has been served.

The loop only decides; it computes nothing.  It needs of the engine `open()`,
`close(slot)`, `step(items)`, `max_tokens` and `max_positions`, and of the sampler
`sample(logits, rows)`, so it can be tested without a GPU.  The decisions themselves (which
requests run together, how prompts are cut into steps, what becomes of a drawn token) are the
engine's host library's (tqe_plan_batches, tqe_prompt_steps, tqe_batch_*); this file calls the
engine and the sampler in the order they ask for.
"""
from .. import native
from ..cache.pages import CacheFull
from ..sampling.params import GenerationParams


class GenerationError(ValueError):
    pass


def plan_batches(prompt_lens, max_new, max_tokens, max_batch, holds_pages=True):
    """Cut the requests, in order, into batches that fit the cache: at most max_batch
    requests and at most max_tokens positions (whole pages each; not counted where the
    engine's cache holds no pages: holds_pages False).  Returns lists of request indices."""
    try:
        return native.plan_batches(prompt_lens, max_new, max_tokens, max_batch, holds_pages)
    except CacheFull as e:
        raise GenerationError(str(e))


def generate(engine, prompts, params=None, eos_ids=None, on_tokens=None, max_batch=64, make_sampler=None,
             max_step_tokens=8192):
    """prompts: token-id lists.  Returns for each prompt the emitted token ids.

    eos_ids: stop tokens (default: those the engine's model names, Model.stop_token_ids; give ()
    for none).  on_tokens(pairs): called after every step with the
    (request index, token) pairs emitted by it.  make_sampler(params, request_ids): the
    sampler of a batch (default: the device sampler).  max_step_tokens: most tokens one step
    runs; a batch's prompts are fed in as many steps as that takes (whole prompts together
    while they fit, a longer prompt in pieces), which bounds the step's working memory."""
    params = params or GenerationParams()
    if eos_ids is None:
        eos_ids = getattr(getattr(engine, "model", None), "stop_token_ids", ())
    eos = set(int(t) for t in eos_ids)
    prompts = [list(p) for p in prompts]
    for i, p in enumerate(prompts):
        if not p:
            raise GenerationError("Empty prompt" if len(prompts) == 1 else "Empty prompt (request %d)" % i)
        if len(p) + max(0, params.max_tokens - 1) > engine.max_positions:
            raise GenerationError("request %d: %d prompt tokens and %d new ones exceed the model's %d positions"
                                  % (i, len(p), params.max_tokens, engine.max_positions))
    if make_sampler is None:
        from ..sampling.sampler import Sampler

        def make_sampler(p, request_ids):
            return Sampler(p, request_ids, engine.model.device)

    emitted = [[] for _ in prompts]
    max_batch = min(max_batch, getattr(engine, "max_slots", max_batch))
    for batch in plan_batches([len(p) for p in prompts], params.max_tokens, engine.max_tokens, max_batch,
                              holds_pages=getattr(engine, "holds_pages", True)):
        _run_batch(engine, prompts, batch, params, eos, emitted, on_tokens, make_sampler(params, batch),
                   max(1, int(max_step_tokens)))
    return emitted


def _prompt_steps(lens, max_step_tokens):
    """Cut prompts of the given lengths into steps of at most max_step_tokens tokens.
    Returns steps, each a list of (index, begin, end); a prompt's pieces come in order."""
    return native.prompt_steps(lens, max_step_tokens)


class _Known:
    """A draw whose tokens the host already has."""

    def __init__(self, tokens):
        self.tokens = list(tokens)

    def read(self):
        return self.tokens


def _run_batch(engine, prompts, batch, params, eos, emitted, on_tokens, sampler, max_step_tokens):
    """One batch from its prompts to its last token.

    Running ahead: if the engine takes a step's tokens from the device and the sampler can
    start a draw without waiting for it (`draw`, `pick`), the step after a draw is started
    before the draw has been read, for every request that goes on unless its unread token
    is a stop token; the host then reads the draw while the device works.  A request that
    did stop has run one step for nothing: its row of the next draw is dropped, and its
    slot goes back as it would have.  What is emitted is the same either way."""
    slots = {}
    borrow = {"borrow": True} if getattr(engine, "use_graphs", False) else {}
    ahead = bool(getattr(engine, "takes_device_tokens", False)) and hasattr(sampler, "draw") and hasattr(sampler, "pick")
    try:
        for r in batch:
            slots[r] = engine.open()
        drawn = {}
        for step in _prompt_steps([len(prompts[r]) for r in batch], max_step_tokens):
            items, ends = [], []
            for b, begin, end in step:
                r = batch[b]
                last = end == len(prompts[r])
                items.append((slots[r], prompts[r][begin:end], [end - begin - 1] if last else []))
                if last:
                    ends.append(b)
            logits = engine.step(items)
            if ends:
                drawn.update(zip(ends, sampler.sample(logits, ends)))
        rows = list(range(len(batch)))                 # indices into `batch` whose token is in `draw`
        draw = _Known([drawn[b] for b in rows])
        progress = native.BatchProgress(len(batch), params.max_tokens, eos)
        while rows:
            # the step after this draw, for those that go on if their unread token is no stop token
            next_rows, next_draw = [], None
            if ahead and not isinstance(draw, _Known):
                next_rows = [b for b in rows if progress.goes_on(b)]
                if next_rows:
                    tokens = sampler.pick(draw, [rows.index(b) for b in next_rows])
                    logits = engine.step([(slots[batch[b]], [0], [0]) for b in next_rows], device_tokens=tokens, **borrow)
                    next_draw = sampler.draw(logits, next_rows)
            feed, pairs = [], []
            for b, tok in zip(rows, draw.read()):
                what = progress.accept(b, tok)
                if what == native.TOKEN_DROPPED:        # it ended while a step with it was under way
                    continue
                r = batch[b]
                if what == native.TOKEN_STOP:
                    engine.close(slots.pop(r))          # stop tokens are not emitted (src/engine.rs:381)
                    continue
                emitted[r].append(tok)
                pairs.append((r, tok))
                if what == native.TOKEN_LAST:
                    engine.close(slots.pop(r))          # nothing more to draw for it
                    continue
                feed.append((b, tok))
            if on_tokens is not None and pairs:
                on_tokens(pairs)
            if next_draw is not None:
                rows, draw = next_rows, next_draw
                continue
            rows = [b for b, _ in feed]
            if not rows:
                break
            logits = engine.step([(slots[batch[b]], [tok], [0]) for b, tok in feed], **borrow)
            draw = sampler.draw(logits, rows) if ahead else _Known(sampler.sample(logits, rows))
    finally:
        for slot in slots.values():
            engine.close(slot)

"""The engine: a model, its cache, and the one step function everything above uses.

The reference's step is `forward(tokens, index_pos)` for one sequence with the last
row's logits (src/models/turbo_generic.rs:1950-1987) and its per-request state is one
position counter (src/engine.rs:117, :322-324).  Here a step takes a batch of
sequences with unequal numbers of new tokens (whole prompts, or one token each, or
anything between), runs exactly those tokens against what the cache holds, and
returns the logits at the wanted places.
"""
import numpy as np
import torch

from ..cache.store import Cache
from ..native import StepError
from ..tracing import span
from .context import HostStaging, StepContext


_NoUpload = object()       # StepContext(into=_NoUpload): build the host arrays only
_PRIMED = set()            # devices on which a captured graph has been launched once


def _prime_graph_launches(device):
    """The first launch of a captured graph in a process leaves the device slower for about a
    quarter of a second: measured at the Qwen2.5-7B sizes, every kernel of a decoding step then takes
    5 to 10 % longer (3.55 against 3.36 ms a step), whichever graph is launched and however many
    steps that is.  A graph of one small kernel, launched once when the first engine on a device is
    made, moves that quarter of a second to where no request waits for it."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key in _PRIMED:
        return
    with torch.cuda.device(key):
        x = torch.zeros(64, device="cuda")
        x.add_(1.0)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            x.add_(1.0)
        graph.replay()
        torch.cuda.synchronize()
    _PRIMED.add(key)


class Engine:
    """model: a loaded Model.  max_tokens: positions live sequences may hold together,
    each sequence counted up to a multiple of 64.  max_slots: most live sequences."""

    GRAPH_WIDTH_STEP = 8       # page-table widths of graphed steps grow in steps of 8 pages
    MAX_GRAPHS = 32
    takes_device_tokens = True

    def __init__(self, model, max_tokens, max_slots=256, use_graphs=True):
        self.model = model
        self.max_tokens = int(max_tokens)
        self.cache = Cache(model.needs, model.cache_of, self.max_tokens, max_slots, model.dtype, model.device)
        self.staging = HostStaging(model.device) if model.device.type == "cuda" else None
        self.holds_pages = self.cache.holds_pages       # False: no run keeps keys and values, max_tokens bounds nothing
        self.max_slots = self.cache.max_slots
        self.vocab_size = model.spec.vocab_size
        self.max_positions = model.spec.max_positions
        # Steps of one token per sequence are captured as HIP graphs and replayed: the step
        # is some hundred short kernels, and launching them one by one from the host would
        # cost more than running them.  Only if every part says its forward can be captured.
        self.use_graphs = bool(use_graphs) and model.device.type == "cuda" and model.graph_safe
        self.graphs = {}
        if self.use_graphs:
            _prime_graph_launches(model.device)

    # -- sequences --------------------------------------------------------
    def open(self):
        """Start a sequence: a slot of the cache with nothing in it."""
        return self.cache.acquire()

    def close(self, slot):
        """End a sequence: its slot and pages go back and will be used again."""
        self.cache.release(slot)

    def length(self, slot):
        return self.cache.length(slot)

    # -- the step ---------------------------------------------------------
    def step(self, items, borrow=False, device_tokens=None):
        """items: [(slot, tokens, want)].  tokens: the sequence's next tokens (at least one);
        want: indices among them whose logits are wanted (may be empty).  Returns float32
        logits [sum of len(want), vocab] in the order of items and of want.  borrow: the
        caller is done with the logits before the next step (they may live in a buffer that
        the next step writes again).  device_tokens: int32 [len(items)] on the device, for a
        step of one token per sequence whose tokens the host does not know yet (they were
        chosen on the device and must lie inside the vocabulary); the items' tokens are then
        placeholders."""
        if not items:
            raise StepError("a step needs at least one sequence")
        if device_tokens is not None:
            if any(len(tokens) != 1 for _, tokens, _ in items):
                raise StepError("tokens on the device stand for one token per sequence")
            if device_tokens.dtype != torch.int32 or tuple(device_tokens.shape) != (len(items),) \
                    or device_tokens.device.type != self.model.device.type:
                raise StepError("device_tokens must be int32 [%d] on %s" % (len(items), self.model.device))
        # the host library checks the rest: slots held and named once, no empty prompt, tokens inside the
        # vocabulary (where the host knows them), no sequence beyond the model's positions
        flat = None
        if device_tokens is None:                   # ids too large for the library's int32 stay too large for any vocabulary
            flat = np.asarray([t for _, tokens, _ in items for t in tokens], dtype=np.int64).clip(-1, 2 ** 31 - 1).astype(np.int32)
        self.cache.native.check_step(np.asarray([slot for slot, _, _ in items], dtype=np.int32),
                                     np.asarray([len(tokens) for _, tokens, _ in items], dtype=np.int32),
                                     flat, self.vocab_size, self.max_positions)
        with span("step"):
            return self._step(items, borrow, device_tokens)

    def _step(self, items, borrow, device_tokens):
        sizes = [(slot, len(tokens)) for slot, tokens, _ in items]
        self.cache.reserve(sizes)
        ctx_items = [(slot, self.cache.length(slot), tokens) for slot, tokens, _ in items]
        wants = [want for _, _, want in items]
        if self.use_graphs and all(n == 1 for _, n in sizes) and len(items) <= self.model.graph_max_rows:
            logits = self._graphed_step(ctx_items, wants, device_tokens)
            if not borrow:
                logits = logits.clone()
        else:
            ctx = StepContext(ctx_items, wants, self.cache, self.model.device, self.staging)
            if device_tokens is not None:
                ctx.dev.tokens.copy_(device_tokens)
            logits = self.model.forward(ctx, self.cache)
        self.cache.commit(sizes)
        return logits

    def _graphed_step(self, ctx_items, wants, device_tokens=None):
        """A step of one token per sequence through a captured graph.  The graph reads the
        step's arrays (tokens, positions, page tables) from one device buffer that is
        overwritten before every replay; its kernels take every size from those arrays or
        from the shapes the graph was captured for."""
        probe = StepContext(ctx_items, wants, self.cache, None, None, self.GRAPH_WIDTH_STEP, into=_NoUpload)
        key = probe.shape_key()
        entry = self.graphs.get(key)
        if entry is None:
            ctx = StepContext(ctx_items, wants, self.cache, self.model.device, self.staging, self.GRAPH_WIDTH_STEP)
            if device_tokens is not None:
                ctx.dev.tokens.copy_(device_tokens)
            logits = self.model.forward(ctx, self.cache)          # this step's work, and the warm-up
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_logits = self.model.forward(ctx, self.cache)
            if len(self.graphs) >= self.MAX_GRAPHS:
                self.graphs.pop(next(iter(self.graphs)))
            self.graphs[key] = (graph, ctx, static_logits)
            return logits
        graph, ctx, static_logits = entry
        self.graphs[key] = self.graphs.pop(key)                     # most recently used last
        self.staging.upload(probe.packed, into=ctx.flat)
        if device_tokens is not None:
            ctx.dev.tokens.copy_(device_tokens)
        graph.replay()
        return static_logits

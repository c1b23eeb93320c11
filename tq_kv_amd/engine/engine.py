"""The engine: a model, its cache, and the one step function everything above uses
(csrc/engine/engine.cpp behind tqe_engine_new / tqe_step; this class holds the handle).

The reference's step is `forward(tokens, index_pos)` for one sequence with the last row's
logits (src/models/turbo_generic.rs:1950-1987) and its per-request state is one position counter
(src/engine.rs:117, :322-324).  Here a step takes a batch of sequences with unequal numbers of new
tokens (whole prompts, or one token each, or anything between), runs exactly those tokens against
what the cache holds, and returns the logits at the wanted places.
"""
import ctypes

import numpy as np
import torch

from .. import native
from ..cache.store import Cache
from ..native import StepError


class Engine:
    """model: a loaded Model.  max_tokens: positions live sequences may hold together,
    each sequence counted up to a multiple of 64.  max_slots: most live sequences."""

    takes_device_tokens = True

    def __init__(self, model, max_tokens, max_slots=256, use_graphs=True):
        self._lib = native.library()
        self.model = model
        self.max_tokens = int(max_tokens)
        self.handle = native.handle(self._lib.tqe_engine_new(model.handle, self.max_tokens, int(max_slots), 1 if use_graphs else 0))
        self.cache = Cache.of_engine(self, model.needs, model.cache_of, model.dtype, model.device)
        info = self._describe()
        self.holds_pages = bool(info["holds_pages"])       # False: no run keeps keys and values, max_tokens bounds nothing
        self.max_slots = int(info["max_slots"])
        self.use_graphs = bool(info["use_graphs"])
        self.vocab_size = model.spec.vocab_size
        self.max_positions = model.spec.max_positions

    def _describe(self):
        return native.parsed(self._lib.tqe_engine_describe(self.handle))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            self.cache = None
            self._lib.tqe_engine_free(h)

    @property
    def graphs(self):
        """The steps captured as graphs so far (their number is what len() gives)."""
        return range(int(self._describe()["n_graphs"]))

    def _stream(self):
        return native.current_stream() if self.model.on_gpu else None

    # -- sequences --------------------------------------------------------
    def open(self):
        """Start a sequence: a slot of the cache with nothing in it."""
        slot = ctypes.c_int32(-1)
        native.check(self._lib.tqe_engine_open(self.handle, ctypes.byref(slot), self._stream()))
        return slot.value

    def close(self, slot):
        """End a sequence: its slot and pages go back and will be used again."""
        native.check(self._lib.tqe_engine_close(self.handle, int(slot)))

    def length(self, slot):
        return self.cache.length(slot)

    # -- the step ---------------------------------------------------------
    def step(self, items, borrow=False, device_tokens=None):
        """items: [(slot, tokens, want)].  tokens: the sequence's next tokens (at least one);
        want: indices among them whose logits are wanted (may be empty).  Returns float32
        logits [sum of len(want), vocab] in the order of items and of want.  borrow: the
        caller is done with the logits before the next step (they may live in memory that
        the next step writes again).  device_tokens: int32 [len(items)] on the device, for a
        step of one token per sequence whose tokens the host does not know yet (they were
        chosen on the device and must lie inside the vocabulary); the items' tokens are then
        placeholders."""
        if not items:
            raise StepError("a step needs at least one sequence")
        slots = np.asarray([slot for slot, _, _ in items], dtype=np.int32)
        n_new = np.asarray([len(tokens) for _, tokens, _ in items], dtype=np.int32)
        want_counts = np.asarray([len(want) for _, _, want in items], dtype=np.int32)
        want_idx = np.asarray([j for _, _, want in items for j in want], dtype=np.int64).clip(-1, 2 ** 31 - 1).astype(np.int32)
        flat, dev_ptr = None, None
        if device_tokens is not None:
            if device_tokens.dtype != torch.int32 or tuple(device_tokens.shape) != (len(items),) \
                    or device_tokens.device.type != self.model.device.type or not device_tokens.is_contiguous():
                raise StepError("device_tokens must be int32 [%d] on %s" % (len(items), self.model.device))
            dev_ptr = ctypes.c_void_p(device_tokens.data_ptr())
        else:                       # ids too large for the library's int32 stay too large for any vocabulary
            flat = np.asarray([t for _, tokens, _ in items for t in tokens], dtype=np.int64).clip(-1, 2 ** 31 - 1).astype(np.int32)
        n_want = int(want_counts.sum())
        kept = ctypes.c_void_p(0)
        logits = None
        if not borrow:
            logits = torch.empty((n_want, self.vocab_size), dtype=torch.float32, device=self.model.device)
        native.check(self._lib.tqe_step(self.handle, len(items), native._ptr(slots), native._ptr(n_new), native._ptr(flat),
                                        native._ptr(want_counts), native._ptr(want_idx), dev_ptr,
                                        ctypes.c_void_p(logits.data_ptr()) if logits is not None and n_want else None, 0,
                                        ctypes.byref(kept), self._stream()))
        if logits is not None:
            return logits
        return native.view(kept.value, native.F32, (n_want, self.vocab_size), self.model.on_gpu)

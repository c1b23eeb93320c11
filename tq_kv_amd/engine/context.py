"""The arrays of one step, for whoever wants to look at them or to call a single part.

A step runs the tokens it is given as one packed batch: the tokens of sequence 0, then of
sequence 1, and so on.  For each token the device knows which sequence of the step it belongs to
and its absolute position; for each sequence its slot, how many positions the cache held before
the step and how many tokens it brings; for each cache group the page table of the step's
sequences.  All of it is laid out by the engine library (tqe_plan_step) as one int32 array; the
engine builds and uploads it inside tqe_step.  This class shows the same arrays to Python: on
the host always, and on the device (a tqe_stepctx_t) where a part is to be called with them.
"""
import numpy as np

from .. import native

_NAMES = list(native.STEP_ARRAYS)


class _Arrays:
    pass


class StepContext:
    """items: [(slot, start, tokens)] with `start` the sequence's length before the step;
    want: for each item the indices among its tokens whose logits are wanted.  device None (or
    into given and no tensor): the host arrays only."""

    def __init__(self, items, want, cache, device, staging=None, width_step=1, into=None):
        self.n_seqs = len(items)
        lens = [len(toks) for _, _, toks in items]
        slots = np.asarray([slot for slot, _, _ in items], dtype=np.int32)
        starts = np.asarray([start for _, start, _ in items], dtype=np.int32)
        n_new = np.asarray(lens, dtype=np.int32)
        tokens = np.concatenate([np.asarray(toks, dtype=np.int64) for _, _, toks in items]).astype(np.int32)
        want_counts = np.asarray([len(w) for w in want], dtype=np.int32)
        want_idx = np.asarray([j for w in want for j in w], dtype=np.int64).astype(np.int32)
        self.groups = list(cache.kv_groups) if cache is not None else []
        packed, meta = native.plan_step(cache.native if cache is not None else None, slots, starts, n_new, tokens,
                                        want_counts, want_idx, width_step)
        self.packed = packed
        self.n_tokens = int(meta[native.META_TOKENS])
        self.n_last = int(meta[native.META_LAST])
        self.all_decode = bool(meta[native.META_ALL_DECODE])
        self.prune_last = bool(meta[native.META_PRUNE_LAST])
        self.max_new = int(meta[native.META_MAX_NEW])
        self.max_end = int(meta[native.META_MAX_END])
        offsets = [int(o) for o in meta[native.META_OFFSETS:native.META_OFFSETS + 12 + len(self.groups)]]
        widths = [int(x) for x in meta[native.META_WIDTHS:native.META_WIDTHS + len(self.groups)]]
        n_want = int(meta[native.META_WANT])
        kept = self.n_last if self.prune_last else 0
        sizes = [self.n_tokens] * 3 + [self.n_seqs] * 3 + [self.n_seqs + 1, n_want, kept, n_want if self.prune_last else 0, kept, kept]
        self._table_shapes = [(self.n_seqs, w) for w in widths]
        self.host = _Arrays()
        for name, off, size in zip(_NAMES, offsets, sizes):
            setattr(self.host, name, packed[off:off + size])
        self.host_tables = [packed[off:off + n * w].reshape(n, w) for off, (n, w) in zip(offsets[12:], self._table_shapes)]
        self.handle = None
        self.dev = None
        if device is None or (into is not None and not hasattr(into, "data_ptr")):
            return                                   # host arrays only
        import torch
        if torch.device(device).type != "cuda" or cache is None or cache.handle is None:
            return
        self._lib = native.library()
        self._cache = cache
        self.handle = native.handle(self._lib.tqe_stepctx_new(
            cache.handle, self.n_seqs, native._ptr(slots), native._ptr(n_new), native._ptr(tokens), native._ptr(want_counts),
            native._ptr(want_idx), native.dtype_code(cache.kv_groups[0].keys.dtype) if cache.kv_groups else native.F32,
            native.current_stream()))
        view = native.tqe_step_view()
        native.check(self._lib.tqe_stepctx_view(self.handle, view))
        from ..parts.registry import StepView
        self.dev = StepView(view, True).dev

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            self._lib.tqe_stepctx_free(h)

    def shape_key(self):
        """What fixes the layout of the device arrays (and so what a captured graph of the
        step depends on): numbers of tokens, sequences and wanted rows, table widths."""
        return (self.n_tokens, self.n_seqs, int(self.host.want_rows.shape[0]), tuple(w for _, w in self._table_shapes))

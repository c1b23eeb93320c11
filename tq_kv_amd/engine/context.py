"""What one step knows about its batch, on the host and on the device.

A step runs the tokens it is given as one packed batch: the tokens of sequence 0,
then of sequence 1, and so on.  For each token the device knows which sequence of
the step it belongs to and its absolute position; for each sequence its slot, how
many positions the cache held before the step and how many tokens it brings; for
each cache group the page table of the step's sequences.  All of it is built on the
host as one int32 array and uploaded in one copy.
"""
import numpy as np
import torch

from .. import native


class _Arrays:
    pass


class HostStaging:
    """Pinned host buffers for small uploads, used in turn; a buffer is written again only
    after the copy that last read it has finished."""

    def __init__(self, device, depth=2):
        self.device = device
        self.bufs = [None] * depth
        self.events = [None] * depth
        self.turn = 0

    def upload(self, packed, into=None):
        """Copy a one-dimensional int32 or float32 array to the device without waiting for
        the device: into `into` (a device buffer of the same size and kind, for instance one
        that a captured graph reads) or into a new tensor."""
        n = packed.shape[0]
        kind = torch.float32 if packed.dtype == np.float32 else torch.int32
        if kind == torch.int32 and packed.dtype != np.int32:
            raise TypeError("uploads are int32 or float32, got %s" % packed.dtype)
        i = self.turn
        self.turn = (i + 1) % len(self.bufs)
        if self.events[i] is not None:
            self.events[i].synchronize()
        if self.bufs[i] is None or self.bufs[i].shape[0] < n:
            self.bufs[i] = torch.empty(max(4096, 2 * n), dtype=torch.int32, pin_memory=True)
        host = self.bufs[i][:n].view(kind)
        host.numpy()[:] = packed
        dev = into if into is not None else torch.empty(n, dtype=kind, device=self.device)
        if dev.shape[0] != n or dev.dtype != kind:
            raise ValueError("the upload is %d values of %s, the buffer holds %d of %s" % (n, kind, dev.shape[0], dev.dtype))
        dev.copy_(host, non_blocking=True)
        self.events[i] = torch.cuda.Event()
        self.events[i].record()
        return dev


_NAMES = ["tokens", "tok_seq", "tok_pos", "seq_slot", "seq_start", "seq_new", "cu", "want_rows",
          "last_rows", "want_in_last", "last_seq", "last_pos"]


class StepContext:
    """items: [(slot, start, tokens)] with `start` the sequence's length before the step;
    want: for each item the indices among its tokens whose logits are wanted.

    The arrays are laid out by the engine's host library (tqe_plan_step): the wanted rows, the
    rows that the last run of the order has to compute (the wanted ones, each once, in order:
    where these are fewer than the step's tokens, a prompt of which the last place is wanted or a
    piece of a prompt of which nothing is, the last run computes its queries, its output product
    and its feed-forward for them alone), and the page tables of the step's sequences."""

    def __init__(self, items, want, cache, device, staging=None, width_step=1, into=None):
        self.n_seqs = len(items)
        lens = [len(toks) for _, _, toks in items]
        slots = np.asarray([slot for slot, _, _ in items], dtype=np.int32)
        starts = np.asarray([start for _, start, _ in items], dtype=np.int32)
        n_new = np.asarray(lens, dtype=np.int32)
        if len(items) == 1:
            tokens = np.asarray(items[0][2], dtype=np.int64).astype(np.int32)
        else:
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

        def carve(flat, make=lambda x: x):
            out = _Arrays()
            for name, off, size in zip(_NAMES, offsets, sizes):
                setattr(out, name, make(flat[off:off + size]))
            return out
        self.host = carve(packed)
        self.host_tables = [packed[off:off + n * w].reshape(n, w) for off, (n, w) in zip(offsets[12:], self._table_shapes)]
        self._lens = lens
        self._tiles = {}              # (which rows, queries per tile) -> device arrays, built when a mixer asks
        self.fuse_small = False       # set by the model for small decoding steps in bfloat16
        self._device, self._staging = device, staging
        if into is not None and not isinstance(into, torch.Tensor):
            return                                   # host arrays only
        if staging is not None:
            flat = staging.upload(packed, into)
        elif into is not None:
            flat = into.copy_(torch.from_numpy(packed))
        else:
            flat = torch.from_numpy(packed).to(device)
        self.flat = flat
        self.dev = carve(flat)
        self._tables = {}
        for g, off, (n, w) in zip(self.groups, offsets[12:], self._table_shapes):
            self._tables[id(g)] = flat[off:off + n * w].view(n, w)

    # -- tiles of consecutive queries, for mixers that work on them -----------------------------
    def _upload_tiles(self, key, seq, tok0, count, order_key):
        order = sorted(range(len(seq)), key=order_key)          # longest first: a tile's work grows with its last position
        packed = np.asarray([seq[k] for k in order] + [tok0[k] for k in order] + [count[k] for k in order], dtype=np.int32)
        n = len(order)
        if n == 0:
            flat = torch.zeros(0, dtype=torch.int32, device=self._device)
        elif self._staging is not None:
            flat = self._staging.upload(packed)
        else:
            flat = torch.from_numpy(packed).to(self._device)
        self._tiles[key] = (flat[:n], flat[n:2 * n], flat[2 * n:3 * n])
        return self._tiles[key]

    def query_tiles(self, tile):
        """The step's tokens cut into tiles of up to `tile` consecutive queries of one sequence:
        (sequence of the step, first packed token, number of queries) per tile, int32 on the
        device, longest reach first.  Built and uploaded when a mixer first asks for this size."""
        key = ("all", int(tile))
        if key in self._tiles:
            return self._tiles[key]
        cu, pos = self.host.cu, self.host.tok_pos
        seq, tok0, count = [], [], []
        for i, n in enumerate(self._lens):
            for a in range(0, n, tile):
                seq.append(i), tok0.append(int(cu[i]) + a), count.append(min(tile, n - a))
        return self._upload_tiles(key, seq, tok0, count, lambda k: -(int(pos[tok0[k]]) + count[k]))

    def last_tiles(self, tile):
        """The same for the step's last_rows, in their own numbering: runs of neighbouring rows of
        one sequence, up to `tile` each."""
        key = ("last", int(tile))
        if key in self._tiles:
            return self._tiles[key]
        h = self.host
        seq, tok0, count = [], [], []
        k = 0
        while self.prune_last and k < self.n_last:
            j = k + 1
            while (j < self.n_last and j - k < tile and h.last_rows[j] == h.last_rows[j - 1] + 1
                   and h.last_seq[j] == h.last_seq[k]):
                j += 1
            seq.append(int(h.last_seq[k])), tok0.append(k), count.append(j - k)
            k = j
        return self._upload_tiles(key, seq, tok0, count, lambda t: -(int(h.last_pos[tok0[t]]) + count[t]))

    def shape_key(self):
        """What fixes the layout of the device arrays (and so what a captured graph of the
        step depends on): numbers of tokens, sequences and wanted rows, table widths."""
        return (self.n_tokens, self.n_seqs, int(self.host.want_rows.shape[0]), tuple(w for _, w in self._table_shapes))

    def page_table(self, group):
        """[sequences of the step, width] int32 page ids of a cache group, on the device."""
        return self._tables[id(group)]

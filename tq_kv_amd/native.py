"""Python face of the engine's host library (csrc/host_engine.cpp, csrc/tq_engine.h): slots,
page lists and the arrays of a step live behind C handles; the classes here hold a handle
and turn status codes into exceptions.  The library has no GPU code and is built with the
host compiler at first use."""
import ctypes

import numpy as np

from .cache.pages import CacheFull
from .csrc import build as _build

_LIB = None
OK, ERR_ARGUMENT, ERR_FULL, ERR_STATE, ERR_RANGE, ERR_STEP, NO_LIST = 0, -1, -2, -3, -4, -5, -100
MAX_GROUPS = 16
META_SIZE = 12 + 12 + 2 * MAX_GROUPS
(META_TOTAL, META_TOKENS, META_WANT, META_LAST, META_ALL_DECODE, META_PRUNE_LAST, META_MAX_NEW, META_MAX_END,
 META_GROUPS) = range(9)
META_OFFSETS = 12
META_WIDTHS = META_OFFSETS + 12 + MAX_GROUPS
_I32P = ctypes.POINTER(ctypes.c_int32)


class EngineLibraryError(RuntimeError):
    pass


class StepError(ValueError):
    """A step the engine cannot run (no sequence, a slot twice, an empty prompt, a token outside
    the vocabulary, more positions than the model has)."""


def library():
    global _LIB
    if _LIB is None:
        path = _build.ensure_host_built()
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise EngineLibraryError("cannot load the engine's host library %s: %s" % (path, e))
        lib.tqe_last_error.restype = ctypes.c_char_p
        lib.tqe_cache_new.restype = ctypes.c_void_p
        lib.tqe_cache_new.argtypes = [ctypes.c_int, ctypes.c_int, _I32P, _I32P]
        lib.tqe_cache_free.argtypes = [ctypes.c_void_p]
        lib.tqe_cache_free.restype = None
        for name, args in (("tqe_cache_acquire", [ctypes.c_void_p, _I32P]), ("tqe_cache_release", [ctypes.c_void_p, ctypes.c_int]),
                           ("tqe_cache_length", [ctypes.c_void_p, ctypes.c_int]), ("tqe_cache_is_held", [ctypes.c_void_p, ctypes.c_int]),
                           ("tqe_cache_counts", [ctypes.c_void_p, ctypes.c_int, _I32P, _I32P]),
                           ("tqe_cache_reserve", [ctypes.c_void_p, ctypes.c_int, _I32P, _I32P]),
                           ("tqe_cache_commit", [ctypes.c_void_p, ctypes.c_int, _I32P, _I32P]),
                           ("tqe_cache_pages", [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, _I32P, ctypes.c_int]),
                           ("tqe_cache_check", [ctypes.c_void_p]),
                           ("tqe_check_step", [ctypes.c_void_p, ctypes.c_int, _I32P, _I32P, _I32P, ctypes.c_int, ctypes.c_int]),
                           ("tqe_plan_step", [ctypes.c_void_p, ctypes.c_int, _I32P, _I32P, _I32P, _I32P, _I32P, _I32P, ctypes.c_int,
                                              _I32P, ctypes.c_int, _I32P]),
                           ("tqe_plan_batches", [ctypes.c_int, _I32P, ctypes.c_int, ctypes.c_longlong, ctypes.c_int, ctypes.c_int, _I32P]),
                           ("tqe_prompt_steps", [ctypes.c_int, _I32P, ctypes.c_int, _I32P, ctypes.c_int]),
                           ("tqe_batch_accept", [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]),
                           ("tqe_batch_goes_on", [ctypes.c_void_p, ctypes.c_int]),
                           ("tqe_batch_emitted", [ctypes.c_void_p, ctypes.c_int]),
                           ("tqe_batch_ended", [ctypes.c_void_p, ctypes.c_int])):
            getattr(lib, name).argtypes = args
            getattr(lib, name).restype = ctypes.c_int
        lib.tqe_batch_new.restype = ctypes.c_void_p
        lib.tqe_batch_new.argtypes = [ctypes.c_int, ctypes.c_int, _I32P, ctypes.c_int]
        lib.tqe_batch_free.argtypes = [ctypes.c_void_p]
        lib.tqe_batch_free.restype = None
        _LIB = lib
    return _LIB


def library_path():
    library()
    return _LIB._name


def _message():
    return library().tqe_last_error().decode("utf-8", "replace")


def _raise(status):
    """The exception of a status code: a full cache, a broken invariant (AssertionError, as the
    bookkeeping's own checks are), a wanted place out of range, anything else."""
    msg = _message()
    if status == ERR_FULL:
        raise CacheFull(msg)
    if status == ERR_STATE:
        raise AssertionError(msg)
    if status == ERR_RANGE:
        raise IndexError(msg)
    if status == ERR_STEP:
        raise StepError(msg)
    raise EngineLibraryError(msg)


def _ptr(a):
    return a.ctypes.data_as(_I32P) if a is not None else None


def _i32(values):
    return np.ascontiguousarray(values, dtype=np.int32)


class NativeCache:
    """A tqe_cache_t: max_slots slots, one page pool per group (pages, window or 0)."""

    def __init__(self, max_slots, groups):
        pages = _i32([p for p, _ in groups])
        windows = _i32([w or 0 for _, w in groups])
        self.n_groups = len(groups)
        self.max_slots = int(max_slots)
        self._lib = library()
        self.handle = self._lib.tqe_cache_new(self.max_slots, self.n_groups, _ptr(pages), _ptr(windows))
        if not self.handle:
            raise EngineLibraryError(_message())

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle and self._lib is not None:
            self._lib.tqe_cache_free(handle)

    def acquire(self):
        slot = ctypes.c_int32(-1)
        status = self._lib.tqe_cache_acquire(self.handle, ctypes.byref(slot))
        if status != OK:
            _raise(status)
        return slot.value

    def release(self, slot):
        status = self._lib.tqe_cache_release(self.handle, int(slot))
        if status != OK:
            _raise(status)

    def length(self, slot):
        n = self._lib.tqe_cache_length(self.handle, int(slot))
        if n < 0:
            _raise(n)
        return n

    def is_held(self, slot):
        return bool(self._lib.tqe_cache_is_held(self.handle, int(slot)))

    def counts(self, group):
        """(free, total) slots (group -1) or pages of a group."""
        free, total = ctypes.c_int32(0), ctypes.c_int32(0)
        status = self._lib.tqe_cache_counts(self.handle, int(group), ctypes.byref(free), ctypes.byref(total))
        if status != OK:
            _raise(status)
        return free.value, total.value

    def _items(self, items):
        return _i32([s for s, _ in items]), _i32([n for _, n in items])

    def reserve(self, items):
        slots, counts = self._items(items)
        status = self._lib.tqe_cache_reserve(self.handle, len(items), _ptr(slots), _ptr(counts))
        if status != OK:
            _raise(status)

    def commit(self, items):
        slots, counts = self._items(items)
        status = self._lib.tqe_cache_commit(self.handle, len(items), _ptr(slots), _ptr(counts))
        if status != OK:
            _raise(status)

    def pages(self, group, slot):
        """The slot's page list in the group (-1 where given back), or None if it has none."""
        n = self._lib.tqe_cache_pages(self.handle, int(group), int(slot), None, 0)
        if n == NO_LIST:
            return None
        if n < 0:
            _raise(n)
        out = np.empty(max(n, 1), dtype=np.int32)
        self._lib.tqe_cache_pages(self.handle, int(group), int(slot), _ptr(out), n)
        return out[:n].tolist()

    def check(self):
        status = self._lib.tqe_cache_check(self.handle)
        if status != OK:
            _raise(status)

    def check_step(self, slots, n_new, tokens, vocab_size, max_positions):
        """Raises StepError unless the step can run (tqe_check_step).  tokens: int32 array of all the
        step's tokens, or None where the host does not know them."""
        status = self._lib.tqe_check_step(self.handle, len(slots), _ptr(slots), _ptr(n_new), _ptr(tokens), int(vocab_size), int(max_positions))
        if status != OK:
            _raise(status)


def plan_step(cache, slots, starts, n_new, tokens, want_counts, want_idx, width_step, out=None):
    """The packed arrays of one step (tqe_plan_step).  cache: a NativeCache or None (then starts
    must be given).  out: an int32 numpy array to fill (grown copies are the caller's business), or
    None for a new one.  Returns (packed array, meta array)."""
    lib = library()
    handle = cache.handle if cache is not None else None
    n = len(slots)
    meta = np.zeros(META_SIZE, dtype=np.int32)
    args = (handle, n, _ptr(slots), _ptr(starts), _ptr(n_new), _ptr(tokens), _ptr(want_counts), _ptr(want_idx), int(width_step))
    if out is None:
        status = lib.tqe_plan_step(*args, None, 0, _ptr(meta))
        if status != OK:
            _raise(status)
        out = np.empty(int(meta[META_TOTAL]), dtype=np.int32)
    status = lib.tqe_plan_step(*args, _ptr(out), out.shape[0], _ptr(meta))
    if status != OK:
        _raise(status)
    return out[:int(meta[META_TOTAL])], meta


# ---- the generation loop's decisions ----------------------------------------------------------
TOKEN_FEED, TOKEN_LAST, TOKEN_STOP, TOKEN_DROPPED = 0, 1, 2, 3


def plan_batches(prompt_lens, max_new, max_tokens, max_batch, holds_pages=True):
    """tqe_plan_batches: lists of request indices, one list per batch.  CacheFull where one request
    alone does not fit."""
    lens = np.ascontiguousarray(prompt_lens, dtype=np.int32)
    batch_of = np.zeros(len(lens), dtype=np.int32)
    n = library().tqe_plan_batches(len(lens), _ptr(lens), int(max_new), int(max_tokens), int(max_batch), 1 if holds_pages else 0,
                                   _ptr(batch_of))
    if n < 0:
        _raise(n)
    batches = [[] for _ in range(n)]
    for i, b in enumerate(batch_of.tolist()):
        batches[b].append(i)
    return batches


def prompt_steps(lens, max_step_tokens):
    """tqe_prompt_steps: steps, each a list of (prompt, begin, end)."""
    lens = np.ascontiguousarray(lens, dtype=np.int32)
    n = library().tqe_prompt_steps(len(lens), _ptr(lens), int(max_step_tokens), None, 0)
    if n < 0:
        _raise(n)
    pieces = np.zeros((max(n, 1), 4), dtype=np.int32)
    n = library().tqe_prompt_steps(len(lens), _ptr(lens), int(max_step_tokens), _ptr(pieces), len(pieces))
    if n < 0:
        _raise(n)
    steps = []
    for i, begin, end, step in pieces[:n].tolist():
        while len(steps) <= step:
            steps.append([])
        steps[step].append((i, begin, end))
    return steps


class BatchProgress:
    """tqe_batch_t: how many tokens each request of a batch has emitted, which have ended, and
    what becomes of a drawn token."""

    def __init__(self, n_requests, max_new, stop_ids):
        stop = np.ascontiguousarray(sorted(set(int(t) for t in stop_ids if -2 ** 31 <= int(t) < 2 ** 31)), dtype=np.int32)
        self._lib = library()
        self.handle = self._lib.tqe_batch_new(int(n_requests), int(max_new), _ptr(stop) if len(stop) else None, len(stop))
        if not self.handle:
            raise EngineLibraryError(_message())

    def __del__(self):
        if getattr(self, "handle", None):
            self._lib.tqe_batch_free(self.handle)
            self.handle = None

    def accept(self, row, token):
        token = int(token)
        if not -2 ** 31 <= token < 2 ** 31:
            token = -1                       # no stop id is outside the library's int32
        status = self._lib.tqe_batch_accept(self.handle, int(row), token)
        if status < 0:
            _raise(status)
        return status

    def goes_on(self, row):
        return bool(self._lib.tqe_batch_goes_on(self.handle, int(row)))

    def emitted(self, row):
        n = self._lib.tqe_batch_emitted(self.handle, int(row))
        if n < 0:
            _raise(n)
        return n

    def ended(self, row):
        return bool(self._lib.tqe_batch_ended(self.handle, int(row)))

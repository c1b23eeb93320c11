"""Kinds of parts, and parts one by one.

The parts a layer is put together from (norm, position, mixer, feed_forward, block) are built
by the engine library from a PartSpec (kind + parameters).  Its own kinds are C++ classes
(csrc/engine/parts_builtin.cpp).  A kind can also be written in Python: a class with
`@register(category, kind)` is handed to the library as a table of callbacks, and the library
then builds, loads and calls it like any other part, inside any model, with tensors that are
views of the engine's memory.  What such a class offers:

  every part    __init__(params, env);  tensors() -> {name: TensorSpec};  load(tensors)
  norm          forward(x) -> y;  add_norm(h, delta) -> y  (h += delta in place, then norm of h);
                gather_add_norm(h, delta, rows) -> y for chosen rows only (h is left as it is)
  position      apply(q, k, ctx) changes q [tokens, heads, d] and k in place; or, for one that acts on
                the stream after the gather, add_to_stream(h, ctx);  max_positions
  mixer         cache_need() -> KVNeed | StateNeed | None;  forward(x, ctx, cache_entry) -> y
  feed_forward  forward(x, ctx) -> y

ctx is the step (n_seqs, n_tokens, host.<array> numpy, dev.<array> torch, page_table(group)); a
cache entry has keys and values (pages) or state (rows per slot), `group` and `writes`.  Parts
written in Python run as they come, never inside a captured graph.

`BuildEnv.build(category, spec)` gives a part alone (any kind), with its methods taking and
returning torch tensors: what the tests of single parts use.
"""
import ctypes
import json

from .. import native
from .spec import PartSpec, TensorSpec, need_from_json, need_to_json

CATEGORIES = ("norm", "position", "mixer", "feed_forward", "block")
_PYTHON_KINDS = {}          # (category, kind) -> (class, callbacks struct, kept alive)
_INSTANCES = {}             # handle -> _Instance
_NEXT = [1]
_LAST_ERROR = native.CString()


class Part:
    """Base of every part written in Python."""
    category = None
    kind = None

    def tensors(self):
        """name (relative to the part's prefix) -> TensorSpec"""
        return {}

    def load(self, tensors):
        """Take the loaded tensors (same names as tensors())."""

    def cache_need(self):
        return None


class _Env:
    """What a part written in Python is told of the run."""

    def __init__(self, act_dtype, on_gpu):
        import torch
        self.act_dtype = native.torch_dtype(act_dtype)
        self.device = torch.device("cuda" if on_gpu else "cpu")
        self.on_gpu = bool(on_gpu)


class _Arrays:
    pass


class StepView:
    """The step as a part written in Python sees it."""

    def __init__(self, view, on_gpu):
        import numpy as np
        for name in ("n_seqs", "n_tokens", "n_want", "n_last", "max_new", "max_end"):
            setattr(self, name, int(getattr(view, name)))
        self.all_decode, self.prune_last = bool(view.all_decode), bool(view.prune_last)
        self.host, self.dev = _Arrays(), _Arrays()
        for i, name in enumerate(native.STEP_ARRAYS):
            n = int(view.sizes[i])
            setattr(self.host, name, np.ctypeslib.as_array(view.host[i], shape=(n,)) if n and view.host[i] else np.zeros(0, dtype=np.int32))
            setattr(self.dev, name, native.view(view.dev[i], native.I32, (n,), on_gpu))
        self._tables = []
        for g in range(int(view.n_groups)):
            self._tables.append(native.view(view.table_dev[g], native.I32, (self.n_seqs, int(view.table_width[g])), on_gpu))
        self.stream = view.stream

    def page_table(self, group):
        """[sequences of the step, width] int32 page ids of a cache group (an entry's `group`), on the device."""
        return self._tables[group if isinstance(group, int) else group.index]


class _Entry:
    """What a mixer written in Python sees of the cache."""

    def __init__(self, tensors, view):
        self.group = int(view.entry_group)
        self.writes = bool(view.entry_writes)
        self.window = int(view.entry_window) or None
        self.keys = self.values = self.state = None
        if len(tensors) == 2:
            self.keys, self.values = tensors
        elif len(tensors) == 1:
            self.state = tensors[0]


class _Instance:
    def __init__(self, part, category, env):
        self.part, self.category, self.env = part, category, env
        self.text = b""


def _guard(fn):
    """A callback must not let an exception escape into the library: it is kept, the status says
    'failed', and it is raised again (the original) once the library has returned."""
    def wrapped(*args):
        try:
            return fn(*args)
        except BaseException as e:          # noqa: B902
            native._pending_exception.append(e)
            _LAST_ERROR.set(("%s: %s" % (type(e).__name__, e)).encode("utf-8", "replace"))
            return native.ERR_PART
    return wrapped


def _stream_scope(view, on_gpu):
    import contextlib

    import torch
    if not on_gpu or view is None or not view.contents.stream:
        return contextlib.nullcontext()
    ptr = int(view.contents.stream)
    if ptr == torch.cuda.current_stream().cuda_stream:
        return contextlib.nullcontext()
    return torch.cuda.stream(torch.cuda.ExternalStream(ptr))


def _make_callbacks(cls):
    @_guard
    def create(user, category, kind, params_json, act_dtype, on_gpu, out):
        params = PartSpec.from_json({"kind": kind.decode(), "params": json.loads(params_json.decode())}).params
        env = _Env(act_dtype, on_gpu)
        part = cls(dict(params), env)
        h = _NEXT[0]
        _NEXT[0] += 1
        _INSTANCES[h] = _Instance(part, category.decode(), env)
        out[0] = h
        return 0

    def destroy(user, h):
        _INSTANCES.pop(h, None)

    def describe(user, h):
        try:
            inst = _INSTANCES[h]
            p = inst.part
            info = {"tensors": {n: s.to_json() for n, s in p.tensors().items()},
                    "cache_need": need_to_json(p.cache_need()) if hasattr(p, "cache_need") else None,
                    "graph_safe": False, "has_apply": hasattr(p, "apply"), "acts_on_stream": hasattr(p, "add_to_stream"),
                    "trace_name": getattr(p, "trace_name", "part")}
            if hasattr(p, "max_positions"):
                info["max_positions"] = int(p.max_positions)
            inst.text = native.CString(json.dumps(info))
            return inst.text.address
        except BaseException as e:          # noqa: B902
            native._pending_exception.append(e)
            _LAST_ERROR.set(("%s: %s" % (type(e).__name__, e)).encode("utf-8", "replace"))
            return None

    @_guard
    def load(user, h, n, names, tensors):
        inst = _INSTANCES[h]
        given = {names[i].decode(): native.view_of(tensors[i], inst.env.on_gpu) for i in range(n)}
        inst.part.load(given)
        return 0

    @_guard
    def call(user, h, method, view, n_args, args):
        inst = _INSTANCES[h]
        p, on_gpu = inst.part, inst.env.on_gpu
        method = method.decode()
        t = [native.view_of(args[i], on_gpu) for i in range(n_args)]
        ctx = StepView(view.contents, on_gpu) if view else None
        with _stream_scope(view, on_gpu):
            if inst.category == "norm":
                if method == "forward":
                    t[1].copy_(p.forward(t[0]))
                elif method == "add_norm":
                    t[2].copy_(p.add_norm(t[0], t[1]))
                elif method == "gather_add_norm":
                    t[3].copy_(p.gather_add_norm(t[0], t[1], t[2]))
                else:
                    raise ValueError("a norm has no method %r" % method)
            elif inst.category == "position":
                if method == "apply":
                    p.apply(t[0], t[1], ctx)
                elif method == "add_to_stream":
                    p.add_to_stream(t[0], ctx)
                else:
                    raise ValueError("a position has no method %r" % method)
            elif inst.category == "mixer":
                entry = _Entry(t[2:], view.contents)
                if view.contents.last_rows_only:
                    t[1].copy_(p.forward(t[0], ctx, entry, last_rows=True))
                else:
                    t[1].copy_(p.forward(t[0], ctx, entry))
            elif inst.category == "feed_forward":
                t[1].copy_(p.forward(t[0], ctx))
            else:
                raise ValueError("parts of category %r cannot be written in Python" % inst.category)
        return 0

    def last_error(user):
        return _LAST_ERROR.address

    cb = native.tqe_part_callbacks(native.PART_CREATE(create), native.PART_DESTROY(destroy), native.PART_DESCRIBE(describe),
                                   native.PART_LOAD(load), native.PART_CALL(call), native.PART_ERROR(last_error))
    return cb


def register(category, kind):
    """Class decorator: make `kind` buildable in `category` (norm, position, mixer, feed_forward)."""
    if category not in CATEGORIES:
        raise KeyError("unknown part category '%s' (known: %s)" % (category, ", ".join(CATEGORIES)))

    def deco(cls):
        cb = _make_callbacks(cls)
        native.check(native.library().tqe_register_part(native.enc(category), native.enc(kind), ctypes.byref(cb), None))
        _PYTHON_KINDS[(category, kind)] = (cls, cb)         # the callbacks live as long as the process
        cls.category = category
        cls.kind = kind
        return cls
    return deco


def known(category):
    return native.parsed(native.library().tqe_known_parts(native.enc(category)))


# ---- parts one by one -----------------------------------------------------------------------------------
class PartHandle:
    """A part of the engine library's, alone: built from a PartSpec, loaded with tensors, its
    methods taking and returning torch tensors on the part's device."""

    def __init__(self, category, spec, act_dtype, on_gpu):
        self._lib = native.library()
        self.category, self.kind = category, spec.kind
        self.on_gpu = bool(on_gpu)
        self.act_dtype = native.torch_dtype(act_dtype)
        self._code = act_dtype
        self.handle = native.handle(self._lib.tqe_part_new(native.enc(category), native.enc(json.dumps(spec.to_json())), act_dtype,
                                                           1 if on_gpu else 0))
        self.info = native.parsed(self._lib.tqe_part_describe(self.handle))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            self._lib.tqe_part_free(h)

    def tensors(self):
        return {n: TensorSpec.from_json(s) for n, s in self.info["tensors"].items()}

    def load(self, tensors):
        stream = native.current_stream() if self.on_gpu else None
        for name in self.tensors():
            t = tensors[name].contiguous()
            ct = native.c_tensor(t)
            native.check(self._lib.tqe_part_set_tensor(self.handle, native.enc(name), ctypes.byref(ct), 1 if t.is_cuda else 0, stream))
        native.check(self._lib.tqe_part_finish(self.handle, stream))
        self.info = native.parsed(self._lib.tqe_part_describe(self.handle))

    def tensor(self, name):
        ct = native.tqe_tensor()
        native.check(self._lib.tqe_part_tensor(self.handle, native.enc(name), ctypes.byref(ct)))
        return native.view_of(ct, self.on_gpu, keep=self)

    def cache_need(self):
        return need_from_json(self.info.get("cache_need"))

    @property
    def graph_safe(self):
        return bool(self.info.get("graph_safe"))

    def _call(self, method, args, ctx=None, cache=None, run=0):
        import torch
        arr = (native.tqe_tensor * len(args))(*[native.c_tensor(a) for a in args])
        stream = native.current_stream() if self.on_gpu else None
        native.check(self._lib.tqe_part_call(self.handle, native.enc(method), ctx.handle if ctx is not None else None,
                                             cache.handle if cache is not None else None, int(run), len(args), arr, stream))
        if self.on_gpu:
            torch.cuda.current_stream().synchronize()      # the part's scratch memory is gone when the call returns

    # -- norm ---------------------------------------------------------------------------------------------
    def forward(self, x, ctx=None, entry=None):
        import torch
        if self.category == "norm":
            out = torch.empty_like(x)
            self._call("forward", [x, out])
            return out
        if self.category == "feed_forward":
            out = torch.empty_like(x)
            self._call("forward", [x, out])
            return out
        if self.category == "mixer":
            out = torch.empty_like(x)
            self._call("forward", [x, out], ctx=ctx, cache=entry.cache, run=entry.run)
            return out
        raise TypeError("a %s has no forward" % self.category)

    def add_norm(self, h, delta):
        import torch
        out = torch.empty(h.shape, dtype=self.act_dtype, device=h.device)
        self._call("add_norm", [h, delta, out])
        return out

    def gather_add_norm(self, h, delta, rows):
        import torch
        out = torch.empty((rows.shape[0], h.shape[1]), dtype=self.act_dtype, device=h.device)
        self._call("gather_add_norm", [h, delta, rows, out])
        return out

    # -- position -------------------------------------------------------------------------------------------
    def tables(self):
        """(cos, sin, rot_dim, style) of a position kind with rotary tables."""
        if not self.info.get("rot_dim"):
            return None, None, 0, 0
        return self.tensor("cos"), self.tensor("sin"), int(self.info["rot_dim"]), int(self.info["style"])

    @property
    def max_positions(self):
        return int(self.info.get("max_positions", 1 << 30))


class BuildEnv:
    """Builds parts one by one: device and activation dtype of the run they are for."""

    def __init__(self, device, act_dtype):
        import torch
        self.device = torch.device(device)
        self.act_dtype = act_dtype
        self._code = native.dtype_code(act_dtype)

    def build(self, category, spec: PartSpec):
        if category not in CATEGORIES:
            raise KeyError("unknown part category '%s' (known: %s)" % (category, ", ".join(CATEGORIES)))
        return PartHandle(category, spec, self._code, self.device.type == "cuda")

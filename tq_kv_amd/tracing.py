"""Named ranges around the parts of a step, after the reference's tracing spans ("model", "attn",
"attn-mlp", "rms-norm", "output": src/models/turbo_generic.rs:36, :1920-1922, :1932-1933, entered
around the work at :43, :1957-1985).  The reference installs no subscriber, so its spans never
show; these show in a profiler's marker trace once switched on (`enable()`, `tq --trace`, or
TQ_TRACE=1 in the environment) and cost one test of a flag otherwise.  A step replayed from a
captured graph launches without passing through the parts, so only its outer range ("step")
appears.  The ranges are the engine library's (csrc/engine/trace.cpp): they go to ROCm's ROCTx
library, or to a pair of functions the caller installs."""
from . import native

_sink = []


def enable(on=True):
    """Switch the ranges on or off; returns whether they are on."""
    return bool(native.library().tqe_trace_enable(1 if on else 0))


def enabled():
    return bool(native.library().tqe_trace_enabled())


def set_sink(push=None, pop=None):
    """push(name: bytes) and pop() receive the ranges in place of ROCTx; None: ROCTx again."""
    import ctypes
    if push is None or pop is None:
        native.library().tqe_trace_sink(ctypes.cast(None, native.TRACE_PUSH), ctypes.cast(None, native.TRACE_POP))
        del _sink[:]
        return
    cbs = (native.TRACE_PUSH(lambda name: push(name) or 0), native.TRACE_POP(lambda: pop() or 0))
    _sink[:] = [cbs]
    native.library().tqe_trace_sink(*cbs)


class span:
    """`with span("attn"):` -- a named range around the work inside, if ranges are on."""
    __slots__ = ("name",)

    def __init__(self, name):
        self.name = name

    def __enter__(self):
        native.library().tqe_trace_push(native.enc(self.name))
        return self

    def __exit__(self, *exc):
        native.library().tqe_trace_pop()
        return False

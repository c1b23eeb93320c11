"""Named ranges around the parts of a step, after the reference's tracing spans ("model",
"attn", "attn-mlp", "rms-norm", "output": src/models/turbo_generic.rs:36, :1920-1922,
:1932-1933, entered around the work at :43, :1957-1985).  The reference installs no subscriber,
so its spans never show; these show in a profiler's marker trace once switched on
(`enable()`, `tq --trace`, or TQ_TRACE=1 in the environment) and cost one test of a flag
otherwise.  A step replayed from a captured graph launches without passing through the parts, so
only its outer range ("step") appears.

The ranges go to ROCm's ROCTx library (roctxRangePushA / roctxRangePop of
librocprofiler-sdk-roctx); where that cannot be loaded, enabling says so once and the ranges
stay inert."""
import ctypes
import os
import sys

_state = {"on": False, "lib": None, "tried": False}


def _load():
    if _state["tried"]:
        return _state["lib"]
    _state["tried"] = True
    for name in ("librocprofiler-sdk-roctx.so", "/opt/rocm/lib/librocprofiler-sdk-roctx.so", "libroctx64.so"):
        try:
            lib = ctypes.CDLL(name)
            lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
            lib.roctxRangePushA.restype = ctypes.c_int
            lib.roctxRangePop.argtypes = []
            lib.roctxRangePop.restype = ctypes.c_int
            _state["lib"] = lib
            return lib
        except (OSError, AttributeError):
            continue
    print("[tq_kv_amd tracing] no ROCTx library found: ranges stay off", file=sys.stderr)
    return None


def enable(on=True):
    """Switch the ranges on or off; returns whether they are on."""
    _state["on"] = bool(on) and _load() is not None
    return _state["on"]


def enabled():
    return _state["on"]


class span:
    """`with span("attn"):` -- a named range around the work inside, if ranges are on."""
    __slots__ = ("name", "pushed")

    def __init__(self, name):
        self.name, self.pushed = name, False

    def __enter__(self):
        if _state["on"]:
            _state["lib"].roctxRangePushA(self.name.encode())
            self.pushed = True
        return self

    def __exit__(self, *exc):
        if self.pushed:
            _state["lib"].roctxRangePop()
            self.pushed = False
        return False


if os.environ.get("TQ_TRACE", "") not in ("", "0"):
    enable()

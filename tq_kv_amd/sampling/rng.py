"""The uniform number of one draw: a function of (seed, request, step) and nothing else, so that
what a request draws does not depend on which other requests share its batch (csrc/engine/
generate.cpp: draw_uniform)."""
from .. import native

_M = (1 << 64) - 1


def uniform(seed, request, step):
    return float(native.library().tqe_draw_uniform(seed & _M, request & _M, step & _M))

"""Switches of the product and attention routines, for tests that compare one routine with
another; nothing else reads these.  They live in the engine library (tqe_policy_set / _get):

  skinny, mid, library   the hand-written products for few rows, for mid-sized steps, and the library's
  fused                  norms and residual sums folded into the products of small decoding steps
  prune_last             the last run of the order computes the wanted rows only
  packed                 parts keep a second copy of their bfloat16 weights in the few-row kernels'
                         order (twice the weight memory, about an eighth less time per decoding step)
  keep_rows              off: the rows are given up once a weight is packed (set it before loading):
                         half the weight memory again; a product of more than 128 rows (a prompt) gets the
                         rows back from the packed copy for its own length
  decode_mfma, prefill_mfma   the two matrix-core attention kernels (off: the plain kernel)
"""
from . import native

NAMES = ("skinny", "library", "fused", "prune_last", "packed", "mid", "keep_rows", "decode_mfma", "prefill_mfma")


class _Policy:
    def __getitem__(self, name):
        v = native.library().tqe_policy_get(native.enc(name))
        if v < 0:
            raise KeyError(name)
        return bool(v)

    def __setitem__(self, name, value):
        native.check(native.library().tqe_policy_set(native.enc(name), 1 if value else 0))

    def keys(self):
        return list(NAMES)

    def __iter__(self):
        return iter(NAMES)

    def items(self):
        return [(n, self[n]) for n in NAMES]

    def update(self, other=(), **kw):
        for k, v in dict(other, **kw).items():
            self[k] = v


POLICY = _Policy()

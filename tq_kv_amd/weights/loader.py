"""Loading a model's tensors by name, with one error for everything that is wrong.

The reference reads tensors by their HF names and fails at the first missing one
("Missing tensor: {name}", src/models/turbo_generic.rs:2056-2066), checks no shapes,
and casts BF16 to F32 (:2060-2065).  Here the wanted names and shapes come from the
model's parts, all of them are checked before anything is copied, and the dtype
policy is:

  run in bfloat16: floating tensors become bfloat16, except those stored in 32 (or
                   64) bit, which stay float32; integer tables become int32
  run in float32:  every floating tensor becomes float32 (exact for bf16 and f16)
"""
import torch

from .safetensors_io import open_folder


class WeightError(ValueError):
    """Missing tensors, unexpected tensors or wrong shapes; lists all of them."""

    def __init__(self, missing, unexpected, wrong_shape, wrong_kind=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_kind = list(wrong_shape), list(wrong_kind)
        lines = ["the weights do not fit the model:"]
        for name in self.missing:
            lines.append("  Missing tensor: %s" % name)
        for name in self.unexpected:
            lines.append("  Unexpected tensor: %s" % name)
        for name, got, want in self.wrong_shape:
            lines.append("  Wrong shape: %s is %s, expected %s" % (name, list(got), list(want)))
        for name, got, want in self.wrong_kind:
            lines.append("  Wrong dtype: %s is %s, expected %s" % (name, got, want))
        super().__init__("\n".join(lines))


def target_dtype(stored, kind, run_dtype):
    """The dtype a stored tensor is kept in (see the module text)."""
    if kind == "int32":
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return run_dtype


def check(stored, wanted, strict=True):
    """stored: name -> object with .shape and .dtype; wanted: name -> TensorSpec.
    Raises WeightError unless names and shapes agree exactly.  strict=False: tensors the model
    does not ask for (a tied checkpoint that still ships its head, rotary tables of an older
    export) are named in a warning instead, as the reference simply never looks them up
    (src/models/turbo_generic.rs:2056-2066)."""
    missing = [n for n in wanted if n not in stored]
    unexpected = sorted(n for n in stored if n not in wanted)
    if unexpected and not strict:
        import warnings
        warnings.warn("the folder holds %d tensors the model does not use: %s" % (len(unexpected), ", ".join(unexpected)))
        unexpected = []
    wrong_shape, wrong_kind = [], []
    for n, spec in wanted.items():
        if n not in stored:
            continue
        if tuple(stored[n].shape) != tuple(spec.shape):
            wrong_shape.append((n, tuple(stored[n].shape), tuple(spec.shape)))
        is_float = stored[n].dtype.is_floating_point
        if (spec.dtype == "float") != is_float:
            wrong_kind.append((n, stored[n].dtype, "a floating type" if spec.dtype == "float" else "an integer type"))
    if missing or unexpected or wrong_shape or wrong_kind:
        raise WeightError(missing, unexpected, wrong_shape, wrong_kind)


def load_folder(model_dir, wanted, run_dtype, device, strict=True):
    """name -> tensor on `device` for every wanted name, after the check."""
    stored = open_folder(model_dir)
    check(stored, wanted, strict)
    out = {}
    for name, spec in wanted.items():
        st = stored[name]
        out[name] = st.read().to(device=device, dtype=target_dtype(st.dtype, spec.dtype, run_dtype)).contiguous()
    return out

"""Weights: safetensors files read by tensor name, the by-name loader's one error, the dtype
policy, and random weights from a configuration and a seed.  All of it is the engine library's
(csrc/engine/weights.cpp); this module shows it to Python with torch tensors.

The reference loads every *.safetensors file of a folder into one map by name
(src/models/turbo_generic.rs:2039-2053), fails at the first missing tensor ("Missing tensor:
{name}", :2056-2066), checks no shapes, and casts BF16 to F32 (:2060-2065).  Here the wanted names
and shapes come from the model's parts, all of them are checked before anything is copied, and
the dtype policy is:

  run in bfloat16: floating tensors become bfloat16, except those stored in 32 (or 64) bit,
                   which stay float32; integer tables become int32
  run in float32:  every floating tensor becomes float32 (exact for bf16 and f16)
"""
import ctypes
import json
import os

import numpy as np
import torch

from .. import native
from ..native import WeightError, WeightFileError

__all__ = ["WeightError", "WeightFileError", "check", "load_folder", "target_dtype", "random_tensor", "random_tensors", "open_folder",
           "write_file", "register_init", "standard_normal_host", "tensor_key"]

DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
          "I32": torch.int32, "I64": torch.int64, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
          "BOOL": torch.bool}
NAMES = {v: k for k, v in DTYPES.items()}


class StoredTensor:
    """A tensor inside a file: name, dtype, shape, and a way to read it."""

    def __init__(self, folder, name, info):
        self._folder, self.name = folder, name
        self.dtype, self.shape = DTYPES[info["dtype"]], tuple(info["shape"])
        self._data, self._bytes = info["data"], info["bytes"]

    def read(self):
        """The tensor as a CPU tensor that views the file's memory map (do not write to it)."""
        if self._bytes == 0:
            return torch.empty(self.shape, dtype=self.dtype)
        buf = (ctypes.c_char * self._bytes).from_address(self._data)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")      # the map is read-only; it is only copied from
            t = torch.frombuffer(buf, dtype=self.dtype).reshape(self.shape)
        t._tq_keep = self._folder
        return t


class Folder(dict):
    """name -> StoredTensor over every *.safetensors file of a folder (memory-mapped by the library)."""

    def __init__(self, model_dir):
        super().__init__()
        self._lib = native.library()
        self.handle = native.handle(self._lib.tqe_folder_open(native.enc(str(model_dir))))
        for name, info in native.parsed(self._lib.tqe_folder_describe(self.handle)).items():
            self[name] = StoredTensor(self, name, info)

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            self._lib.tqe_folder_free(h)


def open_folder(model_dir):
    return Folder(model_dir)


def write_file(path, tensors, metadata=None):
    """Write name -> CPU tensor as one safetensors file."""
    items = list(tensors.items() if isinstance(tensors, dict) else tensors)
    keep, header = [], {}
    for name, t in items:
        t = t.detach().cpu().contiguous()
        keep.append(t)
        header[name] = {"dtype": NAMES[t.dtype], "shape": list(t.shape)}
    ptrs = (ctypes.c_void_p * max(len(keep), 1))(*[t.data_ptr() if t.numel() else None for t in keep])
    meta = None if not metadata else native.enc(json.dumps({str(k): str(v) for k, v in metadata.items()}))
    native.check(native.library().tqe_write_safetensors(native.enc(str(path)), native.enc(json.dumps(header)), ptrs, meta))
    return [name for name, _ in items]


def target_dtype(stored, kind, run_dtype):
    """The dtype a stored tensor is kept in (see the module text)."""
    if kind == "int32":
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return run_dtype


def check(folder, wanted, strict=True):
    """folder: an open Folder; wanted: name -> TensorSpec.  Raises WeightError unless names, shapes
    and kinds agree.  strict=False: tensors the model does not ask for are named in a warning
    instead, as the reference simply never looks them up (src/models/turbo_generic.rs:2056-2066)."""
    spec = native.enc(json.dumps({n: s.to_json() for n, s in wanted.items()}))
    native.check(native.library().tqe_check_weights(folder.handle, spec, 1 if strict else 0))
    native.warn_if_any()


def load_folder(model_dir, wanted, run_dtype, device, strict=True):
    """name -> tensor on `device` for every wanted name, after the check (what Model.from_dir does
    inside the library, as torch tensors for whoever wants to look at them)."""
    stored = open_folder(model_dir)
    check(stored, wanted, strict)
    out = {}
    for name, spec in wanted.items():
        st = stored[name]
        out[name] = st.read().to(device=device, dtype=target_dtype(st.dtype, spec.dtype, run_dtype)).contiguous()
    return out


# ---- random weights ------------------------------------------------------------------------------------
def tensor_key(seed, name):
    """The 64-bit key of a tensor's stream."""
    return int(native.library().tqe_tensor_key(int(seed), native.enc(name)))


def standard_normal_host(key, begin, count):
    """z for the elements begin .. begin + count - 1 of the stream `key`: float32 numpy array."""
    out = np.empty(int(count), dtype=np.float32)
    native.check(native.library().tqe_random_stream_of_key(int(key) & 0xFFFFFFFFFFFFFFFF, int(begin), int(count),
                                                           out.ctypes.data_as(ctypes.POINTER(ctypes.c_float))))
    return out


_INIT_FILLS = {}


def register_init(kind, fill):
    """Another way to fill a random tensor: fill(name, spec, seed, begin, count) -> float32 numpy array of the
    elements begin .. begin + count - 1, a function of (seed, name, index) alone."""
    from ..parts.spec import TensorSpec

    def call(user, name, spec_json, seed, begin, count, out):
        try:
            vals = np.asarray(fill(name.decode(), TensorSpec.from_json(json.loads(spec_json.decode())), int(seed), int(begin), int(count)),
                              dtype=np.float32)
            np.ctypeslib.as_array(out, shape=(int(count),))[:] = vals
            return 0
        except BaseException as e:      # noqa: B902
            native._pending_exception.append(e)
            return native.ERR_PART
    cb = native.INIT_FILL(call)
    _INIT_FILLS[kind] = (fill, cb)
    native.check(native.library().tqe_register_init(native.enc(kind), cb, None))


def random_tensor(name, spec, seed, dtype, device="cpu"):
    """One tensor of the random-weights stream, as the library makes it (the same values wherever it is made)."""
    device = torch.device(device)
    if spec.dtype == "int32":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    if dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("random weights are made in float32 or bfloat16, not %s" % dtype)
    numel = 1
    for s in spec.shape:
        numel *= int(s)
    if spec.init in ("normal", "one_plus_normal"):
        if device.type == "cuda":
            from .. import kernels as K
            out = torch.empty(tuple(spec.shape), dtype=dtype, device=device)
            return K.random_normal(out, tensor_key(seed, name), spec.std, spec.init == "one_plus_normal")
        val = standard_normal_host(tensor_key(seed, name), 0, numel) * np.float32(spec.std)
        if spec.init == "one_plus_normal":
            val = np.float32(1.0) + val
    elif spec.init in _INIT_FILLS:
        val = np.asarray(_INIT_FILLS[spec.init][0](name, spec, seed, 0, numel), dtype=np.float32)
    else:
        raise ValueError("unknown init '%s' for tensor %s" % (spec.init, name))
    return torch.from_numpy(np.ascontiguousarray(val)).to(dtype).reshape(tuple(spec.shape)).to(device)


def random_tensors(wanted, seed, dtype, device="cpu"):
    """name -> tensor for every wanted name; the same values wherever they are made."""
    return {name: random_tensor(name, spec, seed, dtype, device) for name, spec in wanted.items()}

"""A model: parts built from a ModelSpec, weights loaded into them, and the forward pass of one
step.  All of it is the engine library's (csrc/engine/model.cpp: embedding, the blocks in the
order the spec gives, final norm and head on the wanted rows, as the reference's forward does for
its one sequence, src/models/turbo_generic.rs:1950-1987); this class holds its handle.
"""
import ctypes
import json

import torch

from .. import native
from ..config import catalog
from ..config.base import ConfigError
from ..parts.spec import ModelSpec, TensorSpec, need_from_json

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
          torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def run_dtype(name):
    if name not in DTYPES:
        raise ValueError("dtype must be bfloat16 or float32, got %r" % (name,))
    return DTYPES[name]


def _shape_json(shape):
    raw = shape if isinstance(shape, dict) else catalog.find(shape)
    if raw is None:
        raise ConfigError("Model '%s' not found. Available shapes: %s"
                          % (shape, ", ".join("%s:%s" % e for e in catalog.entries())))
    return raw


class Model:
    """Model(spec, dtype, device): a model without weights from a ModelSpec made by hand; `load`
    gives it tensors.  Model.from_dir / Model.random / Model.from_config_dict are the usual ways."""

    def __init__(self, spec, dtype="bfloat16", device="cuda", config=None, _handle=None):
        self._lib = native.library()
        self.dtype = run_dtype(dtype)
        self.device = torch.device(device)
        self.on_gpu = self.device.type == "cuda"
        if self.on_gpu:
            from .. import kernels
            kernels.library()               # builds the kernels on a first call, with progress lines
            torch.cuda.current_device()     # the GPU is set up by torch, whose streams the engine works on
        if _handle is None:
            if spec is None:
                raise ValueError("a model needs a spec")
            _handle = native.handle(self._lib.tqe_model_from_spec(native.enc(json.dumps(spec.to_json())), native.dtype_code(self.dtype),
                                                                  1 if self.on_gpu else 0))
        self.handle = _handle
        self.config = config
        self._refresh()

    def _refresh(self):
        info = native.parsed(self._lib.tqe_model_describe(self.handle))
        self.spec = ModelSpec.from_json(info["spec"])
        self.needs = [need_from_json(n) for n in info["needs"]]
        self.cache_of = list(info["cache_of"])
        self.graph_safe = bool(info["graph_safe"])
        self.loaded = bool(info["loaded"])
        self.stop_token_ids = tuple(info["stop_token_ids"])
        self._tensors = {n: TensorSpec.from_json(s) for n, s in info["tensors"].items()}
        if self.config is None and info.get("config"):
            from ..config.registry import _CONFIG_CLASSES
            cls = _CONFIG_CLASSES.get(info["config"]["architecture"])
            self.config = cls.from_typed(info["config"]["config"]) if cls is not None else info["config"]["config"]

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            self._lib.tqe_model_free(h)

    # -- tensors ----------------------------------------------------------
    def tensor_specs(self):
        """Full tensor name -> TensorSpec of everything the model loads."""
        return dict(self._tensors)

    def load(self, tensors, strict=True):
        """Give the model its tensors (full names; torch tensors on any device, copied).  One
        WeightError lists everything that is missing, unexpected or misshapen."""
        stream = native.current_stream() if self.on_gpu else None
        for name, t in tensors.items():
            t = t.contiguous()
            if t.dtype not in (torch.float32, torch.bfloat16, torch.int32):
                t = t.to(torch.float32 if t.dtype.is_floating_point else torch.int32)
            ct = native.c_tensor(t)
            native.check(self._lib.tqe_model_set_tensor(self.handle, native.enc(name), ctypes.byref(ct), 1 if t.is_cuda else 0, stream))
        native.check(self._lib.tqe_model_finish(self.handle, 1 if strict else 0, stream))
        native.warn_if_any()
        self._refresh()
        return self

    def tensor(self, name):
        """A loaded tensor by its name, as a view of the model's memory.  Tensors that were folded into
        others are gone; what the parts made of them has names of its own (layer prefix +
        "self_attn.qkv.weight", "mlp.gate_up.weight", and "<weight>.packed" for the few-row kernels' copies)."""
        ct = native.tqe_tensor()
        native.check(self._lib.tqe_model_tensor(self.handle, native.enc(name), ctypes.byref(ct)))
        return native.view_of(ct, self.on_gpu, keep=self)

    def holds(self, name):
        try:
            self.tensor(name)
            return True
        except native.EngineLibraryError:
            return False

    @property
    def head_is_embedding(self):
        return self.spec.head_name is None

    # -- construction -----------------------------------------------------
    @classmethod
    def _made(cls, handle, dtype, device):
        return cls(None, dtype, device, _handle=native.handle(handle))

    @classmethod
    def from_config_dict(cls, raw, dtype="bfloat16", device="cuda"):
        """A model without weights from a parsed config.json."""
        dev = torch.device(device)
        if not isinstance(raw, dict):
            raise ConfigError("config.json: expected a JSON object at the top level")
        return cls._made(native.library().tqe_model_new(native.enc(json.dumps(raw)), native.dtype_code(run_dtype(dtype)),
                                                        1 if dev.type == "cuda" else 0), dtype, device)

    @classmethod
    def from_dir(cls, model_dir, dtype="bfloat16", device="cuda", strict=True):
        """A model folder: config.json picks the architecture, *.safetensors hold the weights.
        strict=False: tensors the model does not use are a warning, not an error."""
        dev = torch.device(device)
        if dev.type == "cuda":
            from .. import kernels
            kernels.library()
            torch.cuda.current_device()
        handle = native.handle(native.library().tqe_model_load(native.enc(str(model_dir)), native.dtype_code(run_dtype(dtype)),
                                                               1 if dev.type == "cuda" else 0, 1 if strict else 0))
        native.warn_if_any()
        return cls._made(handle, dtype, device)

    @classmethod
    def random(cls, shape, seed=0, dtype="bfloat16", device="cuda"):
        """Random weights made in memory.  shape: a catalog name ("tiny:a", "qwen2.5:7b") or a
        config.json dictionary.  Weights are drawn on `device`."""
        raw = _shape_json(shape)
        dev = torch.device(device)
        if dev.type == "cuda":
            from .. import kernels
            kernels.library()
            torch.cuda.current_device()
        return cls._made(native.library().tqe_model_random(native.enc(json.dumps(raw)), int(seed), native.dtype_code(run_dtype(dtype)),
                                                           1 if dev.type == "cuda" else 0), dtype, device)

    def randomize(self, seed=0):
        """Random weights for a model made from a spec."""
        native.check(self._lib.tqe_model_randomize(self.handle, int(seed), native.current_stream() if self.on_gpu else None))
        self._refresh()
        return self

    @staticmethod
    def write_random_folder(folder, shape, seed=0, store_dtype=torch.bfloat16):
        """Write config.json and model.safetensors with random weights; returns the folder."""
        raw = _shape_json(shape)
        native.check(native.library().tqe_write_random_folder(native.enc(str(folder)), native.enc(json.dumps(raw, indent=2)), int(seed),
                                                              native.dtype_code(store_dtype)))
        return str(folder)

    def tune_library(self, rows):
        """Let the matrix library try its kernels once for every product of the model at `rows` rows (more than the own
        kernels take: fewer never reach the library) and keep the fastest for later steps of that size.  Takes some
        milliseconds per distinct weight shape."""
        native.check(self._lib.tqe_model_tune_library(self.handle, int(rows), native.current_stream() if self.on_gpu else None))

    def __repr__(self):
        s = self.spec
        return "Model(architecture=%s, layers=%d, runs=%d, hidden=%d, vocab=%d, dtype=%s)" % (
            s.architecture, len(s.layers), len(s.order), s.hidden_size, s.vocab_size, str(self.dtype).replace("torch.", ""))

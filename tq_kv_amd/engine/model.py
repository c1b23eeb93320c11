"""A model: parts built from a ModelSpec, weights loaded into them, and the forward
pass of one step.  It knows nothing of any architecture: embedding, the blocks in
the order the spec gives, final norm and head on the wanted rows, as the
reference's forward does for its one sequence (src/models/turbo_generic.rs:1950-1987).
"""
import torch

from .. import kernels as K
from ..config import catalog
from ..config.base import ConfigError, read_config_json
from ..config.generation import stop_token_ids
from ..config.registry import config_from_dict, spec_for
from ..parts import linear as L
from ..parts.linear import linear
from ..parts.registry import BuildEnv
from ..parts.spec import TensorSpec
from ..tracing import span
from ..weights import load_folder, random_tensors, write_model_folder

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
          torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def run_dtype(name):
    if name not in DTYPES:
        raise ValueError("dtype must be bfloat16 or float32, got %r" % (name,))
    return DTYPES[name]


class Model:
    def __init__(self, spec, dtype="bfloat16", device="cuda", config=None):
        self.spec = spec
        self.config = config
        # stop tokens: what the configuration names; a model folder may add more (from_dir)
        self.stop_token_ids = tuple(spec.eos_token_ids)
        self.dtype = run_dtype(dtype)
        self.device = torch.device(device)
        self.env = BuildEnv(self.device, self.dtype)
        self.blocks = [self.env.build("block", layer.block) for layer in spec.layers]
        self.final_norm = self.env.build("norm", spec.final_norm)
        self.stream_position = (self.env.build("position", spec.stream_position)
                                if spec.stream_position is not None else None)
        if self.stream_position is not None and not hasattr(self.stream_position, "add_to_stream"):
            raise ValueError("position kind '%s' cannot act on the stream (it has no add_to_stream)" % spec.stream_position.kind)
        self.head_bias = None
        for i, run in enumerate(spec.order):
            if not 0 <= run.layer < len(self.blocks):
                raise ValueError("run %d names layer %d, the model has %d" % (i, run.layer, len(self.blocks)))
            if run.cache_of is not None and not 0 <= run.cache_of < i:
                raise ValueError("run %d reads the cache of run %r, which is not an earlier run" % (i, run.cache_of))
        self.needs = [self.blocks[run.layer].cache_need() for run in spec.order]
        self.cache_of = [run.cache_of for run in spec.order]
        for run in spec.order:
            mixer = getattr(self.blocks[run.layer], "mixer", None)
            if run.cache_of is not None and hasattr(mixer, "reads_other_cache"):
                mixer.reads_other_cache = True
        self.embedding = None
        self.head = None
        self.few_head = None
        self.loaded = False
        # a step can be captured as a graph if every part's forward launches the same kernels
        # whatever the step's data are; up to 128 rows (the hand-written products; where a weight
        # has no packed copy the library's, which capture as they are)
        self.graph_safe = (all(getattr(b, "graph_safe", False) for b in self.blocks) and getattr(self.final_norm, "graph_safe", False)
                           and (self.stream_position is None or getattr(self.stream_position, "graph_safe", False)))
        self.graph_max_rows = K.MID_MAX_ROWS

    # -- tensors ----------------------------------------------------------
    def tensor_specs(self):
        """Full tensor name -> TensorSpec of everything the model loads."""
        s = self.spec
        out = {s.embedding_name: TensorSpec((s.vocab_size, s.hidden_size))}
        for layer, block in zip(s.layers, self.blocks):
            for name, spec in block.tensors().items():
                out[layer.prefix + name] = spec
        for name, spec in self.final_norm.tensors().items():
            out[s.final_norm_prefix + name] = spec
        if s.head_name is not None:
            out[s.head_name] = TensorSpec((s.vocab_size, s.hidden_size))
        if self.stream_position is not None:
            for name, spec in self.stream_position.tensors().items():
                out[s.stream_position_prefix + name] = spec
        if s.head_bias_name is not None:
            out[s.head_bias_name] = TensorSpec((s.vocab_size,))
        return out

    def load(self, tensors):
        """Give every part its tensors (full names, already on the device)."""
        s = self.spec
        self.embedding = tensors[s.embedding_name]
        for layer, block in zip(s.layers, self.blocks):
            block.load({name: tensors[layer.prefix + name] for name in block.tensors()})
        self.final_norm.load({name: tensors[s.final_norm_prefix + name] for name in self.final_norm.tensors()})
        self.head = self.embedding if s.head_name is None else tensors[s.head_name]
        if self.stream_position is not None:
            self.stream_position.load({name: tensors[s.stream_position_prefix + name] for name in self.stream_position.tensors()})
        if s.head_bias_name is not None:
            self.head_bias = tensors[s.head_bias_name].to(torch.float32)
        self.few_head = L.few_rows_form(self.head)      # the head's copy for the few-row kernel
        self.head = L.rows_or_stand_in(self.head, self.few_head, needed=s.head_name is None)       # a tied head's rows are the embedding
        self.loaded = True
        return self

    # -- construction -----------------------------------------------------
    @classmethod
    def from_config_dict(cls, raw, dtype="bfloat16", device="cuda"):
        name, config = config_from_dict(raw)
        return cls(spec_for(name, config), dtype, device, config=config)

    @classmethod
    def from_dir(cls, model_dir, dtype="bfloat16", device="cuda", strict=True):
        """A model folder: config.json picks the architecture, *.safetensors hold the weights.
        strict=False: tensors the model does not use are a warning, not an error."""
        model = cls.from_config_dict(read_config_json(model_dir), dtype, device)
        model.stop_token_ids = stop_token_ids(model_dir, model.spec.eos_token_ids)
        return model.load(load_folder(model_dir, model.tensor_specs(), model.dtype, model.device, strict))

    @classmethod
    def random(cls, shape, seed=0, dtype="bfloat16", device="cuda"):
        """Random weights made in memory.  shape: a catalog name ("tiny:a", "qwen2.5:7b") or a
        config.json dictionary.  Weights are drawn on `device`."""
        raw = shape if isinstance(shape, dict) else catalog.find(shape)
        if raw is None:
            raise ConfigError("Model '%s' not found. Available shapes: %s"
                              % (shape, ", ".join("%s:%s" % e for e in catalog.entries())))
        model = cls.from_config_dict(raw, dtype, device)
        store = torch.bfloat16 if model.dtype == torch.bfloat16 else torch.float32
        return model.load(random_tensors(model.tensor_specs(), seed, store, model.device))

    @staticmethod
    def write_random_folder(folder, shape, seed=0, store_dtype=torch.bfloat16):
        """Write config.json and model.safetensors with random weights; returns the folder."""
        raw = shape if isinstance(shape, dict) else catalog.find(shape)
        if raw is None:
            raise ConfigError("Model '%s' not found. Available shapes: %s"
                              % (shape, ", ".join("%s:%s" % e for e in catalog.entries())))
        model = Model.from_config_dict(raw, "float32", "cpu")
        return write_model_folder(folder, raw, model.tensor_specs(), seed, store_dtype)

    def tune_library(self, rows):
        """Let the library try its kernels once for every product of the model at `rows`
        rows (more than 128, or 16 without packed weights: fewer never reach the library) and
        keep the fastest for later calls.  Takes seconds per distinct weight shape."""
        own_rows = K.MID_MAX_ROWS if L.POLICY["mid"] and L.POLICY["packed"] else L.POLICY["skinny_max_rows"]
        if self.dtype != torch.bfloat16 or rows <= own_rows:
            return
        L.tune_library(True)
        seen = set()
        products = [w for b in self.blocks for w in b.product_weights()] + [(self.head, torch.float32)]
        products = [(w, d) for w, d in products if torch.is_tensor(w)]
        for weight, out_dtype in products:
            key = (tuple(weight.shape), out_dtype)
            if weight.dtype != torch.bfloat16 or key in seen:
                continue
            seen.add(key)
            x = torch.zeros((rows, weight.shape[1]), dtype=torch.bfloat16, device=self.device)
            L.linear(x, weight, out_dtype=out_dtype)
        torch.cuda.synchronize()
        L.freeze_library_tuning()

    # -- one step ---------------------------------------------------------
    def forward(self, ctx, cache):
        """Run the step's tokens through every run of the order; logits [wanted rows, vocab]
        float32 for ctx's wanted rows."""
        if not self.loaded:
            raise RuntimeError("the model has no weights yet")
        with span("model"):                 # the reference's span, src/models/turbo_generic.rs:1932
            return self._forward(ctx, cache)

    def _forward(self, ctx, cache):
        s = self.spec
        h = torch.empty((ctx.n_tokens, s.hidden_size), dtype=torch.float32, device=self.device)
        # small decoding steps: products fold the norms and the residual sums around them in
        ctx.fuse_small = (L.POLICY["fused"] and self.dtype == torch.bfloat16 and ctx.all_decode
                          and ctx.n_tokens <= 16 and s.hidden_size % 32 == 0)
        # steps of 17 to 128 tokens: a part's last product may leave its sums to the next norm's kernel
        ctx.fuse_mid = (L.POLICY["mid"] and self.dtype == torch.bfloat16
                        and L.POLICY["skinny_max_rows"] < ctx.n_tokens <= K.MID_MAX_ROWS)
        # the norm that reads the stream first in every run, and after the last one
        firsts = [self.blocks[run.layer].first_norm() for run in s.order] + [self.final_norm]
        scale = 1.0 if s.embedding_scale is None else float(s.embedding_scale)
        if ctx.fuse_small:
            xw = torch.empty((ctx.n_tokens, s.hidden_size), dtype=torch.bfloat16, device=self.device)
            ss = torch.empty(((s.hidden_size + 15) // 16, 16), dtype=torch.float32, device=self.device)      # the most pieces a product gives
            stream = L.Stream(h, xw, ss)
            norm = firsts[0] if getattr(firsts[0], "foldable", False) else None
            K.embed(self.embedding, ctx.dev.tokens, h, copy=xw, copy_weight=norm.weight if norm is not None else None, ss_out=ss,
                    scale=scale)
            stream.xw_for, stream.n_ss = norm, 1
        else:
            stream = L.Stream(h)
            K.embed(self.embedding, ctx.dev.tokens, h, scale=scale)
        if self.stream_position is not None:
            self.stream_position.add_to_stream(h, ctx)
            stream.invalidate()              # what the gather prepared for the first norm is of the stream before this
        for i, run in enumerate(s.order):
            stream = self.blocks[run.layer].forward(stream, ctx, cache.entry(i), next_norm=firsts[i + 1],
                                                    last=i + 1 == len(s.order)) or stream
        n_rows = ctx.dev.want_rows.shape[0]
        if n_rows == 0:
            return torch.empty((0, s.vocab_size), dtype=torch.float32, device=self.device)
        with span("output"):                # src/models/turbo_generic.rs:1933
            return self._finish(self._head(stream, ctx, n_rows))

    def _finish(self, logits):
        """Bias, scale and cap of the logits, where the architecture has them."""
        s = self.spec
        if self.head_bias is not None or s.logit_scale is not None or s.logit_cap is not None:
            K.finish_logits(logits, self.head_bias, 1.0 if s.logit_scale is None else float(s.logit_scale),
                            0.0 if s.logit_cap is None else float(s.logit_cap))
        return logits

    def _head(self, stream, ctx, n_rows):
        s = self.spec
        # the last block may have gone on with the wanted rows alone, numbered among themselves
        want_rows = ctx.dev.want_in_last if getattr(stream, "of_last_rows", False) else ctx.dev.want_rows
        lazy = self.final_norm.lazy(stream) if ctx.fuse_small and hasattr(self.final_norm, "lazy") else None
        if lazy is not None and n_rows <= 16 and L.fusable(n_rows, self.head):
            logits = torch.empty((n_rows, s.vocab_size), dtype=torch.float32, device=self.device)
            return K.fused_store(lazy.xw, self.few_head or self.head, logits, lazy.norm, rows=want_rows)
        x = self.final_norm.gather_add_norm(stream.h, stream.pending, want_rows)
        return linear(x, self.head, out_dtype=torch.float32, few=self.few_head)

    def __repr__(self):
        s = self.spec
        return "Model(architecture=%s, layers=%d, runs=%d, hidden=%d, vocab=%d, dtype=%s)" % (
            s.architecture, len(s.layers), len(s.order), s.hidden_size, s.vocab_size, str(self.dtype).replace("torch.", ""))

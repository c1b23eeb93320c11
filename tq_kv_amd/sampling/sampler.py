"""Choosing next tokens on the device for the live requests of a batch (csrc/engine/generate.cpp:
DeviceSampler, behind tqe_sampler_*; this class holds the handle).

The reference samples one request on the host (src/engine.rs:353-373, 403-423): repeat penalty over
the generated tokens (not on the first draw, when none exist), then argmax if temperature <= 0,
else top-k then top-p at the temperature.  Here the same steps run as kernels on the rows of the
step's logits; the history of generated tokens lives on the device and is appended to by a kernel.
The generation loop makes its samplers inside the library; this one is for whoever steps an engine
by hand.
"""
import ctypes

import numpy as np

from .. import native


class Sampler:
    """params: GenerationParams.  request_ids: for each request of the batch its number in the
    whole run (feeds the random stream)."""

    def __init__(self, params, request_ids, device, vocab_size=None):
        from ..engine.generate import _c_params
        self._lib = native.library()
        self.params = params
        self.request_ids = list(request_ids)
        self.device = device
        self._vocab = vocab_size
        self._cp = _c_params(params)
        self.handle = None

    def _ensure(self, vocab):
        if self.handle is None:
            ids = np.asarray(self.request_ids, dtype=np.int32)
            self._vocab = int(vocab)
            self.handle = native.handle(self._lib.tqe_sampler_new(ctypes.byref(self._cp), len(ids), native._ptr(ids), self._vocab,
                                                                  native.current_stream()))
        elif int(vocab) != self._vocab:
            raise ValueError("this sampler was made for a vocabulary of %d, the logits have %d" % (self._vocab, vocab))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            self._lib.tqe_sampler_free(h)

    def sample(self, logits, rows):
        """logits: [R, V] float32 on the device (changed in place by the penalty); rows: for each row
        the request's index in the batch.  The R chosen token ids as a list."""
        import torch
        if logits.dtype != torch.float32 or not logits.is_contiguous() or logits.dim() != 2 or logits.shape[0] != len(rows):
            raise ValueError("the sampler takes float32 logits [%d, vocab], got %s %s" % (len(rows), logits.dtype, tuple(logits.shape)))
        self._ensure(logits.shape[1])
        r = np.asarray(list(rows), dtype=np.int32)
        out = np.zeros(max(1, len(r)), dtype=np.int32)
        native.check(self._lib.tqe_sampler_sample(self.handle, ctypes.c_void_p(logits.data_ptr()), len(r), native._ptr(r), native._ptr(out)))
        return out[:len(r)].tolist()

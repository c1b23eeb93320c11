"""Choosing next tokens on the device for the live requests of a batch.

The reference samples one request on the host (src/engine.rs:353-373, 403-423):
repeat penalty over the generated tokens (not on the first draw, when none exist),
then argmax if temperature <= 0, else top-k then top-p at the temperature.  Here the
same steps run as kernels on the rows of the step's logits; the history of generated
tokens lives on the device and is appended to by a kernel.
"""
import numpy as np
import torch

from .. import kernels as K
from .rng import uniform


class Sampler:
    """params: GenerationParams.  n_requests: requests of the batch; request_ids: for each
    its number in the whole run (feeds the random stream)."""

    def __init__(self, params, request_ids, device):
        self.params = params
        self.request_ids = list(request_ids)
        self.device = device
        n = len(self.request_ids)
        self.use_penalty = params.repeat_penalty != 1.0
        if self.use_penalty:
            self.hist = torch.zeros((n, max(1, params.max_tokens + 1)), dtype=torch.int32, device=device)
            self.hist_len = torch.zeros((n,), dtype=torch.int32, device=device)
        self.steps = [0] * n

    def sample(self, logits, rows):
        """logits: [R, V] float32 (changed in place by the penalty); rows: for each row the
        request's index in the batch.  Returns the R chosen token ids as a list."""
        p = self.params
        n = len(rows)
        out = torch.empty((n,), dtype=torch.int32, device=self.device)
        row_req = None
        if self.use_penalty:
            row_req = torch.tensor(rows, dtype=torch.int32).to(self.device)
            K.repeat_penalty(logits, row_req, self.hist, self.hist_len, p.repeat_penalty)
        if p.greedy:
            K.argmax(logits, out)
        else:
            u = np.asarray([uniform(p.seed, self.request_ids[r], self.steps[r]) for r in rows], dtype=np.float32)
            K.sample(logits, p.temperature, p.top_k, p.top_p, torch.from_numpy(u).to(self.device), out)
        for r in rows:
            self.steps[r] += 1
        if self.use_penalty:
            K.append_history(out, row_req, self.hist, self.hist_len)
        return out.tolist()

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


class Drawn:
    """Tokens that have been chosen on the device and are on their way to the host.
    `device`: int32 [rows].  read() waits for this draw's copy alone, not for work that was
    started after it."""

    def __init__(self, device, host, event):
        self.device, self._host, self._event = device, host, event

    def read(self):
        self._event.synchronize()
        return self._host.tolist()


class Sampler:
    """params: GenerationParams.  n_requests: requests of the batch; request_ids: for each
    its number in the whole run (feeds the random stream)."""

    READ_AHEAD = 4         # draws that may be unread at a time

    def __init__(self, params, request_ids, device):
        from ..engine.context import HostStaging
        self.params = params
        self.request_ids = list(request_ids)
        self.device = device
        n = len(self.request_ids)
        self.use_penalty = params.repeat_penalty != 1.0
        if self.use_penalty:
            self.hist = torch.zeros((n, max(1, params.max_tokens + 1)), dtype=torch.int32, device=device)
            self.hist_times = torch.zeros_like(self.hist)
            self.hist_len = torch.zeros((n,), dtype=torch.int32, device=device)
        self.steps = [0] * n
        self.staging = HostStaging(device, depth=2 * self.READ_AHEAD)
        self.landing = torch.empty((self.READ_AHEAD, max(1, n)), dtype=torch.int32, pin_memory=True)
        self.turn = 0

    def draw(self, logits, rows):
        """logits: [R, V] float32 (changed in place by the penalty); rows: for each row the
        request's index in the batch.  Starts the choice and the copy of the R chosen token
        ids to the host, waits for neither."""
        p = self.params
        n = len(rows)
        out = torch.empty((n,), dtype=torch.int32, device=self.device)
        row_req = None
        if self.use_penalty:
            row_req = self.staging.upload(np.asarray(rows, dtype=np.int32))
            K.repeat_penalty(logits, row_req, self.hist, self.hist_times, self.hist_len, p.repeat_penalty)
        if p.greedy:
            K.argmax(logits, out)
        else:
            u = np.asarray([uniform(p.seed, self.request_ids[r], self.steps[r]) for r in rows], dtype=np.float32)
            K.sample(logits, p.temperature, p.top_k, p.top_p, self.staging.upload(u), out)
        for r in rows:
            self.steps[r] += 1
        if self.use_penalty:
            K.append_history(out, row_req, self.hist, self.hist_times, self.hist_len)
        host = self.landing[self.turn, :n]
        self.turn = (self.turn + 1) % self.READ_AHEAD
        host.copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return Drawn(out, host, event)

    def pick(self, drawn, places):
        """The tokens of a draw at the given places, on the device, in that order."""
        if list(places) == list(range(drawn.device.shape[0])):
            return drawn.device
        return drawn.device[self.staging.upload(np.asarray(places, dtype=np.int32)).long()]

    def sample(self, logits, rows):
        """draw() and wait: the R chosen token ids as a list."""
        return self.draw(logits, rows).read()

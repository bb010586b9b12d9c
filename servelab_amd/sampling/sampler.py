"""Logits -> tokens, on the device.

Reference: ``Sampler`` (servelab/engine/sampler.py:10-45) handles rows one at a
time on the host: temperature 0 is argmax; else softmax(logits / T), top-k
(which ignores top-p) or top-p, multinomial from one engine-wide generator, or
from a fresh generator per call when the request has a seed.  Here one kernel
call samples all rows; a row's random stream is keyed by (seed, number of
tokens the request has drawn), so it does not depend on the batch it shares.
"""
from typing import List, Sequence

import numpy as np
import torch


def _mix(seed: int, number: int) -> int:
    """A 63-bit key from the engine seed and the request's submission number."""
    z = (seed * 0x9E3779B97F4A7C15 + (number + 1) * 0xBF58476D1CE4E5B9) & 0xFFFFFFFFFFFFFFFF
    z ^= z >> 31
    return z & 0x7FFFFFFFFFFFFFFF


class _RowBuffers:
    """Pinned host buffers for the per-row arrays of a sampling call, taken in turn: the copy to the
    device is queued behind the step that is still running and must not make the host wait for it (a
    copy from pageable memory does, which cost a decode step of 16 requests 0.16 of its 4.2 ms), and
    a buffer is written again only after its last copy has left it."""

    TURNS = 4

    def __init__(self):
        self.buffers = [None] * self.TURNS
        self.copied = [None] * self.TURNS
        self.turn = 0

    def take(self, n: int) -> np.ndarray:
        self.turn = (self.turn + 1) % self.TURNS
        if self.copied[self.turn] is not None:
            self.copied[self.turn].synchronize()
        if self.buffers[self.turn] is None or self.buffers[self.turn].numel() < n:
            self.buffers[self.turn] = torch.empty(max(2 * n, 256), dtype=torch.int32).pin_memory()
        return self.buffers[self.turn][:n].numpy()

    def to_device(self, n: int, device) -> torch.Tensor:
        dev = torch.empty(n, dtype=torch.int32, device=device)
        dev.copy_(self.buffers[self.turn][:n], non_blocking=True)
        if self.copied[self.turn] is None:
            self.copied[self.turn] = torch.cuda.Event()
        self.copied[self.turn].record()
        return dev


class Sampler:
    def __init__(self, ops, device, seed: int = 0):
        self.ops = ops
        self.device = torch.device(device)
        self.seed = int(seed)
        self._rows = _RowBuffers() if self.device.type == "cuda" else None

    def row_seed(self, params, number: int) -> int:
        return int(params.seed) if params.seed >= 0 else _mix(self.seed, number)

    def sample(self, logits: torch.Tensor, params: Sequence, numbers: Sequence[int],
               draws: Sequence[int]) -> List[int]:
        """``logits`` [B, V] float32; ``params[i]`` the SamplingParams of row i,
        ``numbers[i]`` its request's submission number, ``draws[i]`` how many
        tokens that request has sampled before.  Returns the tokens on the host."""
        if logits.shape[0] == 0:
            return []
        return self.sample_on_device(logits, params, numbers, draws).tolist()

    def sample_on_device(self, logits: torch.Tensor, params: Sequence, numbers: Sequence[int],
                         draws: Sequence[int]) -> torch.Tensor:
        """The same, but the tokens stay on the device (int32 [B]) and nothing
        waits for them: the next step can take them from there."""
        if all(p.temperature == 0.0 for p in params):
            return self.ops.argmax(logits)
        # one host buffer and one copy for the five per-row arrays:
        # seeds and draw counters (int64), temperature and top_p (float32), top_k (int32)
        B = len(params)
        buf = self._rows.take(7 * B) if self._rows is not None else np.empty(7 * B, dtype=np.int32)
        buf[:2 * B].view(np.int64)[:] = [self.row_seed(p, n) for p, n in zip(params, numbers)]
        buf[2 * B:4 * B].view(np.int64)[:] = list(draws)
        buf[4 * B:5 * B].view(np.float32)[:] = [p.temperature for p in params]
        buf[5 * B:6 * B].view(np.float32)[:] = [p.top_p for p in params]
        buf[6 * B:] = [p.top_k for p in params]
        dev = self._rows.to_device(7 * B, self.device) if self._rows is not None else torch.from_numpy(buf).to(self.device)
        cut = any(p.top_k > 0 or p.top_p < 1.0 for p in params)
        return self.ops.sample(
            logits, dev[4 * B:5 * B].view(torch.float32), dev[6 * B:] if cut else None,
            dev[5 * B:6 * B].view(torch.float32) if cut else None,
            dev[:2 * B].view(torch.int64), dev[2 * B:4 * B].view(torch.int64))

"""Position encodings, as parameters of a mixer.

Rotary: inv_freq[j] = theta^(-2j/D) built in float32 as
``1 / theta ** (arange(0, D, 2) / D)`` (servelab/parallel/tp_model.py:94-96);
angles, cos and sin are float32; the rotation pairs (j, j + D/2)
(docs/architecture.md:69).
"""
import torch

from .base import PositionEncoding


class RotaryPosition(PositionEncoding):
    graph_safe = True

    kind = "rotary"

    def __init__(self, head_dim: int, theta: float):
        if head_dim % 2:
            raise ValueError(f"rotary head_dim must be even, is {head_dim}")
        self.head_dim = int(head_dim)
        self.theta = float(theta)

    def load(self, tensors, rt):
        self.rt = rt
        inv = 1.0 / (self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32)
                                    / self.head_dim))
        self.inv_freq = inv.to(rt.device)

    def tables(self, batch, shared):
        key = ("rotary", self.head_dim, self.theta)
        if key not in shared:
            shared[key] = self.rt.ops.rope_tables(batch.positions, self.inv_freq)
        return shared[key]


class NoPosition(PositionEncoding):
    graph_safe = True

    kind = "none"

    def tables(self, batch, shared):
        return None

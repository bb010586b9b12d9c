"""Position encodings, as parameters of a mixer.

Rotary: inv_freq[j] = theta^(-2j/D) built in float32 as
``1 / theta ** (arange(0, D, 2) / D)`` (servelab/parallel/tp_model.py:94-96);
angles, cos and sin are float32; the rotation pairs (j, j + D/2)
(docs/architecture.md:69).  ``rotary_dim`` (the leading channels that are
rotated) and ``pairing`` go beyond the reference, whose heads turn whole and in
halves.
"""
import torch

from .base import PositionEncoding, RotaryLayout, RotaryTables


class RotaryPosition(PositionEncoding):
    graph_safe = True

    kind = "rotary"

    def __init__(self, head_dim: int, theta: float, rotary_dim=None, pairing: str = "half"):
        self.head_dim = int(head_dim)
        self.rotary_dim = self.head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"the rotated width must be even and within head_dim {head_dim}, "
                             f"is {self.rotary_dim}")
        self.theta = float(theta)
        self.pairing = pairing

    def layout(self):
        return RotaryLayout(self.rotary_dim, self.pairing)

    def load(self, tensors, rt):
        self.rt = rt
        inv = 1.0 / (self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32)
                                    / self.rotary_dim))
        self.inv_freq = inv.to(rt.device)

    def tables(self, batch, shared):
        key = ("rotary", self.rotary_dim, self.theta)
        if key not in shared:
            shared[key] = RotaryTables(*self.rt.ops.rope_tables(batch.positions, self.inv_freq))
        return shared[key]


class NoPosition(PositionEncoding):
    graph_safe = True

    kind = "none"

    def tables(self, batch, shared):
        return None

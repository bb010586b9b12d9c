"""Gated feed-forward (SwiGLU): down(silu(gate(x)) * up(x)), no biases.

Reference: servelab/parallel/tp_model.py:56-68 (two GEMMs, silu, multiply, one
GEMM).  Here gate and up are one GEMM over [Wg; Wu] followed by one fused
silu-multiply kernel.
"""
import torch

from .base import FeedForward, ParamSpec


class GatedMLP(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation != "silu":
            raise ValueError(f"GatedMLP: activation '{activation}' is not supported")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)

    def param_specs(self):
        h, i = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": ParamSpec((i, h)),
                "up_proj.weight": ParamSpec((i, h)),
                "down_proj.weight": ParamSpec((h, i))}

    def load(self, tensors, rt):
        self.rt = rt
        self.w_gate_up = rt.linear_weight(torch.cat(
            [tensors("gate_proj.weight"), tensors("up_proj.weight")], 0))
        self.w_down = rt.linear_weight(tensors("down_proj.weight"))

    def forward(self, x):
        ops = self.rt.ops
        gate_up = ops.linear(x, self.w_gate_up, None)
        return ops.linear(ops.silu_mul(gate_up), self.w_down, None)

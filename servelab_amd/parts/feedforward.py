"""Gated feed-forward (SwiGLU): down(silu(gate(x)) * up(x)), no biases.

Reference: servelab/parallel/tp_model.py:56-68 (two GEMMs, silu, multiply, one
GEMM).  Here gate and up are one GEMM over a matrix that holds the rows of Wg
and Wu interleaved in blocks of 8 (so that one output tile of the few-rows
kernel has a channel's gate and up and can apply silu-multiply itself), then
the down GEMM.
"""
import torch

from .base import FeedForward, ParamSpec


class GatedMLP(FeedForward):
    graph_safe = True
    takes_scaled_rows = True

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
        gate, up = tensors("gate_proj.weight"), tensors("up_proj.weight")
        i, h = self.intermediate_size, self.hidden_size
        self.block = getattr(rt.ops, "GATE_BLOCK", i)
        if i % self.block:
            self.block = i                       # plain [Wg; Wu]
        b = self.block
        self.w_gate_up = rt.linear_weight(torch.stack(
            [gate.reshape(i // b, b, h), up.reshape(i // b, b, h)], 1).reshape(2 * i, h))
        self.w_down = rt.linear_weight(tensors("down_proj.weight"), delta=True)

    def forward(self, x):
        ops = self.rt.ops
        return ops.gated_mlp(x, self.w_gate_up, self.block, self.w_down, defer=True)

"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w in float32.

Reference: servelab/attention/triton/paged_attention.py:76-91 and the vector
in tests/test_triton_kernels.py:57-59.  Here the residual add that precedes
every use (servelab/parallel/tp_model.py:131-133) is fused in.
"""
from .base import Norm, ParamSpec


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), init="gain")}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.vector(tensors("weight"))

    def forward(self, resid, delta, fuse=False):
        return self.rt.ops.add_rmsnorm(resid, delta, self.weight, self.eps, fuse=fuse)

    def forward_rows(self, resid, delta, rows, fuse=False):
        return self.rt.ops.rows_add_rmsnorm(resid, delta, rows, self.weight, self.eps, fuse=fuse)

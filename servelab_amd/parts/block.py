"""Arrangements of parts in a block.

PreNormBlock: h += Mixer(Norm1(h)); h += FeedForward(Norm2(h))
(servelab/parallel/tp_model.py:124-133).  The adds are fused into the norm
that follows them, so a block returns its feed-forward output as a pending
delta for the next norm to add.
"""
from .base import Block, prefixed


class PreNormBlock(Block):
    def __init__(self, norm1, mixer, norm2, feedforward,
                 names=("input_layernorm.", "self_attn.", "post_attention_layernorm.", "mlp.")):
        self.norm1, self.mixer, self.norm2, self.feedforward = norm1, mixer, norm2, feedforward
        self.names = tuple(names)

    @property
    def graph_safe(self):
        return all(part.graph_safe for _, part in self._children())

    def _children(self):
        return list(zip(self.names, (self.norm1, self.mixer, self.norm2, self.feedforward)))

    def cache_specs(self):
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def param_specs(self):
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[prefix + name] = spec
        return specs

    def load(self, tensors, rt):
        self.rt = rt
        for prefix, part in self._children():
            part.load(prefixed(prefix, tensors), rt)

    def forward(self, resid, delta, batch, caches, shared):
        x = self.norm1.forward(resid, delta, fuse=self.mixer.takes_scaled_rows)
        a = self.mixer.forward(x, batch, caches[0] if caches else None, shared)
        x2 = self.norm2.forward(resid, a, fuse=self.feedforward.takes_scaled_rows)
        return self.feedforward.forward(x2)

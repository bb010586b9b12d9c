"""Token embedding and output head.

Embedding lookup servelab/parallel/tp_model.py:123; head = embedding table when
tied, else its own matrix, no bias, logits returned in float32
(servelab/parallel/tp_model.py:115-119, servelab/engine/engine.py:218).
"""
from .base import Embedding, Part, ParamSpec


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.matrix(tensors("weight"))

    def forward(self, batch):
        """The rows of the table at ``batch.ids`` (int32 [T]) as the float32
        residual stream [T, H]."""
        return self.rt.ops.embed(batch.ids, self.weight)


class OutputHead(Part):
    graph_safe = True
    takes_scaled_rows = True

    """``tied_to`` is the embedding part whose table the head shares, or None."""

    def __init__(self, vocab_size: int, hidden_size: int, tied_to=None):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to

    def param_specs(self):
        if self.tied_to is not None:
            return {}
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors, rt):
        self.rt = rt
        if self.tied_to is not None:
            self.weight = rt.linear_weight(self.tied_to.weight, shared=True)
        else:
            self.weight = rt.linear_weight(tensors("weight"))

    def forward(self, rows):
        """normed rows [R, H] -> float32 logits [R, V]."""
        return self.rt.ops.linear(rows, self.weight, None, out_f32=True)

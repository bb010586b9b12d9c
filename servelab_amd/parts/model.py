"""A decoder model as data: an embedding, a set of blocks, the list of layer
calls that says in which order the blocks run and which cache stream each call
uses, a final norm and an output head.

Reference: ``forward_packed`` + ``lm_head_forward``
(servelab/parallel/tp_model.py:115-134) run blocks 0..L-1 once each with one
cache per block.  Here that order is the list ``run``; it may name a block
twice (each call with a cache stream of its own) or let a call read the stream
another call wrote.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from .base import PagedKVSpec, ParamSpec, Part, Runtime, StateSpec, prefixed


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run list: run block ``layer`` against cache stream
    ``stream``, or against several streams (a tuple) when the block declares
    several cache needs, one stream for each in the order of its
    ``cache_specs()``; ``()`` for a block that caches nothing.  ``write`` False
    reads streams that an earlier call of this step has written."""
    layer: int
    stream: Union[int, Tuple[int, ...]] = ()
    write: bool = True

    @property
    def streams(self) -> Tuple[int, ...]:
        return (self.stream,) if isinstance(self.stream, int) else tuple(self.stream)


@dataclass
class ModelSpec:
    embedding: Tuple[str, Part]                 # (checkpoint prefix, part)
    layers: List[Tuple[str, Part]]              # (prefix, block)
    run: List[LayerCall]
    final_norm: Tuple[str, Part]
    head: Tuple[str, Part]
    vocab_size: int
    hidden_size: int
    eos_token_id: int = 0
    max_position_embeddings: int = 1 << 30
    optional_tensors: Tuple[str, ...] = ()      # names a checkpoint may hold unused

    def children(self):
        return [self.embedding] + list(self.layers) + [self.final_norm, self.head]

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self.children())

    def param_specs(self) -> Dict[str, ParamSpec]:
        """Every checkpoint tensor of the model, in a fixed order."""
        specs: Dict[str, ParamSpec] = {}
        for prefix, part in self.children():
            for name, spec in part.param_specs().items():
                specs[prefix + name] = spec
        return specs

    def stream_specs(self) -> Dict[int, Any]:
        """{cache stream: the cache need it serves}, from what the blocks of
        the run list declare (``Block.cache_specs``)."""
        def needs(call):
            specs = list(self.layers[call.layer][1].cache_specs())
            if len(specs) != len(call.streams):
                raise ValueError(f"layer call of block {call.layer} names {len(call.streams)} cache "
                                 f"streams, the block declares {len(specs)} cache needs")
            return zip(call.streams, specs)
        out: Dict[int, Any] = {}
        for call in self.run:
            if call.write:
                for stream, spec in needs(call):
                    if stream in out:
                        raise ValueError(f"cache stream {stream} is written by two layer calls")
                    out[stream] = spec
        for call in self.run:
            if not call.write:
                for stream, spec in needs(call):
                    if stream not in out:
                        raise ValueError(f"layer call reads stream {stream} that no call writes")
                    if spec != out[stream]:
                        raise ValueError(
                            f"layer {call.layer} reads stream {stream} of a different cache kind")
        return out


def build_model_spec(config) -> ModelSpec:
    """The registered builder of ``config.architecture``."""
    from ..config.registry import resolve_architecture
    return resolve_architecture({"architectures": [config.architecture]}).build_spec(config)


class DecoderModel:
    """A ModelSpec with its weights on the device."""

    def __init__(self, spec: ModelSpec, rt: Runtime):
        self.spec = spec
        self.rt = rt
        self.loaded = False

    def load(self, checkpoint) -> None:
        """``checkpoint``: a weights.Checkpoint or a {name: tensor} dict.  All
        names and shapes are checked first, in one error."""
        from ..weights.loader import check_tensors
        specs = self.spec.param_specs()
        if isinstance(checkpoint, dict):
            found = {n: tuple(t.shape) for n, t in checkpoint.items()}
            get = checkpoint.__getitem__
        else:
            found = checkpoint.shapes()
            get = checkpoint.get
        check_tensors({n: s.shape for n, s in specs.items()}, found,
                      optional=self.spec.optional_tensors)
        plan = getattr(self.rt.ops, "plan_weights", None)
        if plan is not None:          # let the kernel table choose its weight layout for this size
            itemsize = torch.empty((), dtype=self.rt.act_dtype).element_size()
            total = 0
            for s in specs.values():
                if len(s.shape) == 2:
                    total += s.shape[0] * s.shape[1] * itemsize
            plan(total)
        for prefix, part in self.spec.children():
            part.load(prefixed(prefix, get), self.rt)
        self.loaded = True

    def forward(self, batch, bindings) -> torch.Tensor:
        """Run the batch's tokens through the run list; returns float32 logits
        [R, V] at ``batch.logit_rows``.  ``bindings[i]`` are the cache bindings of
        ``spec.run[i]``, one for each of its streams."""
        spec = self.spec
        shared: Dict[Any, Any] = {}
        resid = spec.embedding[1].forward(batch)
        delta = None
        for call, caches in zip(spec.run, bindings):
            delta = spec.layers[call.layer][1].forward(resid, delta, batch, caches, shared)
        if batch.num_logit_rows == 0:
            # the last block's output is never read; nothing to add
            return torch.empty((0, spec.vocab_size), dtype=torch.float32, device=self.rt.device)
        rows = spec.final_norm[1].forward_rows(resid, delta, batch.logit_rows,
                                               fuse=getattr(spec.head[1], "takes_scaled_rows", False))
        return spec.head[1].forward(rows)

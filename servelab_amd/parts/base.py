"""What every part is made of: parameter and cache declarations, the runtime a
part computes with, and the interfaces of the five kinds of part.

A part owns its sizes and constants as constructor parameters, declares the
checkpoint tensors it needs under names *relative to itself* (the model puts
the prefix in front), says what it needs cached per request, and computes
through the kernel table of the runtime.  No part knows which model it is in.
"""
from dataclasses import dataclass
from typing import Callable, Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One checkpoint tensor a part needs."""
    shape: Tuple[int, ...]
    init: str = "normal"       # random-weights mode: "normal" N(0, std) | "gain" 1 + N(0, norm_std)


@dataclass(frozen=True)
class PagedKVSpec:
    """Cache need: keys and values of past tokens, in pages.  ``window`` None
    keeps every token; a window W keeps the last W."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    """Cache need: one fixed-size state per request."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


class Runtime:
    """Device, activation dtype and kernel table that parts compute with."""

    def __init__(self, ops, device, act_dtype: torch.dtype):
        self.ops = ops
        self.device = torch.device(device)
        self.act_dtype = act_dtype

    def matrix(self, t: torch.Tensor) -> torch.Tensor:
        """A matrix or table in the activation dtype, on the device."""
        return t.to(device=self.device, dtype=self.act_dtype).contiguous()

    def linear_weight(self, t: torch.Tensor, shared: bool = False, delta: bool = False):
        """A matrix that only ``ops.linear`` reads, in whatever form the kernel
        table wants it.  ``shared``: another part keeps ``t`` itself as well.
        ``delta``: its products are only ever added to the residual stream."""
        m = self.matrix(t)
        prepare = getattr(self.ops, "prepare_weight", None)
        return prepare(m, keep_rows=shared, residual_delta=delta) if prepare is not None else m

    def vector(self, t: torch.Tensor) -> torch.Tensor:
        """A gain or bias: always float32 on the device (they enter float32 math)."""
        return t.to(device=self.device, dtype=torch.float32).contiguous()


TensorSource = Callable[[str], torch.Tensor]


def prefixed(prefix: str, source: TensorSource) -> TensorSource:
    return lambda name: source(prefix + name)


class Part:
    """Base of all parts.  ``graph_safe`` says that the part's computation is a
    fixed sequence of kernel launches that reads sizes only from the batch's
    host fields and data only from device memory (no host synchronisation, no
    library call that records memsets), so a decode step through it may be
    captured into a HIP graph and replayed."""

    graph_safe = False

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def load(self, tensors: TensorSource, rt: Runtime) -> None:
        """Fetch the declared tensors by relative name and keep device copies."""
        self.rt = rt


class Norm(Part):
    """forward(resid, delta) adds ``delta`` (or nothing) into the float32
    residual stream in place and returns the normed rows in the activation
    dtype; forward_rows returns the normed selected rows.

    ``delta`` is what the part before returned: a tensor, or a product the
    kernel table deferred (``ops.linear(..., defer=True)``), which the norm's
    kernel call runs.  ``fuse`` says that the reader of the normed rows passes
    them only to ``ops.linear`` / ``ops.gated_linear`` / ``ops.gated_mlp`` (it has
    ``takes_scaled_rows``); the kernel table may then hand it rows whose
    normalisation the reader's product completes."""

    def forward(self, resid, delta, fuse=False):
        raise NotImplementedError

    def forward_rows(self, resid, delta, rows, fuse=False):
        raise NotImplementedError


@dataclass(frozen=True)
class RotaryLayout:
    """Which channels of a head a rotary encoding turns: the first ``rot_dim``
    (the rest pass), in pairs (j, j + rot_dim / 2) ("half") or (2j, 2j + 1)
    ("interleaved")."""
    rot_dim: int
    pairing: str = "half"


@dataclass
class RotaryTables:
    """A rotary encoding's work for one step: cos and sin of every token's
    angles, float32 [T, rot_dim / 2]."""
    cos: torch.Tensor
    sin: torch.Tensor


class PositionEncoding(Part):
    """A parameter of a mixer, which never looks inside it.  ``layout()`` says
    at load time what the encoding does to the channels of a head (None:
    nothing; a ``RotaryLayout``), from which the kernel table decides the
    channel order it wants; ``tables(batch, shared)`` returns what the kernels
    need for this step's positions (None, or ``RotaryTables``), which the mixer
    hands to the kernel table as it is.  ``shared`` is a per-step dict so that
    equal encodings in many layers are prepared once."""

    def layout(self):
        return None

    def tables(self, batch, shared):
        raise NotImplementedError


class Mixer(Part):
    """Sequence mixer.  ``takes_scaled_rows``: forward hands ``x`` to nothing but
    ``ops.linear`` / ``ops.gated_linear`` (same flag on FeedForward and the head).  ``cache_spec`` declares its per-request cache need
    (PagedKVSpec, StateSpec or None); ``forward(x, batch, cache, shared)`` maps
    normed rows [T, H] to rows [T, H].  ``cache`` is the binding the cache
    manager made for the layer call: pages plus block tables, or state plus
    slot ids; ``cache.write`` is False when the call reads another call's
    cache."""

    takes_scaled_rows = False

    def cache_spec(self):
        return None

    def forward(self, x, batch, cache, shared):
        raise NotImplementedError


class FeedForward(Part):
    """forward(x [T, H]) -> [T, H] (or a deferred product of that shape)."""

    takes_scaled_rows = False

    def forward(self, x):
        raise NotImplementedError


class Block(Part):
    """An arrangement of norms, mixers and a feed-forward around the residual
    stream.  ``cache_specs()`` lists what the block needs cached per request,
    one entry for each of its parts that caches (none, one, or several: an
    attention and a state mixer side by side have two); a layer call names one
    cache stream for each.  ``forward(resid, delta, batch, caches, shared) ->
    delta``: ``resid`` is the float32 stream (updated in place), ``delta`` the
    not yet added output of what ran before (None at the start), ``caches`` the
    bindings of the call's streams in the order of ``cache_specs()``."""

    def cache_specs(self):
        return []

    def forward(self, resid, delta, batch, caches, shared):
        raise NotImplementedError


class Embedding(Part):
    """forward(batch) -> the float32 residual stream [T, H] of the step's
    tokens.  The whole batch is at hand: ``batch.ids``, and ``batch.positions``
    for an embedding that adds a table of absolute positions."""

    def forward(self, batch):
        raise NotImplementedError

"""Typed model configuration, read from the architecture's own config.json keys.

Reference: ``ModelConfig.from_hf`` (servelab/config.py:48-72) reads the same
keys with the same defaults.  This build adds the sliding-window keys, a
per-key error for a missing required key (the reference raises a bare
KeyError) and validation of the sizes the kernels rely on.
"""
from dataclasses import dataclass, field, fields
from typing import Any, Dict, List, Optional


class ConfigError(ValueError):
    """config.json lacks a required key, or holds a value no model can have."""


# what the attention kernels take (csrc/attention.hip, MAX_D): a head's channels
# sit in the registers of one wavefront, 256 at most
MAX_HEAD_DIM = 256
# the layer kinds a ``layer_types`` list may name, and what they mean here
LAYER_KINDS = {"full_attention": False, "sliding_attention": True}


_MISSING = object()


def read_key(cfg: Dict[str, Any], key: str, default: Any = _MISSING, kind=None):
    """One config.json key; a required key that is absent names itself."""
    if key not in cfg or cfg[key] is None:
        if default is _MISSING:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    value = cfg[key]
    if kind is not None:
        try:
            if kind is int and isinstance(value, float) and value != int(value):
                raise ValueError
            value = kind(value)
        except (TypeError, ValueError):
            raise ConfigError(
                f"config.json: key '{key}' = {cfg[key]!r} is not a {kind.__name__}")
    return value


def refuse_rope_scaling(cfg: Dict[str, Any]) -> None:
    """The rotary angles here are position * theta^(-2j/D) and nothing else
    (servelab/parallel/tp_model.py:94-96; servelab/config.py:48-72 reads no
    scaling key).  A ``rope_scaling`` entry that asks for other angles (linear,
    dynamic, yarn, ...) is refused rather than dropped: the model would run, with
    other logits than its authors meant.  null and the type "default" ask for
    the plain angles and pass."""
    scaling = cfg.get("rope_scaling")
    if scaling is None:
        return
    kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
    if kind in (None, "default") and isinstance(scaling, dict) and \
            float(scaling.get("factor", 1.0) or 1.0) == 1.0:
        return
    raise ConfigError(f"config.json: rope_scaling = {scaling!r} is not supported: this engine "
                      f"computes plain rotary angles (no scaling of any kind)")


@dataclass
class Qwen2Config:
    """Qwen2 dense decoder (servelab/config.py:10-28 plus the window keys)."""

    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float = 1000000.0
    max_position_embeddings: int = 4096
    tie_word_embeddings: bool = False
    dtype: str = "float16"
    eos_token_id: int = 0
    attention_bias: bool = True
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: int = 0
    hidden_act: str = "silu"
    architecture: str = "Qwen2ForCausalLM"
    path: str = ""
    raw: Dict[str, Any] = field(default_factory=dict, repr=False, compare=False)

    # ------------------------------------------------------------ derived
    @property
    def num_query_groups(self) -> int:
        """servelab/config.py:30-32."""
        return self.num_heads // self.num_kv_heads

    def layer_window(self, layer_index: int) -> Optional[int]:
        """Window of a layer: windowed iff use_sliding_window and
        layer_index >= max_window_layers; None means all keys."""
        if self.use_sliding_window and self.sliding_window and \
                layer_index >= self.max_window_layers:
            return int(self.sliding_window)
        return None

    def num_params(self) -> int:
        """Exact parameter count (the reference's servelab/config.py:34-46
        counts q/k/v three times over)."""
        h, d = self.hidden_size, self.head_dim
        qkv_out = (self.num_heads + 2 * self.num_kv_heads) * d
        per_layer = (h * qkv_out + (qkv_out if self.attention_bias else 0)
                     + self.num_heads * d * h
                     + 3 * h * self.intermediate_size + 2 * h)
        n = self.num_layers * per_layer + h + self.vocab_size * h
        if not self.tie_word_embeddings:
            n += self.vocab_size * h
        return n

    # ------------------------------------------------------------ reading
    @classmethod
    def from_hf(cls, cfg: Dict[str, Any], path: str = "") -> "Qwen2Config":
        heads = read_key(cfg, "num_attention_heads", kind=int)
        hidden = read_key(cfg, "hidden_size", kind=int)
        if heads <= 0:
            raise ConfigError("config.json: num_attention_heads must be positive")
        eos = read_key(cfg, "eos_token_id", 0)
        if isinstance(eos, (list, tuple)):
            # servelab/engine/scheduler.py:336 compares with `==`; take the first
            eos = eos[0] if eos else 0
        archs = cfg.get("architectures") or ["Qwen2ForCausalLM"]
        refuse_rope_scaling(cfg)
        out = cls(
            hidden_size=hidden,
            num_layers=read_key(cfg, "num_hidden_layers", kind=int),
            num_heads=heads,
            num_kv_heads=read_key(cfg, "num_key_value_heads", heads, kind=int),
            head_dim=read_key(cfg, "head_dim", hidden // heads, kind=int),
            intermediate_size=read_key(cfg, "intermediate_size", kind=int),
            vocab_size=read_key(cfg, "vocab_size", kind=int),
            rms_norm_eps=read_key(cfg, "rms_norm_eps", kind=float),
            rope_theta=read_key(cfg, "rope_theta", 1000000.0, kind=float),
            max_position_embeddings=read_key(cfg, "max_position_embeddings", 4096, kind=int),
            tie_word_embeddings=bool(read_key(cfg, "tie_word_embeddings", False)),
            dtype=str(read_key(cfg, "torch_dtype", "float16")),
            eos_token_id=int(eos),
            attention_bias=bool(read_key(cfg, "attention_bias", True)),
            use_sliding_window=bool(read_key(cfg, "use_sliding_window", False)),
            sliding_window=read_key(cfg, "sliding_window", None, kind=int),
            max_window_layers=read_key(cfg, "max_window_layers", 0, kind=int),
            hidden_act=str(read_key(cfg, "hidden_act", "silu")),
            architecture=str(archs[0]),
            path=path,
            raw=dict(cfg),
        )
        out.validate()
        out.check_layer_types(cfg.get("layer_types"))
        return out

    def validate(self) -> None:
        problems: List[str] = []
        for name in ("hidden_size", "num_layers", "num_heads", "num_kv_heads",
                     "head_dim", "intermediate_size", "vocab_size",
                     "max_position_embeddings"):
            if getattr(self, name) <= 0:
                problems.append(f"{name} must be positive, is {getattr(self, name)}")
        if not problems:
            if self.num_heads % self.num_kv_heads:
                problems.append(
                    f"num_attention_heads {self.num_heads} is not a multiple of "
                    f"num_key_value_heads {self.num_kv_heads}")
            if self.head_dim % 2:
                problems.append(f"head_dim {self.head_dim} must be even for rotary pairs")
            if self.head_dim > MAX_HEAD_DIM:
                problems.append(
                    f"head_dim {self.head_dim} is more than the attention kernels take "
                    f"({MAX_HEAD_DIM}: a head's channels sit in one wavefront's registers)")
        if not self.rms_norm_eps > 0:
            problems.append(f"rms_norm_eps must be positive, is {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            problems.append(f"rope_theta must be positive, is {self.rope_theta}")
        if self.hidden_act != "silu":
            problems.append(f"hidden_act '{self.hidden_act}' is not supported (silu only)")
        if self.use_sliding_window and (self.sliding_window is None or self.sliding_window < 1):
            problems.append("use_sliding_window needs sliding_window >= 1")
        if self.dtype not in ("float16", "bfloat16", "float32"):
            problems.append(f"torch_dtype '{self.dtype}' is not float16|bfloat16|float32")
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))

    def check_layer_types(self, layer_types) -> None:
        """A ``layer_types`` list in config.json must say, layer by layer, what
        ``use_sliding_window`` / ``max_window_layers`` say: the window of a layer
        is computed from those keys, and a list that contradicts them names
        another model than the one that would be served."""
        if layer_types is None:
            return
        if not isinstance(layer_types, (list, tuple)) or len(layer_types) != self.num_layers:
            raise ConfigError(
                f"config.json: layer_types must list {self.num_layers} layers, is {layer_types!r}")
        for i, kind in enumerate(layer_types):
            if kind not in LAYER_KINDS:
                raise ConfigError(f"config.json: layer_types[{i}] = {kind!r} is not one of "
                                  f"{sorted(LAYER_KINDS)}")
            windowed = self.layer_window(i) is not None
            if LAYER_KINDS[kind] != windowed:
                raise ConfigError(
                    f"config.json: layer_types[{i}] = {kind!r} contradicts use_sliding_window="
                    f"{self.use_sliding_window}, sliding_window={self.sliding_window}, "
                    f"max_window_layers={self.max_window_layers}, by which layer {i} "
                    f"{'has a window' if windowed else 'sees all keys'}")

    def to_hf(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        return {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "torch_dtype": self.dtype,
            "eos_token_id": self.eos_token_id,
            "attention_bias": self.attention_bias,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
            "hidden_act": self.hidden_act,
        }

    def replace(self, **changes) -> "Qwen2Config":
        values = {f.name: getattr(self, f.name) for f in fields(self)}
        values.update(changes)
        return Qwen2Config(**values)

"""How a request's tokens are drawn.  Field names, meanings and defaults are
the reference's (servelab/engine/sampling_params.py:6-14); every field is
checked at construction and all faults are reported in one message."""
from dataclasses import dataclass
from typing import Tuple


@dataclass
class SamplingParams:
    temperature: float = 1.0           # 0 => greedy
    top_p: float = 1.0                 # in (0, 1]
    top_k: int = -1                    # -1: off, else >= 1 (top_p is then ignored, as in the reference)
    max_tokens: int = 16
    ignore_eos: bool = False
    seed: int = -1                     # -1: drawn from the engine's seed and the request's number
    stop_token_ids: Tuple[int, ...] = ()

    def __post_init__(self):
        self.stop_token_ids = tuple(int(t) for t in self.stop_token_ids)
        faults = [f"{name}={value!r} ({rule})" for name, value, ok, rule in (
            ("temperature", self.temperature, self.temperature >= 0.0, "negative"),
            ("top_p", self.top_p, 0.0 < self.top_p <= 1.0, "outside (0, 1]"),
            ("top_k", self.top_k, self.top_k == -1 or self.top_k >= 1, "neither -1 nor positive"),
            ("max_tokens", self.max_tokens, self.max_tokens >= 1, "below 1"),
        ) if not ok]
        if faults:
            raise ValueError("SamplingParams: " + "; ".join(faults))

    @staticmethod
    def greedy(max_tokens: int = 16) -> "SamplingParams":
        return SamplingParams(temperature=0.0, max_tokens=max_tokens)

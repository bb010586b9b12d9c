"""Result records (servelab/engine/output.py:9-41): the field names callers of
the reference read."""
from dataclasses import dataclass, field
from typing import Callable, List, Optional


@dataclass
class CompletionOutput:
    index: int = 0
    text: str = ""
    token_ids: List[int] = field(default_factory=list)
    finish_reason: Optional[str] = None     # "eos" | "length" | "aborted"


@dataclass
class RequestOutput:
    request_id: str
    prompt: str = ""
    prompt_token_ids: List[int] = field(default_factory=list)
    outputs: List[CompletionOutput] = field(default_factory=list)
    finished: bool = False
    metrics: Optional[dict] = None


def result_of(req, to_text: Optional[Callable[[List[int]], str]] = None) -> RequestOutput:
    """The record of a request as it stands (usually: finished)."""
    generated = list(req.output)
    completion = CompletionOutput(token_ids=generated, finish_reason=req.finish_reason,
                                  text=to_text(generated) if to_text else "")
    return RequestOutput(req.request_id, prompt_token_ids=list(req.prompt), outputs=[completion],
                         finished=req.done, metrics=req.times.report())

"""One request as the engine sees it between steps (no tensors).

A request is three things: what was *asked* (prompt ids, sampling parameters,
priority, when and in which order it came), what it *holds* (its tokens so far,
and how many of them the cache has keys and values for) and what it is *owed*
(the tokens that must still run before its next token can be sampled).  A
request whose cache is complete but for its newest token is owed one token, a
decode step; a fresh prompt, or a request that lost its cache to a preemption,
is owed everything it holds and gets it in portions.  The scheduler plans from
``owed`` alone, so a rebuilt request needs no special case and its outputs are
never mistaken for prompt.

Reference: ``Sequence`` (servelab/engine/sequence.py:52-113) keeps a prompt
count that a preemption overwrites (:102-109), which loses the tokens generated
before it; the reference's status names survive only as finish reasons
("eos" | "length" | "aborted", servelab/engine/output.py:14).
"""
from dataclasses import dataclass
from typing import List, Optional

from .sampling_params import SamplingParams

QUEUED, ACTIVE, DONE = "queued", "active", "done"


@dataclass
class Timeline:
    """When things happened to a request, on the engine's clock."""
    arrived: float = 0.0
    admitted: Optional[float] = None
    first_token: Optional[float] = None
    finished: Optional[float] = None
    preemptions: int = 0

    def report(self) -> dict:
        """The figures a caller gets with the result (servelab/engine/sequence.py:36-48)."""
        end = self.finished if self.finished is not None else self.arrived
        first = self.first_token if self.first_token is not None else end
        return {"ttft": first - self.arrived, "latency": end - self.arrived,
                "preemptions": self.preemptions}


class Request:
    def __init__(self, request_id: str, prompt_token_ids: List[int], params: SamplingParams,
                 priority: int = 0, arrived: float = 0.0, number: int = 0):
        if len(prompt_token_ids) < 1:
            raise ValueError("a request needs at least one prompt token")
        # asked
        self.request_id = request_id
        self.params = params
        self.priority = priority
        self.number = number                  # order of submission: breaks ties, keys the random stream
        self.prompt_len = len(prompt_token_ids)
        # held
        self.tokens: List[int] = [int(t) for t in prompt_token_ids]
        self.cached = 0                       # tokens whose keys and values are in the cache
        self.phase = QUEUED
        self.finish_reason: Optional[str] = None
        self.times = Timeline(arrived=arrived)

    # ------------------------------------------------------------- views
    @property
    def prompt(self) -> List[int]:
        return self.tokens[:self.prompt_len]

    @property
    def output(self) -> List[int]:
        return self.tokens[self.prompt_len:]

    @property
    def num_output(self) -> int:
        return len(self.tokens) - self.prompt_len

    @property
    def owed(self) -> int:
        """Tokens that must run before the next token can be sampled (>= 1
        while the request is unfinished)."""
        return len(self.tokens) - self.cached

    @property
    def decoding(self) -> bool:
        """Owed exactly its newest token, with everything before it cached."""
        return self.cached > 0 and self.owed == 1

    @property
    def done(self) -> bool:
        return self.phase == DONE

    # ----------------------------------------------------------- changes
    def ran(self, count: int) -> bool:
        """``count`` more tokens were run and cached; True when nothing is owed
        any more, that is when this step's last logits are the request's next
        token."""
        if not 0 < count <= self.owed:
            raise ValueError(f"{self.request_id}: ran {count} tokens, owed {self.owed}")
        self.cached += count
        return self.cached == len(self.tokens)

    def sampled(self, token: int, now: float) -> None:
        if self.cached != len(self.tokens):
            raise ValueError(f"{self.request_id}: sampled while {self.owed} tokens are owed")
        self.tokens.append(int(token))
        if self.times.first_token is None:
            self.times.first_token = now

    def lost_cache(self) -> None:
        """A preemption took the pages: everything held is owed again."""
        self.cached = 0
        self.phase = QUEUED
        self.times.preemptions += 1

    def finish(self, reason: str, now: float) -> None:
        self.phase, self.finish_reason = DONE, reason
        self.times.finished = now

    def __repr__(self) -> str:
        return (f"Request({self.request_id}, {len(self.tokens)} tokens, {self.cached} cached, "
                f"{self.finish_reason or self.phase})")

"""Continuous batching with chunked prefill and recompute preemption (no tensors).

Reference: ``Scheduler`` (servelab/engine/scheduler.py:107-369).  One pass per
step under a token budget: first one decode token for every running request
whose prompt is cached (:176-188), then the next portion of prompts that are
part-way (:190-198), then admission from the waiting queue in policy order
until a request does not fit (:201-241).  Pages are reserved while planning.

What happens when pages run out (reference :276-316, with these decisions):
  * a running request that cannot grow takes the pages of the request that the
    policy would schedule last and that has nothing planned in this step; the
    victim's cache is dropped, it returns to the front of the waiting queue and
    is computed again from its first token (generated tokens included).  The
    reference preempts one victim and leaves the failing request out of the
    step; here the request tries again until it fits or no victim is left.
  * with no victim left the request preempts itself.
  * a waiting request never evicts a running one: admission simply stops
    (head-of-line blocking, reference :231-237).
  * a request that could not fit in the whole pool, or is longer than the
    model's positions, is aborted at admission (reference :211-215) and — unlike
    there — is reported with finish reason "aborted".
"""
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional

from ..config import SchedulerConfig
from .sequence import Sequence, SequenceStatus


# ------------------------------------------------------------------ policies
def fcfs_key(seq: Sequence):
    """First come first served (servelab/engine/scheduler.py:37-41); ties by
    submission number rather than by the id string."""
    return (seq.arrival_time, seq.number)


def priority_key(seq: Sequence):
    """Smaller priority value first (servelab/engine/scheduler.py:44-48)."""
    return (seq.priority, seq.arrival_time, seq.number)


POLICIES = {"fcfs": fcfs_key, "priority": priority_key}


@dataclass
class PrefillSched:
    seq: Sequence
    num_new_tokens: int          # portion size
    num_computed: int            # tokens cached before this portion


@dataclass
class SchedulerOutput:
    prefills: List[PrefillSched] = field(default_factory=list)
    decodes: List[Sequence] = field(default_factory=list)
    preempted: List[str] = field(default_factory=list)
    aborted: List[Sequence] = field(default_factory=list)

    def is_empty(self) -> bool:
        return not self.prefills and not self.decodes

    @property
    def num_batched_tokens(self) -> int:
        return sum(p.num_new_tokens for p in self.prefills) + len(self.decodes)

    def planned_ids(self):
        return {p.seq.request_id for p in self.prefills} | {s.request_id for s in self.decodes}


class Scheduler:
    def __init__(self, config: SchedulerConfig, manager, clock: Callable[[], float],
                 eos_token_id: int = -1, max_positions: Optional[int] = None):
        self.cfg = config
        self.manager = manager
        self.clock = clock
        self.eos_token_id = eos_token_id
        self.max_positions = max_positions
        self.key = POLICIES[config.policy]
        self.waiting: List[Sequence] = []
        self.running: List[Sequence] = []
        self.num_preemptions = 0

    # -------------------------------------------------------------- intake
    def add_request(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def abort_request(self, request_id: str) -> bool:
        """servelab/engine/scheduler.py:132-144."""
        for queue in (self.waiting, self.running):
            for i, s in enumerate(queue):
                if s.request_id == request_id:
                    queue.pop(i)
                    self.manager.close(request_id)
                    s.status = SequenceStatus.FINISHED_ABORTED
                    return True
        return False

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------ schedule
    def schedule(self) -> SchedulerOutput:
        now = self.clock()
        out = SchedulerOutput()
        budget = self.cfg.max_num_batched_tokens

        # 1) one token for every running request whose prompt is cached
        if self.cfg.chunked_prefill or not self.waiting:
            for seq in list(self.running):
                if not seq.is_prefill_done():
                    continue
                if len(out.decodes) >= self.cfg.max_num_seqs or budget < 1:
                    break
                if seq not in self.running:
                    continue                     # preempted earlier in this pass
                if self._reserve(seq, seq.num_computed_tokens + 1, out):
                    out.decodes.append(seq)
                    budget -= 1

        # 2) prompts that are part-way, in policy order
        for seq in sorted((s for s in self.running if not s.is_prefill_done()), key=self.key):
            if budget <= 0:
                break
            if seq not in self.running:
                continue
            chunk = self._portion(seq, budget)
            if self._reserve(seq, seq.num_computed_tokens + chunk, out):
                out.prefills.append(PrefillSched(seq, chunk, seq.num_computed_tokens))
                budget -= chunk

        # 3) admission
        self.waiting.sort(key=self.key)
        while self.waiting and len(self.running) < self.cfg.max_num_seqs and budget > 0:
            seq = self.waiting[0]
            too_long = self.max_positions is not None and seq.get_len() > self.max_positions
            if too_long or not self.manager.can_ever_hold(seq.get_len()):
                self.waiting.pop(0)
                seq.status = SequenceStatus.FINISHED_ABORTED
                seq.metrics.finished_time = now
                out.aborted.append(seq)
                continue
            if not self.manager.open(seq.request_id):
                break                            # no state slot free
            chunk = self._portion(seq, budget)
            if not self.manager.grow(seq.request_id, seq.num_computed_tokens + chunk):
                self.manager.close(seq.request_id)
                break                            # head-of-line blocking
            seq.metrics.first_scheduled_time = seq.metrics.first_scheduled_time or now
            self.waiting.pop(0)
            seq.status = SequenceStatus.RUNNING
            self.running.append(seq)
            out.prefills.append(PrefillSched(seq, chunk, seq.num_computed_tokens))
            budget -= chunk
        return out

    # ------------------------------------------------------------- helpers
    def _portion(self, seq: Sequence, budget: int) -> int:
        """Next portion of a prompt: what the budget leaves, at least one token;
        the whole rest when chunking is off (servelab/engine/scheduler.py:254-258)."""
        remaining = seq.remaining_prefill_tokens()
        if self.cfg.chunked_prefill:
            return max(1, min(remaining, budget))
        return max(1, remaining)

    def _reserve(self, seq: Sequence, total_tokens: int, out: SchedulerOutput) -> bool:
        """Pages for ``total_tokens`` of a running request, preempting others
        while none are free.  False when the request itself had to go."""
        while not self.manager.grow(seq.request_id, total_tokens):
            planned = out.planned_ids()
            victim = None
            for cand in sorted(self.running, key=self.key, reverse=True):
                if cand is not seq and cand.request_id not in planned:
                    victim = cand
                    break
            if victim is None:
                self._preempt(seq, out)
                return False
            self._preempt(victim, out)
        return True

    def _preempt(self, seq: Sequence, out: SchedulerOutput) -> None:
        """Recompute preemption (servelab/engine/scheduler.py:300-316)."""
        self.running.remove(seq)
        self.manager.close(seq.request_id)
        seq.on_preempt_recompute()
        self.waiting.insert(0, seq)
        out.preempted.append(seq.request_id)
        self.num_preemptions += 1

    # ------------------------------------------------------ after the step
    def update_after_exec(self, sampled: Dict[str, int], now: Optional[float] = None) -> List[Sequence]:
        """Append sampled tokens, apply the stop conditions, free what finished
        (servelab/engine/scheduler.py:319-349).  Returns the requests that
        finished in this step."""
        now = self.clock() if now is None else now
        by_id = {s.request_id: s for s in self.running}
        finished: List[Sequence] = []
        for request_id, token in sampled.items():
            seq = by_id.get(request_id)
            if seq is None:
                continue
            seq.append_token(token)
            if seq.metrics.first_token_time == 0.0:
                seq.metrics.first_token_time = now
            sp = seq.sampling_params
            is_stop = token == self.eos_token_id or token in sp.stop_token_ids
            if is_stop and not sp.ignore_eos:
                seq.status = SequenceStatus.FINISHED_EOS          # the stop token stays in the output
            elif seq.num_output_tokens >= sp.max_tokens:
                seq.status = SequenceStatus.FINISHED_LENGTH
            elif self.max_positions is not None and seq.get_len() >= self.max_positions:
                seq.status = SequenceStatus.FINISHED_LENGTH       # no position left for another token
            if seq.is_finished():
                finished.append(seq)
        for seq in finished:
            self.running.remove(seq)
            self.manager.close(seq.request_id)
            seq.metrics.finished_time = now
        return finished

    def stats(self) -> dict:
        """servelab/engine/scheduler.py:358-369, without the prefix cache."""
        return {"waiting": len(self.waiting), "running": len(self.running),
                "gpu_cache_usage": round(self.manager.usage(), 4),
                "num_preemptions_total": self.num_preemptions}

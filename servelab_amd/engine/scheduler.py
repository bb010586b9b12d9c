"""Continuous batching with chunked prefill and recompute preemption (no tensors).

Reference: ``Scheduler`` (servelab/engine/scheduler.py:107-369).  One pass per
step under a token budget: one token for every active request that is owed
only its newest token (:176-188), then the next portion of requests that are
owed more (:190-198), then admission from the queue in policy order until a
request does not fit (:201-241).  Pages are reserved while planning, and the
scheduler itself books the outcome of the step (``complete``): how much more
of each request is cached, the sampled tokens, who is finished.

What happens when pages run out (reference :276-316, with these decisions):
  * an active request that cannot grow takes the pages of the request that the
    policy would schedule last and that has nothing planned in this step; the
    victim's cache is dropped, it returns to the front of the queue and is owed
    everything it holds (generated tokens included).  The reference preempts
    one victim and leaves the failing request out of the step; here the request
    tries again until it fits or no victim is left.
  * with no victim left the request preempts itself.
  * a queued request never evicts an active one: admission simply stops
    (head-of-line blocking, reference :231-237).
  * a request that could not fit in the whole pool, or is longer than the
    model's positions, is aborted at admission (reference :211-215) and — unlike
    there — is reported with finish reason "aborted".
  * with ``chunked_prefill`` off, whole prompts go before decode tokens
    (reference :177), but only while a prompt can in fact be admitted: when
    every slot is taken or the head of the queue does not fit, the active
    requests decode on, which is what frees the room.  (The reference plans
    nothing in that case and stops for good.)
"""
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional

from ..config import SchedulerConfig
from .request import ACTIVE, QUEUED, Request


# ------------------------------------------------------------------ policies
def fcfs_key(req: Request):
    """First come first served (servelab/engine/scheduler.py:37-41); ties by
    submission number rather than by the id string."""
    return (req.times.arrived, req.number)


def priority_key(req: Request):
    """Smaller priority value first (servelab/engine/scheduler.py:44-48)."""
    return (req.priority, req.times.arrived, req.number)


def shortest_predicted_key(predictor):
    """Fewest predicted tokens still to come first (servelab/engine/scheduler.py:51-70).
    ``predictor.predict_remaining(request)`` says how many tokens the request
    will generate in all (servelab/engine/scheduler.py:19-22); what it has
    generated already is taken off, also for a request that lost its cache
    to a preemption and keeps its tokens (the reference takes it off only
    once the prompt has run, and forgets it after a preemption)."""
    def key(req: Request):
        remaining = int(predictor.predict_remaining(req)) - req.num_output
        return (max(1, remaining), req.times.arrived, req.number)
    return key


POLICIES = {"fcfs": fcfs_key, "priority": priority_key}
PREDICTED_POLICY = "sjf-predicted"


def policy_key(name: str, predictor=None):
    """The sort key of a policy by name (servelab/engine/scheduler.py:74-83)."""
    if name == PREDICTED_POLICY:
        if predictor is None:
            raise ValueError("sjf-predicted policy requires an output-length predictor")
        return shortest_predicted_key(predictor)
    if name not in POLICIES:
        raise ValueError(f"unknown scheduler policy: {name}")
    return POLICIES[name]


@dataclass
class Planned:
    """``count`` tokens of ``request`` from position ``start`` on run in this step."""
    request: Request
    start: int
    count: int

    @property
    def samples(self) -> bool:
        """Whether the step's last logits of this request are its next token."""
        return self.start + self.count == len(self.request.tokens)

    @property
    def token_ids(self) -> List[int]:
        return self.request.tokens[self.start:self.start + self.count]


@dataclass
class Plan:
    portions: List[Planned] = field(default_factory=list)     # requests owed more than a token
    decodes: List[Planned] = field(default_factory=list)      # one token each
    preempted: List[str] = field(default_factory=list)
    aborted: List[Request] = field(default_factory=list)

    def is_empty(self) -> bool:
        return not self.portions and not self.decodes

    @property
    def num_tokens(self) -> int:
        return sum(p.count for p in self.portions) + len(self.decodes)

    def items(self) -> List[Planned]:
        """Everything that runs, in the order the step function wants it."""
        return self.portions + self.decodes

    def planned_ids(self):
        return {p.request.request_id for p in self.items()}


class Scheduler:
    def __init__(self, config: SchedulerConfig, manager, clock: Callable[[], float],
                 eos_token_id: int = -1, max_positions: Optional[int] = None, predictor=None):
        self.cfg = config
        self.manager = manager
        self.clock = clock
        self.eos_token_id = eos_token_id
        self.max_positions = max_positions
        self.key = policy_key(config.policy, predictor)
        self.queue: List[Request] = []
        self.active: List[Request] = []
        self.num_preemptions = 0

    # -------------------------------------------------------------- intake
    def add_request(self, req: Request) -> None:
        self.queue.append(req)

    def abort_request(self, request_id: str) -> Optional[Request]:
        """servelab/engine/scheduler.py:132-144; the aborted request, or None
        when no unfinished request has that id."""
        for held in (self.queue, self.active):
            for i, r in enumerate(held):
                if r.request_id == request_id:
                    held.pop(i)
                    self.manager.close(request_id)
                    r.finish("aborted", self.clock())
                    return r
        return None

    def has_unfinished(self) -> bool:
        return bool(self.queue or self.active)

    # ------------------------------------------------------------ schedule
    def schedule(self) -> Plan:
        now = self.clock()
        plan = Plan()
        budget = self.cfg.max_num_batched_tokens
        prompts_first = not self.cfg.chunked_prefill and bool(self.queue)
        if not prompts_first:
            budget = self._plan_decodes(plan, budget)
        budget = self._plan_portions(plan, budget)
        budget = self._admit(plan, budget, now)
        if prompts_first and not plan.portions:
            self._plan_decodes(plan, budget)
        return plan

    def _plan_decodes(self, plan: Plan, budget: int) -> int:
        for req in list(self.active):
            if not req.decoding:
                continue
            if len(plan.decodes) >= self.cfg.max_num_seqs or budget < 1:
                break
            if req.phase != ACTIVE:
                continue                         # preempted earlier in this pass
            if self._reserve(req, req.cached + 1, plan):
                plan.decodes.append(Planned(req, req.cached, 1))
                budget -= 1
        return budget

    def _plan_portions(self, plan: Plan, budget: int) -> int:
        for req in sorted((r for r in self.active if not r.decoding), key=self.key):
            if budget <= 0:
                break
            if req.phase != ACTIVE:
                continue
            count = self._portion(req, budget)
            if self._reserve(req, req.cached + count, plan):
                plan.portions.append(Planned(req, req.cached, count))
                budget -= count
        return budget

    def _admit(self, plan: Plan, budget: int, now: float) -> int:
        self.queue.sort(key=self.key)
        while self.queue and len(self.active) < self.cfg.max_num_seqs and budget > 0:
            req = self.queue[0]
            too_long = self.max_positions is not None and len(req.tokens) > self.max_positions
            if too_long or not self.manager.can_ever_hold(len(req.tokens)):
                self.queue.pop(0)
                req.finish("aborted", now)
                plan.aborted.append(req)
                continue
            if not self.manager.open(req.request_id):
                break                            # no state slot free
            count = self._portion(req, budget)
            if not self.manager.grow(req.request_id, req.cached + count):
                self.manager.close(req.request_id)
                break                            # head-of-line blocking
            if req.times.admitted is None:
                req.times.admitted = now
            self.queue.pop(0)
            req.phase = ACTIVE
            self.active.append(req)
            plan.portions.append(Planned(req, req.cached, count))
            budget -= count
        return budget

    def plan_ahead(self, plan: Plan) -> Optional[Plan]:
        """The step after ``plan``, planned while ``plan`` still runs and its
        sampled tokens are not known: one more token for every request of
        ``plan`` that cannot end with this step by its length.  Possible only
        when ``plan`` samples for every active request and the step after it
        would be exactly this one, unless a stop token ends a request (its row
        of the step ahead is then wasted and ignored).  That holds when nothing
        waits for admission, and also under a standing queue as long as nobody
        can be admitted in the next step: every slot is taken and stays taken,
        the token budget is used up by the decode tokens, or the head of the
        queue does not fit the pages that the step ahead leaves free.  Pages
        are reserved; None when the step cannot be planned ahead.  ``complete``
        must see ``plan`` before the plan ahead."""
        if not plan.items() or len(plan.items()) != len(self.active):
            return None
        if not all(item.samples and item.request.phase == ACTIVE for item in plan.items()):
            return None
        ahead = Plan()
        for item in plan.items():
            req = item.request
            length = len(req.tokens) + 1                      # once this step's token is appended
            if req.num_output + 1 >= req.params.max_tokens:
                continue                                      # ends with this step
            if self.max_positions is not None and length >= self.max_positions:
                continue
            ahead.decodes.append(Planned(req, item.start + item.count, 1))
        if not ahead.decodes or len(ahead.decodes) > self.cfg.max_num_batched_tokens:
            return None
        if self.queue and len(ahead.decodes) < len(plan.items()):
            return None                                       # a request ends: its slot and pages go to the queue
        for item in ahead.decodes:
            if not self.manager.grow(item.request.request_id, item.start + 1):
                return None                                   # (pages taken so far stay with their requests)
        if self.queue and self._could_admit(len(ahead.decodes)):
            return None                                       # (likewise: the next step asks for the same pages)
        return ahead

    def _could_admit(self, decodes: int) -> bool:
        """Whether the next ``schedule`` would take (or abort) the head of the
        queue beside ``decodes`` decode tokens, as the pool stands now."""
        budget = self.cfg.max_num_batched_tokens - decodes
        if len(self.active) >= self.cfg.max_num_seqs or budget <= 0:
            return False
        head = min(self.queue, key=self.key)
        too_long = self.max_positions is not None and len(head.tokens) > self.max_positions
        if too_long or not self.manager.can_ever_hold(len(head.tokens)):
            return True                                       # it is aborted there, and the next one is looked at
        return self.manager.can_admit(head.cached + self._portion(head, budget))

    # ------------------------------------------------------------- helpers
    def _portion(self, req: Request, budget: int) -> int:
        """Next portion of what a request is owed: what the budget leaves, at
        least one token; all of it when chunking is off
        (servelab/engine/scheduler.py:254-258)."""
        if self.cfg.chunked_prefill:
            return max(1, min(req.owed, budget))
        return req.owed

    def _reserve(self, req: Request, total_tokens: int, plan: Plan) -> bool:
        """Pages for ``total_tokens`` of an active request, preempting others
        while none are free.  False when the request itself had to go."""
        while not self.manager.grow(req.request_id, total_tokens):
            planned = plan.planned_ids()
            victim = None
            for cand in sorted(self.active, key=self.key, reverse=True):
                if cand is not req and cand.request_id not in planned:
                    victim = cand
                    break
            if victim is None:
                self._preempt(req, plan)
                return False
            self._preempt(victim, plan)
        return True

    def _preempt(self, req: Request, plan: Plan) -> None:
        """Recompute preemption (servelab/engine/scheduler.py:300-316)."""
        self.active.remove(req)
        self.manager.close(req.request_id)
        req.lost_cache()
        self.queue.insert(0, req)
        plan.preempted.append(req.request_id)
        self.num_preemptions += 1

    # ------------------------------------------------------ after the step
    def complete(self, plan: Plan, sampled: Dict[str, int],
                 now: Optional[float] = None) -> List[Request]:
        """Book a step that ran ``plan``: every planned request has that much
        more cached; those whose step ended at their newest token take their
        sampled token from ``sampled`` and meet the stop conditions
        (servelab/engine/scheduler.py:319-349).  Returns the requests that
        finished in this step; their pages are free again."""
        now = self.clock() if now is None else now
        finished: List[Request] = []
        for item in plan.items():
            req = item.request
            if req.phase != ACTIVE:
                continue                         # aborted while the step ran
            if not req.ran(item.count):
                continue
            token = int(sampled[req.request_id])
            req.sampled(token, now)
            sp = req.params
            stops = token == self.eos_token_id or token in sp.stop_token_ids
            if stops and not sp.ignore_eos:
                req.finish("eos", now)           # the stop token stays in the output
            elif req.num_output >= sp.max_tokens:
                req.finish("length", now)
            elif self.max_positions is not None and len(req.tokens) >= self.max_positions:
                req.finish("length", now)        # no position left for another token
            if req.done:
                finished.append(req)
        for req in finished:
            self.active.remove(req)
            self.manager.close(req.request_id)
        return finished

    def stats(self) -> dict:
        """servelab/engine/scheduler.py:358-369, without the prefix cache."""
        return {"waiting": len(self.queue), "running": len(self.active),
                "gpu_cache_usage": round(self.manager.usage(), 4),
                "num_preemptions_total": self.num_preemptions}

"""Scheduler decisions with a fake executor and a fake clock (no GPU), after
the reference's tests/test_scheduler.py:29-154."""
import pytest

from servelab_amd.cache import CacheManager
from servelab_amd.config import SchedulerConfig
from servelab_amd.engine import Request, SamplingParams, Scheduler
from servelab_amd.parts import PagedKVSpec


class FakeClock:
    def __init__(self):
        self.t = 0.0

    def __call__(self):
        return self.t


class Driver:
    """Executes whatever the scheduler plans: advances the computed counts,
    'samples' token 7, and checks the invariants after every step."""

    def __init__(self, num_pages=16, page_size=4, max_batched=32, max_seqs=8, policy="fcfs",
                 chunked=True, eos=-1, max_positions=None, window=None, predictor=None):
        self.clock = FakeClock()
        specs = {0: PagedKVSpec(1, 16, None)}
        if window:
            specs[1] = PagedKVSpec(1, 16, window)
        self.manager = CacheManager(specs, num_pages, page_size, num_state_slots=max_seqs)
        self.scheduler = Scheduler(
            SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=max_batched,
                            chunked_prefill=chunked, policy=policy),
            self.manager, self.clock, eos_token_id=eos, max_positions=max_positions, predictor=predictor)
        self.finished, self.aborted, self.n, self.plans = [], [], 0, []
        self.token = 7

    def submit(self, rid, prompt_len, output_len, priority=0, ignore_eos=True):
        self.n += 1
        req = Request(rid, list(range(1000, 1000 + prompt_len)),
                      SamplingParams(max_tokens=output_len, ignore_eos=ignore_eos),
                      priority=priority, arrived=self.clock.t, number=self.n)
        self.scheduler.add_request(req)
        return req

    def step(self):
        out = self.scheduler.schedule()
        self.plans.append(out)
        sampled = {}
        assert out.num_tokens <= max(self.scheduler.cfg.max_num_batched_tokens, 1) \
            or not self.scheduler.cfg.chunked_prefill
        for item in out.items():
            assert item.start == item.request.cached and 1 <= item.count <= item.request.owed
            self.manager.commit(item.request.request_id, item.start + item.count)
            if item.samples:
                sampled[item.request.request_id] = self.token
        assert all(d.count == 1 and d.samples for d in out.decodes)
        self.clock.t += 0.01
        self.finished += self.scheduler.complete(out, sampled)
        self.aborted += out.aborted
        self.manager.check()
        # servelab's invariant (tests/test_engine_smoke.py:113-127): between steps an active
        # request has everything cached but what it is owed, and it is owed at least a token
        for r in self.scheduler.active:
            assert r.owed >= 1 and self.manager.lengths[r.request_id] == r.cached
        assert set(self.manager.lengths) == {r.request_id for r in self.scheduler.active}
        return out

    def run(self, max_steps=2000):
        steps = 0
        while self.scheduler.has_unfinished():
            steps += 1
            assert steps < max_steps, "scheduler makes no progress"
            out = self.step()
            assert not out.is_empty() or out.aborted
        assert self.manager.num_free_pages() == self.manager.num_pages
        return steps


def test_all_finish_with_exact_counts():
    d = Driver()
    for i in range(5):
        d.submit(f"r{i}", 10, 5)
    d.run()
    assert {s.request_id: s.num_output for s in d.finished} == {f"r{i}": 5 for i in range(5)}
    assert all(s.finish_reason == "length" for s in d.finished)


def test_portions_respect_the_budget():
    d = Driver(max_batched=8)
    d.submit("big", 40, 1)
    out = d.scheduler.schedule()
    assert len(out.portions) == 1 and out.portions[0].count == 8
    assert out.portions[0].start == 0


def test_decodes_first_then_portions_share_the_budget():
    d = Driver(max_batched=16, num_pages=64)
    d.submit("a", 6, 4)
    d.step()                               # a: whole prompt, first token sampled
    d.submit("b", 40, 2)
    out = d.step()
    assert [d.request.request_id for d in out.decodes] == ["a"]
    assert out.portions[0].request.request_id == "b" and out.portions[0].count == 15
    out = d.step()
    assert out.portions[0].start == 15 and out.portions[0].count == 15


def test_several_prompts_are_cut_in_one_step():
    d = Driver(max_batched=20, num_pages=64)
    d.submit("a", 12, 1)
    d.submit("b", 12, 1)
    out = d.scheduler.schedule()
    assert [(p.request.request_id, p.count) for p in out.portions] == [("a", 12), ("b", 8)]


def test_fcfs_and_priority_order():
    d = Driver(max_batched=12)
    for i in range(4):
        d.submit(f"r{i}", 20, 1)
    assert d.scheduler.schedule().portions[0].request.request_id == "r0"
    d = Driver(max_batched=12, policy="priority")
    d.submit("low", 20, 1, priority=5)
    d.submit("high", 20, 1, priority=0)
    assert d.scheduler.schedule().portions[0].request.request_id == "high"


class KnowsTheLength:
    """The predictor of the policy "sjf-predicted": here it knows what each request asks for."""

    def predict_remaining(self, req):
        return req.params.max_tokens


def test_shortest_predicted_job_first():
    # servelab/engine/scheduler.py:51-70,79-81
    with pytest.raises(ValueError, match="requires an output-length predictor"):
        Driver(policy="sjf-predicted")
    with pytest.raises(ValueError, match="unknown scheduler policy"):
        SchedulerConfig(policy="shortest")
    d = Driver(max_batched=8, max_seqs=2, policy="sjf-predicted", predictor=KnowsTheLength())
    d.submit("long", 8, 9)
    d.submit("short", 8, 2)
    d.submit("middle", 8, 5)
    # admission: the shortest predicted output first, whatever the order of arrival
    assert [p.request.request_id for p in d.step().portions] == ["short"]
    assert [p.request.request_id for p in d.step().portions] == ["middle"]
    d.step()
    d.step()
    # what a request has generated counts off its prediction: "middle" (5 predicted, 2 made) now goes
    # before a fresh request that predicts 4, and the victim of a preemption is the one with most to come
    key = d.scheduler.key
    middle = next(r for r in d.scheduler.active if r.request_id == "middle")
    fresh = Request("fresh", [1, 2], SamplingParams(max_tokens=4), arrived=d.clock.t, number=99)
    assert middle.num_output == 2 and key(middle) < key(fresh)
    d.run()
    assert [r.request_id for r in d.finished] == ["short", "middle", "long"]
    # equal predictions: first come first served; a prediction at or below what is made counts as 1
    a = Request("a", [1], SamplingParams(max_tokens=3), arrived=1.0, number=1)
    b = Request("b", [1], SamplingParams(max_tokens=3), arrived=0.5, number=2)
    assert key(b) < key(a)
    a.cached = 1
    for _ in range(5):
        a.sampled(7, 2.0)
        a.cached += 1
    assert key(a)[0] == 1


def test_request_numbers_not_id_strings_break_ties():
    d = Driver(max_batched=4)
    d.submit("req-10", 4, 1)
    d.submit("req-2", 4, 1)
    assert d.scheduler.schedule().portions[0].request.request_id == "req-10"


def test_preemption_when_pages_run_out():
    # 8 pages of 4 tokens; four requests need 18 tokens each
    d = Driver(num_pages=8, page_size=4, max_batched=64, max_seqs=4)
    seqs = [d.submit(f"r{i}", 8, 10) for i in range(4)]
    d.run()
    assert len(d.finished) == 4
    assert sum(s.times.preemptions for s in d.finished) > 0
    # outputs survive a preemption: ten tokens each, the prompt untouched
    assert all(s.num_output == 10 and s.prompt_len == 8 for s in seqs)
    # the victim is the request that came last, and it goes to the front of the queue
    first = next(p for p in d.plans if p.preempted)
    assert first.preempted[0] == "r3" or first.preempted[0] == "r2"


def test_the_victim_is_the_last_in_policy_order_and_requeues_first():
    d = Driver(num_pages=4, page_size=4, max_batched=64, max_seqs=4)
    a = d.submit("a", 7, 8)
    b = d.submit("b", 7, 8)
    d.step()                         # both prompts (2 pages each), first tokens
    d.step()                         # position 7 still fits the second page
    out = d.step()                   # a needs position 8 -> a third page: b is evicted
    assert out.preempted == ["b"] and [d.request.request_id for d in out.decodes] == ["a"]
    assert b.phase == "queued" and d.scheduler.queue[0] is b
    assert b.cached == 0 and b.owed == 9 and b.prompt_len == 7 and b.num_output == 2
    d.run()
    assert a.num_output == 8 and b.num_output == 8


def test_a_single_request_too_big_for_what_is_left_preempts_itself_then_aborts_or_finishes():
    d = Driver(num_pages=3, page_size=4, max_batched=64, max_seqs=2)
    s = d.submit("a", 10, 8)         # grows to 18 tokens > 12
    d.run()
    assert s.finish_reason == "aborted" and d.aborted == [s]
    assert s.times.preemptions == 1


def test_oversize_and_overlong_requests_abort_at_admission():
    d = Driver(num_pages=4, page_size=4, max_positions=64)
    big = d.submit("big", 17, 2)
    ok = d.submit("ok", 8, 2)
    out = d.step()
    assert out.aborted == [big] and big.finish_reason == "aborted" and big.done
    assert out.portions[0].request is ok
    d = Driver(num_pages=64, page_size=4, max_positions=12)
    assert d.submit("long", 13, 1) and d.step().aborted[0].request_id == "long"
    s = d.submit("edge", 10, 20)
    d.run()
    assert len(s.tokens) == 12 and s.finish_reason == "length"


def test_head_of_line_blocking_and_max_num_seqs():
    d = Driver(num_pages=6, page_size=4, max_batched=64, max_seqs=8)
    d.submit("a", 16, 1)
    d.submit("b", 12, 1)             # does not fit beside a
    d.submit("c", 2, 1)              # would fit, but waits behind b
    out = d.scheduler.schedule()
    assert [p.request.request_id for p in out.portions] == ["a"]
    d = Driver(max_seqs=2, max_batched=64)
    for i in range(5):
        d.submit(f"r{i}", 4, 3)
    assert len(d.scheduler.schedule().portions) == 2
    d.run()


def test_eos_and_stop_tokens():
    d = Driver(eos=7)
    s = d.submit("a", 4, 10, ignore_eos=False)
    t = d.submit("b", 4, 3, ignore_eos=True)
    d.run()
    assert s.finish_reason == "eos" and s.output == [7]
    assert t.finish_reason == "length" and t.num_output == 3


def test_abort():
    d = Driver()
    d.submit("x", 10, 10)
    d.submit("y", 10, 10)
    d.step()
    assert d.scheduler.abort_request("x") and d.scheduler.abort_request("y")
    assert not d.scheduler.abort_request("z")
    assert not d.scheduler.has_unfinished()
    d.manager.check()
    assert d.manager.num_free_pages() == 16


def test_unchunked_mode_runs_whole_prompts_before_decode_tokens():
    d = Driver(chunked=False, max_batched=8, num_pages=64, max_seqs=2)
    d.submit("a", 20, 3)
    out = d.step()
    assert out.portions[0].count == 20         # the whole prompt, beyond the token budget
    d.submit("b", 20, 2)
    out = d.step()                             # b can be admitted: it goes first, a holds
    assert [p.request.request_id for p in out.portions] == ["b"] and not out.decodes
    out = d.step()
    assert sorted(x.request.request_id for x in out.decodes) == ["a", "b"]
    d.run()


def test_unchunked_mode_decodes_on_when_nothing_can_be_admitted():
    # every slot taken: the reference plans nothing here (servelab/engine/scheduler.py:177) and
    # stops for good; the active request has to go on, since that is what frees the slot
    d = Driver(chunked=False, max_batched=8, num_pages=64, max_seqs=1)
    a = d.submit("a", 20, 3)
    b = d.submit("b", 20, 2)
    d.step()
    out = d.step()
    assert [x.request.request_id for x in out.decodes] == ["a"] and not out.portions
    d.run()
    assert a.num_output == 3 and b.num_output == 2
    # the head of the queue does not fit beside what is active (tight pool): same decision
    d = Driver(chunked=False, max_batched=64, num_pages=8, page_size=4, max_seqs=4)
    reqs = [d.submit(f"r{i}", 14, 6) for i in range(3)]
    d.run()
    assert all(r.num_output == 6 and r.finish_reason == "length" for r in reqs)


def test_window_groups_keep_few_pages_during_long_decoding():
    d = Driver(num_pages=12, page_size=4, max_batched=64, window=8)
    s = d.submit("a", 6, 40)
    d.run()
    assert s.num_output == 40
    assert d.manager.page_groups[1].allocator.high_water <= 4
    assert d.manager.page_groups[0].allocator.high_water == 12


def ahead_driver(**kw):
    """A driver that does what the engine does around every step: ask for the
    step ahead while the step's tokens are not known yet, and when there is one
    run it as the next step."""
    d = Driver(**kw)

    def run_plan(out):
        """Runs ``out``; returns the step ahead that was planned meanwhile."""
        sampled = {}
        for item in out.items():
            if item.request.phase == "active":
                d.manager.commit(item.request.request_id, item.start + item.count)
            if item.samples:
                sampled[item.request.request_id] = d.token
        ahead = d.scheduler.plan_ahead(out)
        d.finished += d.scheduler.complete(out, sampled)
        d.aborted += out.aborted
        d.manager.check()
        return ahead

    def step_and_ahead():
        out = d.scheduler.schedule()
        return out, run_plan(out)

    def run_with_ahead(max_steps=500):
        planned_ahead = steps = 0
        while d.scheduler.has_unfinished():
            steps += 1
            assert steps < max_steps
            out = d.scheduler.schedule()
            while out is not None:
                assert all(it.request.phase == "active" for it in out.items())   # (no stop tokens here)
                out = run_plan(out)
                planned_ahead += out is not None
        assert d.manager.num_free_pages() == d.manager.num_pages
        return planned_ahead
    d.run_plan, d.step_and_ahead, d.run_with_ahead = run_plan, step_and_ahead, run_with_ahead
    return d


def test_the_step_ahead_is_planned_under_a_standing_queue_when_nobody_can_be_admitted():
    # two slots, five requests: while both slots decode and nobody ends by length, the queue
    # cannot move, so the next step is known
    d = ahead_driver(max_seqs=2, num_pages=64)
    reqs = [d.submit(f"r{i}", 6, 9) for i in range(5)]
    out, ahead = d.step_and_ahead()            # r0, r1 admitted; three wait
    assert len(d.scheduler.queue) == 3 and len(out.portions) == 2
    assert ahead is not None and [x.request.request_id for x in ahead.decodes] == ["r0", "r1"]
    # the pages of the step ahead are reserved: the ordinary plan of that step is the same one
    free = d.manager.num_free_pages()
    again = d.scheduler.schedule()
    assert [(x.request.request_id, x.start) for x in again.decodes] == \
        [(x.request.request_id, x.start) for x in ahead.decodes] and not again.portions
    assert d.manager.num_free_pages() == free
    d.run_plan(again)
    planned = d.run_with_ahead()
    assert all(r.num_output == 9 for r in reqs)
    # of a request's 8 decode steps, all but the one in which it ends are planned ahead
    assert planned >= 3 * 5


def test_no_step_ahead_when_a_slot_or_the_pages_open_up_for_the_queue():
    d = ahead_driver(max_seqs=2, num_pages=64)
    d.submit("a", 6, 3), d.submit("b", 6, 8), d.submit("c", 6, 2)
    assert d.step_and_ahead()[1] is not None   # a gets the first of its 3 tokens
    assert d.step_and_ahead()[1] is not None   # ... its second
    out, ahead = d.step_and_ahead()            # ... its third: it ends with this step
    assert ahead is None                       # so c takes its slot in the next
    # a free slot but no pages for the head of the queue: the active request decodes ahead
    d = ahead_driver(max_seqs=4, num_pages=6, page_size=4)
    d.submit("a", 9, 6)                        # 3 pages, grows into a fourth
    d.step_and_ahead()
    d.submit("big", 13, 2)                     # 4 pages: does not fit beside a
    out, ahead = d.step_and_ahead()
    assert [x.request.request_id for x in out.decodes] == ["a"] and not out.portions
    assert ahead is not None
    # a head that fits is admitted in the next step: no step ahead
    d = ahead_driver(max_seqs=4, num_pages=16, page_size=4)
    d.submit("a", 9, 6)
    d.step_and_ahead()
    d.submit("b", 5, 2)
    out = d.scheduler.schedule()
    assert [p.request.request_id for p in out.portions] == ["b"]
    assert d.run_plan(out) is not None         # nothing waits any more
    d.submit("c", 5, 2)
    out = d.scheduler.schedule()
    d.scheduler.queue.append(d.scheduler.active.pop())     # (as if c had come a moment later)
    d.manager.close("c")
    out.portions.clear()
    assert d.run_plan(out) is None             # c fits: the next step admits it
    # a head that can never be held is aborted by the next schedule: no step ahead either
    d = ahead_driver(max_seqs=4, num_pages=6, page_size=4)
    d.submit("a", 9, 6)
    d.step_and_ahead()
    out = d.scheduler.schedule()
    d.submit("never", 40, 2)
    assert d.run_plan(out) is None
    d.run_with_ahead()
    assert [r.request_id for r in d.aborted] == ["never"]


@pytest.mark.parametrize("seed", range(6))
def test_steps_ahead_under_random_loads_lose_nothing(seed):
    import random
    rng = random.Random(seed)
    d = ahead_driver(max_seqs=rng.choice([1, 2, 3]), num_pages=rng.choice([8, 12, 40]),
                     page_size=4, max_batched=rng.choice([4, 16, 64]))
    reqs = [d.submit(f"r{i}", rng.randint(1, 14), rng.randint(1, 12)) for i in range(9)]
    d.run_with_ahead()
    for r in reqs:
        assert r.finish_reason == "length" and r.num_output == r.params.max_tokens

"""The load benchmark's own parts on the CPU: workload, the two load patterns
against a scripted engine, the summary's formulas."""
import os
import sys
import types

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench_serving as bs


def test_workload_is_seeded_and_bounded():
    a = bs.synthetic_requests(50, 1000, 200, 64, seed=3, longest=256)
    b = bs.synthetic_requests(50, 1000, 200, 64, seed=3, longest=256)
    assert [(r.prompt_token_ids, r.output_tokens) for r in a] == \
        [(r.prompt_token_ids, r.output_tokens) for r in b]
    assert a != bs.synthetic_requests(50, 1000, 200, 64, seed=4, longest=256)
    for r in a:
        assert 1 <= len(r.prompt_token_ids) and r.output_tokens >= 1
        assert len(r.prompt_token_ids) + r.output_tokens <= 256
        assert all(0 <= t < 1000 for t in r.prompt_token_ids)
    lengths = [len(r.prompt_token_ids) for r in bs.synthetic_requests(400, 1000, 200, 64, seed=1)]
    assert 190 < sum(lengths) / len(lengths) < 210 and min(lengths) >= 8


def test_percentile_interpolates():
    assert bs.percentile([1.0], 99) == 1.0
    assert bs.percentile([1.0, 3.0], 50) == 2.0
    assert bs.percentile([4.0, 1.0, 2.0, 3.0], 0) == 1.0
    assert bs.percentile([4.0, 1.0, 2.0, 3.0], 100) == 4.0
    assert bs.percentile(list(range(101)), 90) == 90


class ScriptedEngine:
    """Finishes every request after as many steps as it has output tokens."""

    def __init__(self):
        self.live, self.n, self.most_live, self.num_steps = {}, 0, 0, 0

    def add_request(self, prompt_token_ids=None, sampling_params=None, **_):
        rid = f"r{self.n}"
        self.n += 1
        self.live[rid] = sampling_params.max_tokens
        self.most_live = max(self.most_live, len(self.live))
        return rid

    def has_unfinished(self):
        return bool(self.live)

    def step(self):
        self.num_steps += 1
        out = []
        for rid in list(self.live):
            self.live[rid] -= 1
            if self.live[rid] == 0:
                del self.live[rid]
                out.append(types.SimpleNamespace(request_id=rid))
        return out


def test_closed_loop_keeps_the_concurrency():
    reqs = bs.synthetic_requests(20, 100, 30, 6, seed=0)
    eng = ScriptedEngine()
    done = bs.drive(eng, reqs, bs.KeepInFlight(3), dict(temperature=0.0))
    assert len(done) == 20 and eng.most_live == 3 and not eng.has_unfinished()


def test_open_loop_submits_everything():
    reqs = bs.synthetic_requests(10, 100, 30, 4, seed=0)
    eng = ScriptedEngine()
    import time
    done = bs.drive(eng, reqs, bs.PoissonArrivals(5000.0, 1, time.monotonic()), dict(temperature=0.0))
    assert sorted(o.request_id for o in done) == sorted(f"r{i}" for i in range(10))


def test_summary_formulas():
    def out(n, ttft, latency, pre=0):
        return types.SimpleNamespace(outputs=[types.SimpleNamespace(token_ids=[0] * n)],
                                     metrics={"ttft": ttft, "latency": latency, "preemptions": pre})
    res = bs.summarise([out(11, 0.1, 0.6), out(5, 3.0, 3.4, pre=1), out(1, 0.05, 0.05)],
                       elapsed=2.0, ttft_slo_ms=2000, tpot_slo_ms=60)
    assert res["requests"] == 3 and res["output_tokens"] == 17
    assert res["output_throughput_tok_s"] == 8.5 and res["preemptions"] == 1
    assert res["ttft_ms_p50"] == 100.0
    assert res["tpot_ms_p50"] == pytest.approx(75.0)       # (500 ms / 10 + 400 ms / 4) / 2
    assert res["goodput"] == 0.5                           # one of the two with a TPOT is inside both bounds


def test_uniform_prompt_lengths():
    reqs = bs.synthetic_requests(200, 1000, 0, 16, seed=3, input_range=(512, 4096), longest=8192)
    lengths = [len(r.prompt_token_ids) for r in reqs]
    assert min(lengths) >= 512 and max(lengths) <= 4096 and 2000 < sum(lengths) / 200 < 2600

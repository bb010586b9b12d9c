#!/usr/bin/env python3
"""Generation through ``LLMEngine`` under load, in one process: time to first
token, time per output token, output throughput and the share of requests
inside both latency bounds.

The workload and the options are those of the reference's harness
(servelab/bench/benchmark_serving.py:58-157, servelab/bench/datasets.py:8-20):
prompts of random token ids whose lengths are Gaussian (``--input-mean``, 40
around it), a Gaussian number of output tokens (``--output-tokens``, 20 around
it) with ``ignore_eos``, either a closed loop that keeps ``--concurrency``
requests in flight (``--load-pattern fixed``) or arrivals with exponential gaps
at ``--request-rate`` a second against the wall clock (``poisson``).  Token ids
are uniform over the vocabulary; no public dataset is read.

    python bench_serving.py                       # Qwen2.5-7B shape, random weights
    python bench_serving.py --model DIR --num-prompts 64 --load-pattern poisson --request-rate 8

The last line printed is one JSON object with the same figures.
"""
import argparse
import json
import math
import os
import random
import sys
import time
from dataclasses import dataclass
from typing import List

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


@dataclass
class Request:
    prompt_token_ids: List[int]
    output_tokens: int


def synthetic_requests(n: int, vocab: int, input_mean: int, output_mean: int, seed: int,
                       input_std: int = 40, output_std: int = 20, longest: int = 0,
                       input_range=None) -> List[Request]:
    """``longest`` > 0 bounds prompt + output (the model's positions);
    ``input_range`` (lo, hi) draws prompt lengths uniformly from it instead of
    from the Gaussian."""
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        if input_range:
            n_in = rng.randint(int(input_range[0]), int(input_range[1]))
        else:
            n_in = max(8, int(rng.gauss(input_mean, input_std)))
        n_out = max(1, int(rng.gauss(output_mean, output_std)))
        if longest:
            n_in = min(n_in, max(1, longest - n_out))
        out.append(Request([rng.randrange(vocab) for _ in range(n_in)], n_out))
    return out


class KeepInFlight:
    """Closed loop: a new request whenever fewer than ``concurrency`` are in flight."""

    def __init__(self, concurrency: int):
        self.concurrency = concurrency

    def due(self, now: float, in_flight: int) -> int:
        return max(0, self.concurrency - in_flight)

    def idle_for(self, now: float) -> float:
        return 0.0


class PoissonArrivals:
    """Open loop: arrivals with exponential gaps at ``rate`` a second against the
    wall clock, whatever the engine is doing."""

    def __init__(self, rate: float, seed: int, start: float):
        self.rng, self.rate, self.next_at = random.Random(seed), rate, start

    def due(self, now: float, in_flight: int) -> int:
        n = 0
        while now >= self.next_at:
            n += 1
            self.next_at += self.rng.expovariate(self.rate)
        return n

    def idle_for(self, now: float) -> float:
        return max(0.0, self.next_at - now)


def drive(engine, requests: List[Request], arrivals, sampling) -> list:
    """One loop for both load patterns: submit what ``arrivals`` says is due,
    step the engine while it has work, sleep until the next arrival otherwise.
    Returns the finished requests' outputs."""
    from servelab_amd import SamplingParams
    queue = list(reversed(requests))
    ours, done = set(), []
    while queue or ours:
        now = time.monotonic()
        for _ in range(min(len(queue), arrivals.due(now, len(ours)))):
            req = queue.pop()
            ours.add(engine.add_request(
                prompt_token_ids=req.prompt_token_ids,
                sampling_params=SamplingParams(max_tokens=req.output_tokens, ignore_eos=True,
                                               **sampling)))
        if engine.has_unfinished():
            for out in engine.step():
                if out.request_id in ours:
                    ours.discard(out.request_id)
                    done.append(out)
        else:
            time.sleep(min(arrivals.idle_for(now), 0.001))
    return done


def percentile(values: List[float], q: float) -> float:
    """Linear interpolation between the order statistics."""
    if not values:
        return float("nan")
    v = sorted(values)
    x = (len(v) - 1) * q / 100.0
    lo = int(math.floor(x))
    hi = min(lo + 1, len(v) - 1)
    return v[lo] + (v[hi] - v[lo]) * (x - lo)


def summarise(done: list, elapsed: float, ttft_slo_ms: float, tpot_slo_ms: float) -> dict:
    """TTFT = first token - arrival; TPOT = (latency - TTFT) / (output tokens - 1)
    (servelab/bench/benchmark_serving.py:102-113)."""
    ttft, tpot, pairs, tokens, preemptions = [], [], [], 0, 0
    for out in done:
        m = out.metrics
        n = len(out.outputs[0].token_ids)
        tokens += n
        preemptions += m["preemptions"]
        t = m["ttft"] * 1e3
        ttft.append(t)
        if n > 1:
            p = (m["latency"] - m["ttft"]) / (n - 1) * 1e3
            tpot.append(p)
            pairs.append((t, p))
    good = sum(1 for t, p in pairs if t <= ttft_slo_ms and p <= tpot_slo_ms)
    return {
        "requests": len(done), "elapsed_s": round(elapsed, 3),
        "output_tokens": tokens, "output_throughput_tok_s": round(tokens / elapsed, 1),
        "ttft_ms_p50": round(percentile(ttft, 50), 2), "ttft_ms_p90": round(percentile(ttft, 90), 2),
        "ttft_ms_p99": round(percentile(ttft, 99), 2),
        "tpot_ms_p50": round(percentile(tpot, 50), 3), "tpot_ms_p99": round(percentile(tpot, 99), 3),
        "goodput": round(good / max(1, len(pairs)), 4), "preemptions": preemptions,
    }


class AsksFor:
    """The output-length predictor of the policy "sjf-predicted" for this load: every request
    generates exactly the tokens it asks for (eos is ignored), so the prediction is exact
    (the "oracle" of examples/run_simulator.py:56-58)."""

    def predict_remaining(self, req) -> int:
        return req.params.max_tokens


def build_engine(args):
    from servelab_amd import CacheConfig, LLMEngine, SchedulerConfig, load_config
    from servelab_amd.cli import tune_option
    cache = CacheConfig(block_size=args.block_size, num_blocks=args.num_blocks or None,
                        gpu_memory_utilization=args.gpu_memory_utilization)
    sched = SchedulerConfig(max_num_seqs=args.max_num_seqs,
                            max_num_batched_tokens=args.max_batched_tokens,
                            chunked_prefill=not args.no_chunked_prefill,
                            policy=args.scheduler_policy)
    warm = dict(tune_products=tune_option(args), capture_graphs_up_to=args.capture_graphs_up_to,
                run_ahead=not args.no_run_ahead,
                predictor=AsksFor() if args.scheduler_policy == "sjf-predicted" else None)
    if args.model:
        cfg = load_config(args.model)
        return cfg, LLMEngine(cfg, cache, sched, dtype=args.dtype, **warm)
    import bench                                     # random weights of a named shape, made on the device
    cfg, model, _ = bench.build(argparse.Namespace(shape=args.shape, layers=args.layers,
                                                   dtype=args.dtype, seed=args.seed))
    return cfg, LLMEngine(cfg, cache, sched, model=model, **warm)


def run(args) -> dict:
    cfg, engine = build_engine(args)
    sampling = dict(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k)
    span = (args.input_min, args.input_max) if args.input_max else None
    requests = synthetic_requests(args.num_prompts, cfg.vocab_size, args.input_mean,
                                  args.output_tokens, args.seed,
                                  longest=min(cfg.max_position_embeddings, args.max_context or 1 << 30),
                                  input_range=span)
    if args.warmup_requests:
        # the first steps of a process compile nothing, but capture a graph per decode shape
        warm = synthetic_requests(args.warmup_requests, cfg.vocab_size, args.input_mean, 8,
                                  args.seed + 1, longest=cfg.max_position_embeddings)
        drive(engine, warm, KeepInFlight(min(args.concurrency, len(warm))), sampling)
    steps0 = engine.num_steps
    t0 = time.monotonic()
    arrivals = KeepInFlight(args.concurrency) if args.load_pattern == "fixed" else \
        PoissonArrivals(args.request_rate, args.seed + 2, t0)
    done = drive(engine, requests, arrivals, sampling)
    elapsed = time.monotonic() - t0
    res = summarise(done, elapsed, args.ttft_slo_ms, args.tpot_slo_ms)
    res["steps"] = engine.num_steps - steps0
    res["config"] = {
        "model": args.model or f"{args.shape} shape, random weights", "dtype": args.dtype,
        "load_pattern": args.load_pattern,
        "concurrency": args.concurrency if args.load_pattern == "fixed" else None,
        "request_rate": args.request_rate if args.load_pattern == "poisson" else None,
        "num_prompts": args.num_prompts,
        "input": f"uniform {span[0]}..{span[1]}" if span else f"gauss {args.input_mean}",
        "output_tokens": args.output_tokens, "max_num_seqs": args.max_num_seqs,
        "max_batched_tokens": args.max_batched_tokens, "block_size": args.block_size,
        "num_blocks": engine.num_blocks, "temperature": args.temperature, "top_p": args.top_p,
        "top_k": args.top_k, "run_ahead": not args.no_run_ahead,
    }
    return res


def parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", default="", help="model folder; empty = random weights of --shape")
    ap.add_argument("--shape", default="7b", choices=["7b", "32b", "72b"])
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0 = all)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--num-prompts", type=int, default=32)
    ap.add_argument("--input-mean", type=int, default=200)
    ap.add_argument("--input-min", type=int, default=1, help="with --input-max: uniform prompt lengths")
    ap.add_argument("--input-max", type=int, default=0, help="0 = Gaussian lengths around --input-mean")
    ap.add_argument("--max-context", type=int, default=0, help="bound on prompt + output (0 = the model's)")
    ap.add_argument("--output-tokens", type=int, default=64)
    ap.add_argument("--load-pattern", choices=["fixed", "poisson"], default="fixed")
    ap.add_argument("--concurrency", type=int, default=8)
    ap.add_argument("--request-rate", type=float, default=2.0)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-blocks", type=int, default=0, help="0 = from free memory")
    ap.add_argument("--max-num-seqs", type=int, default=64)
    ap.add_argument("--max-batched-tokens", type=int, default=2048)
    ap.add_argument("--no-chunked-prefill", action="store_true")
    ap.add_argument("--scheduler-policy", default="fcfs", choices=["fcfs", "priority", "sjf-predicted"],
                    help="sjf-predicted: fewest tokens still to come first, the output lengths being known here")
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.85)
    ap.add_argument("--ttft-slo-ms", type=float, default=2000)
    ap.add_argument("--tpot-slo-ms", type=float, default=50)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--warmup-requests", type=int, default=4,
                    help="short requests run before the clock starts (0 = none)")
    ap.add_argument("--tune-products", action="store_true")
    ap.add_argument("--capture-graphs-up-to", type=int, default=0,
                    help="capture decode graphs for contexts up to this length before the clock starts")
    ap.add_argument("--no-run-ahead", action="store_true",
                    help="wait for every step's tokens before the next step is planned")
    ap.add_argument("--tune-rows", default="", help="further step sizes (rows) to tune the library products for")
    return ap


def main(argv=None) -> int:
    args = parser().parse_args(argv)
    res = run(args)
    rows = [("requests", res["requests"]), ("elapsed_s", res["elapsed_s"]),
            ("output_throughput_tok/s", res["output_throughput_tok_s"]),
            ("TTFT ms p50/p90/p99",
             f"{res['ttft_ms_p50']:.1f} / {res['ttft_ms_p90']:.1f} / {res['ttft_ms_p99']:.1f}"),
            ("TPOT ms p50/p99", f"{res['tpot_ms_p50']:.2f} / {res['tpot_ms_p99']:.2f}"),
            ("goodput (TTFT and TPOT bound)", f"{res['goodput']:.1%}"),
            ("preemptions", res["preemptions"]), ("engine steps", res["steps"])]
    width = max(len(k) for k, _ in rows)
    for k, v in rows:
        print(f"{k:<{width}}  {v}")
    print(json.dumps(res), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

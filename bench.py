#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

Default run: the layer sizes of the Qwen2.5-7B shape with random weights,
bfloat16, a batch of 8 requests whose context ends at 4,096 tokens, 16-token
pages.  A "step" is one decode step of the whole batch through the engine
(scheduler, step function, greedy sampling); ``value`` is decoded tokens per second.
The same line carries a 2,048-token prefill, the decode step's HBM roofline
(every weight the step uses once plus the cache of the live requests, over its
time) and decode at batch 1 and 64.

The reference has no recorded numbers; its harness measures the same kind of
quantities over synthetic random-id prompts (servelab/bench/benchmark_serving.py:102-121,
servelab/bench/datasets.py:8-20, 10 warm-up + 50 timed iterations with device
events in servelab/bench/kernel_bench.py:12-23).

    python bench.py --gpus 1 --steps 20 --warmup 3
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN25_7B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=28,
    hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
    intermediate_size=18944, vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=False, use_sliding_window=False, max_position_embeddings=32768,
    torch_dtype="bfloat16", eos_token_id=151645)


# the other shapes of the same architecture that the engine is sized for
QWEN25_32B = dict(QWEN25_7B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=40,
                  num_key_value_heads=8, intermediate_size=27648)
QWEN25_72B = dict(QWEN25_7B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                  num_key_value_heads=8, intermediate_size=29568)
QWEN25_05B = dict(QWEN25_7B, num_hidden_layers=24, hidden_size=896, num_attention_heads=14, num_key_value_heads=2,
                  head_dim=64, intermediate_size=4864, vocab_size=151936, tie_word_embeddings=True)
QWEN25_15B = dict(QWEN25_7B, num_hidden_layers=28, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2,
                  intermediate_size=8960, vocab_size=151936, tie_word_embeddings=True)
QWEN25_3B = dict(QWEN25_7B, num_hidden_layers=36, hidden_size=2048, num_attention_heads=16, num_key_value_heads=2,
                 intermediate_size=11008, vocab_size=151936, tie_word_embeddings=True)
QWEN25_14B = dict(QWEN25_7B, num_hidden_layers=48, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                  intermediate_size=13824)
SHAPES = {"7b": ("Qwen2.5-7B shape", QWEN25_7B), "32b": ("Qwen2.5-32B shape", QWEN25_32B),
          "72b": ("Qwen2.5-72B shape", QWEN25_72B), "0.5b": ("Qwen2.5-0.5B shape", QWEN25_05B),
          "1.5b": ("Qwen2.5-1.5B shape", QWEN25_15B), "3b": ("Qwen2.5-3B shape", QWEN25_3B),
          "14b": ("Qwen2.5-14B shape", QWEN25_14B)}


def build(args):
    import torch
    import servelab_amd  # noqa: F401
    from servelab_amd import Qwen2Config
    from servelab_amd.engine.session import random_model_on_device

    raw = dict(SHAPES[args.shape][1])
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    cfg = Qwen2Config.from_hf(raw)
    model = random_model_on_device(cfg, args.seed, args.dtype, "cuda:0")
    torch.cuda.synchronize()
    return cfg, model, full_layers


def weight_bytes_per_step(cfg, itemsize):
    """Bytes of weights one decode step reads: every matrix, bias and gain of
    every layer once, the final gain and the head; of the embedding only the
    batch's rows (counted with the activations, not here)."""
    h, d = cfg.hidden_size, cfg.head_dim
    qkv = (cfg.num_heads + 2 * cfg.num_kv_heads) * d
    per_layer = (qkv * h + cfg.num_heads * d * h + 3 * h * cfg.intermediate_size) * itemsize \
        + (qkv + 2 * h) * 4
    return cfg.num_layers * per_layer + h * 4 + cfg.vocab_size * h * itemsize


def cache_bytes_per_token(cfg, itemsize):
    return 2 * cfg.num_layers * cfg.num_kv_heads * cfg.head_dim * itemsize


def prefill_flops(cfg, T):
    h, d = cfg.hidden_size, cfg.head_dim
    qkv = (cfg.num_heads + 2 * cfg.num_kv_heads) * d
    linear = cfg.num_layers * (qkv * h + cfg.num_heads * d * h + 3 * h * cfg.intermediate_size)
    attn = 2 * cfg.num_heads * d * T * T * cfg.num_layers          # causal half of 4 T^2 nh D
    return 2 * T * linear + attn + 2 * cfg.vocab_size * h


def time_decode(cfg, model, batch, ctx_end, steps, warmup, page, seed=0):
    """Contract timing of decode steps through the engine itself (scheduler,
    step function, sampler): ``batch`` requests with prompts of random ids are
    prefilled (untimed), then ``warmup`` untimed decode steps, then exactly
    ``steps`` steps between two synchronisations.  The longest context reaches
    ``ctx_end`` at the last step (requests whose prompts were prefilled a step
    later are a token shorter each).  Returns (seconds a step: the region over
    ``steps``; mean context; the median of the times between the returns of
    two engine steps, which in the steady state is the median step).  The engine keeps one decode step
    queued ahead of the host; the region starts with that step finished and not
    yet consumed, so exactly ``steps`` steps are queued and finished inside it."""
    import torch
    from servelab_amd import CacheConfig, LLMEngine, SamplingParams, SchedulerConfig
    total = warmup + steps
    budget = max(8192, ctx_end)                          # a prompt fits one step, so requests start a step apart
    prompt_len = ctx_end - total - 1
    prefill_steps = -(-batch * prompt_len // budget)
    prompt_len -= prefill_steps - 1                      # the first request decodes while the others prefill
    pages = batch * (-(-(ctx_end + 2) // page)) + 16
    engine = LLMEngine(cfg, CacheConfig(block_size=page, num_blocks=pages),
                       SchedulerConfig(max_num_seqs=max(batch, 1), max_num_batched_tokens=budget),
                       model=model)
    gen = torch.Generator().manual_seed(seed)
    params = SamplingParams(temperature=0.0, max_tokens=total + prefill_steps + 64, ignore_eos=True)
    for _ in range(batch):
        engine.add_request(prompt_token_ids=torch.randint(0, cfg.vocab_size, (prompt_len,),
                                                          generator=gen).tolist(),
                           sampling_params=params)
    while any(not r.decoding for r in engine.scheduler.active) or engine.scheduler.queue:
        engine.step()                                  # prompts, in portions
    before = engine.num_steps
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks = [t0]
    for _ in range(steps):
        engine.step()
        marks.append(time.perf_counter())            # a step returns when the step before it has finished
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    gaps = sorted(b - a for a, b in zip(marks, marks[1:]))
    assert engine.num_steps - before == total and len(engine.scheduler.active) == batch
    lengths = [engine.runner.manager.length(r.request_id) for r in engine.scheduler.active]
    assert ctx_end - 2 <= max(lengths) <= ctx_end and min(lengths) >= ctx_end - 2 - batch, lengths
    mean_ctx = sum(lengths) / batch - (steps + 1) / 2.0
    del engine
    torch.cuda.empty_cache()
    return dt / steps, mean_ctx, gaps[len(gaps) // 2]


def time_prefill(model, T, page, repeats, max_chunk, seed=1, tune=True):
    """A prompt of T tokens from an empty cache, in portions of at most
    ``max_chunk`` tokens (one portion when T fits).  ``tune``: before the
    warm-up run the library's kernels are timed for a portion of that size, as
    the engine does at start-up with ``tune_products``.  Returns the median
    and the best of ``repeats`` runs, each between two synchronisations."""
    import torch
    from servelab_amd.engine import ModelRunner, StepEntry
    runner = ModelRunner(model, -(-T // page) + 8, page, max_num_seqs=4)
    vocab = model.spec.vocab_size
    toks = torch.randint(0, vocab, (T,), generator=torch.Generator().manual_seed(seed)).tolist()
    ops = model.rt.ops
    if tune:
        runner.tune_products([min(max_chunk, T)])

    def once(tag):
        pos = 0
        while pos < T:
            n = min(max_chunk, T - pos)
            logits = runner.step([StepEntry(tag, toks[pos:pos + n], [n - 1] if pos + n == T else [])])
            pos += n
        first = ops.argmax(logits).tolist()
        runner.close(tag)
        return first

    once("w")
    torch.cuda.synchronize()
    times = []
    for i in range(repeats):
        t0 = time.perf_counter()
        once(f"p{i}")
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    del runner
    torch.cuda.empty_cache()
    times.sort()
    return times[len(times) // 2], times[0]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--prefill-chunk", type=int, default=2048)
    ap.add_argument("--shape", default="7b", choices=sorted(SHAPES))
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0 = all)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-tune", action="store_true",
                    help="leave the library's default kernel choice for the prompt products")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; --gpus N > 1 is not supported")
        return 2

    cfg, model, full_layers = build(args)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    itemsize = 2 if short == "bf16" else 4
    page = args.block_size

    step_s, mean_ctx, median_s = time_decode(cfg, model, args.batch, args.context, args.steps, args.warmup, page)
    value = args.batch / step_s
    step_bytes = weight_bytes_per_step(cfg, itemsize) + \
        args.batch * mean_ctx * cache_bytes_per_token(cfg, itemsize)
    achieved = step_bytes / step_s / 1e9

    line = {
        "metric": "decode_tokens_per_s", "value": round(value, 2), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4),
        "ms_per_step_median": round(median_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short,
        "data": "synthetic: seeded random weights, prompts of uniform random token ids prefilled "
                "by the engine up to the context",
        "config": {
            "model": SHAPES[args.shape][0], "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "none", "layers": cfg.num_layers, "layers_of_shape": full_layers,
            "hidden_size": cfg.hidden_size, "num_heads": cfg.num_heads,
            "num_kv_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "page_size": page, "prefill_tokens": args.prefill_tokens,
            "decode_mean_context": round(mean_ctx, 1), "sampling": "greedy",
            "weight_layout": model.rt.ops.layout_summary(),
            "library_tuning": "off" if args.no_tune or args.no_prefill else "tunableop",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    if not args.no_prefill:
        T = args.prefill_tokens
        pre_s, best_s = time_prefill(model, T, page, repeats=5, max_chunk=args.prefill_chunk,
                                     tune=not args.no_tune)
        line["prefill"] = {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
                           "frac": round(prefill_flops(cfg, T) / pre_s / PEAK_FLOPS[short], 4),
                           "timing": "median of 5", "best_ms": round(best_s * 1e3, 3)}
    if not args.no_points:
        import gc
        import torch
        points = {}
        for b in (1, 64):
            try:
                s, _, _ = time_decode(cfg, model, b, args.context, max(5, args.steps // 2), 2, page)
                points[f"decode_b{b}"] = round(b / s, 2)
            except torch.OutOfMemoryError:
                # (the 72B shape: the cache of 64 requests at this context does not fit beside 145 GB of
                # weights and the row-major copies kept for the prompt products)
                points[f"decode_b{b}"] = None
                gc.collect()
                torch.cuda.empty_cache()
        line["points"] = points
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Offline generation from the command line.

Reference: examples/run_engine.py:27-72 — same options with the same meanings
(--model, --prompt, --max-tokens, --block-size, --num-blocks; --no-prefix-cache
and --kv-cache-dtype are accepted for compatibility: this engine has no prefix
cache and keeps the cache in the compute dtype), the same fixed
max_num_seqs=16 / max_num_batched_tokens=1024 defaults, temperature 1.0
sampling unless told otherwise, the same printed lines.  Without --model a
tiny random model is used, as there; here its weights (and those of any
``--config`` with ``--random-weights SEED``) are drawn on the device, so a
configuration of any size starts at once and no folder is written, unless
--model names one to write.
"""
import argparse
import json
import os
import sys

TINY_DEFAULT = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=96, hidden_size=32,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=8,
    intermediate_size=64, rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=512,
    tie_word_embeddings=False, torch_dtype="float32", eos_token_id=95)   # tests/helpers_tiny_model.py:7-33


def build_parser():
    ap = argparse.ArgumentParser(prog="run_engine", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", default="", help="model folder; empty = tiny random model")
    ap.add_argument("--prompt", default="The meaning of life is")
    ap.add_argument("--max-tokens", type=int, default=32)
    ap.add_argument("--no-prefix-cache", action="store_true", help="accepted; there is no prefix cache")
    ap.add_argument("--kv-cache-dtype", default="auto", help="only 'auto' (the compute dtype)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-blocks", type=int, default=0, help="0 = auto")
    # beyond the reference's script
    ap.add_argument("--dtype", default="auto", choices=["auto", "bfloat16", "bf16", "float32", "fp32"])
    ap.add_argument("--config", default="", help="config.json for --random-weights")
    ap.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                    help="seeded random weights for --config (or the tiny default), made on the "
                         "device; with --model DIR they are written there as a model folder first")
    ap.add_argument("--prompt-ids", default="", help="comma-separated token ids instead of --prompt")
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--max-num-seqs", type=int, default=16)
    ap.add_argument("--max-batched-tokens", type=int, default=1024)
    ap.add_argument("--tune-products", action="store_true",
                    help="at start-up, time the library's matrix kernels for a full-budget step "
                         "and keep the fastest (bfloat16 only)")
    ap.add_argument("--capture-graphs-up-to", type=int, default=0, metavar="TOKENS",
                    help="capture the decode graphs for contexts up to this length at start-up "
                         "instead of when a request first needs them")
    ap.add_argument("--tune-rows", default="",
                    help="comma-separated further step sizes (rows) to time them for, e.g. typical "
                         "prompt lengths; implies --tune-products")
    return ap


def tune_option(args):
    """What ``LLMEngine(tune_products=...)`` takes: False, True, or the further row counts."""
    rows = [int(n) for n in args.tune_rows.split(",") if n.strip()] if getattr(args, "tune_rows", "") else []
    return rows if rows else bool(args.tune_products)


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.kv_cache_dtype != "auto":
        print(f"--kv-cache-dtype {args.kv_cache_dtype}: only 'auto' is supported", file=sys.stderr)
        return 2
    from . import (CacheConfig, LLMEngine, SamplingParams, SchedulerConfig, load_config,
                   write_random_model)
    from .config import resolve_architecture

    tokenizer = None
    seed = None
    if args.model and args.random_weights is None:
        mc = load_config(args.model)
        has_files = any(os.path.exists(os.path.join(args.model, f))
                        for f in ("tokenizer.json", "tokenizer_config.json", "tokenizer.model"))
        try:
            if not has_files:
                raise FileNotFoundError("no tokenizer files in the model folder")
            from transformers import AutoTokenizer          # tokenizer files only, optional
            tokenizer = AutoTokenizer.from_pretrained(args.model)
        except Exception as e:                              # noqa: BLE001
            print(f"[warn] no tokenizer: {e}")
    else:
        raw = dict(TINY_DEFAULT)
        if args.config:
            with open(args.config, encoding="utf-8") as f:
                raw = json.load(f)
        mc = resolve_architecture(raw).config_from_hf(raw, "")
        seed = args.random_weights or 0
        if args.model:                                      # keep the model: a folder, made on the host
            write_random_model(mc, args.model, seed=seed)
            mc, seed = load_config(args.model), None
    engine = LLMEngine(
        mc, CacheConfig(block_size=args.block_size, num_blocks=args.num_blocks or None),
        SchedulerConfig(max_num_seqs=args.max_num_seqs,
                        max_num_batched_tokens=args.max_batched_tokens),
        seed=args.seed, tokenizer=tokenizer, dtype=args.dtype, tune_products=tune_option(args),
        random_weights=seed, capture_graphs_up_to=args.capture_graphs_up_to)
    if args.prompt_ids:
        prompts = [[int(t) for t in args.prompt_ids.split(",")]]
    elif tokenizer is not None:
        prompts = [args.prompt]
    else:
        prompts = [[t % mc.vocab_size for t in range(10, 40)]]     # examples/run_engine.py:64
    outputs = engine.generate(
        prompts, SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature,
                                top_k=args.top_k, top_p=args.top_p), verbose=True)
    for out in outputs:
        comp = out.outputs[0]
        text = comp.text if comp.text else str(comp.token_ids)
        print(f"[{out.request_id}] finish={comp.finish_reason} -> {text}")
    print("stats:", engine.stats())
    return 0


if __name__ == "__main__":
    sys.exit(main())

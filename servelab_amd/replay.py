"""Trace replay: feed given token ids through a model step by step and write
the logits.  It samples nothing and has no forward pass, cache or loader of its
own: it drives the model, step function, cache manager and kernels that
generation uses.

The reference has no such tool; its nearest relatives build batches by hand and
diff logits against a second implementation
(scripts/debug/debug_spec_crossval.py:27-71, scripts/debug/debug_decode_step.py:27-43).

Input, one JSON object a line on standard input:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted ``<out>/<step>.f32`` holds the logits at
the wanted places, in the order of the entries and of ``want``, little-endian
float32 [wanted, vocab].  After every step a line ``done <step>`` is printed.
"""
import argparse
import json
import os
import sys

import numpy as np


def parse_args(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--max-live", type=int, default=16, help="most requests live at a time")
    return ap.parse_args(argv)


def run(args, stdin=sys.stdin, stdout=sys.stdout, ops=None) -> int:
    from .engine.batch import StepEntry
    from .engine.session import load_model_on_device, make_runner

    os.makedirs(args.out, exist_ok=True)
    _, model = load_model_on_device(args.model, args.dtype, args.device, ops=ops)
    page = args.block_size
    num_pages = max(1, -(-args.max_tokens // page))
    runner = make_runner(model, num_pages, page, max_num_seqs=max(1, getattr(args, "max_live", 16)))
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in msg.get("entries", [])]
        logits = runner.step(entries)
        if logits.shape[0] > 0:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = os.path.join(args.out, f".{step}.f32.tmp")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        for request in msg.get("end", []):
            runner.close(request)
        stdout.write(f"done {step}\n")
        stdout.flush()
    return 0


def main(argv=None) -> int:
    return run(parse_args(argv))

"""Runs a schedule through the replay tool (in process or as the bin/trace_run
program) and compares every written row with the plain implementation."""
import argparse
import io
import json
import os
import subprocess
import sys

import numpy as np
import torch

import plain_qwen2 as plain
from replay_schedules import expected_rows, max_tokens_needed

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_logits(folder, requests):
    cfg, w = plain.load_folder(folder)
    return {rid: plain.forward(cfg, w, toks).numpy() for rid, toks in requests.items()}


def tolerance(dtype, reference):
    """Largest allowed absolute difference of a logit, where no tighter bar is
    at hand (``bfloat16_bar`` is one).

    float32: 1e-4, the bar of the reference's own cross-checks for hidden states
    (tests/test_parallel.py:103-104).  bfloat16: 3 % of the largest logit of the
    plain implementation (at least of 1): an envelope for weights, activations
    and cache rounded to 8 bits of mantissa."""
    if dtype == "float32":
        return 1e-4
    top = max(float(np.abs(r).max()) for r in reference.values())
    return 0.03 * max(1.0, top)


_emulated_error = {}


def bfloat16_bar(folder, requests, reference, vocab, key):
    """The bar for bfloat16 logits of a model with random weights: 1.5 times the
    error of a float32 computation that rounds to bfloat16 at the places where
    the kernels do (tests/emulated_ops.py in bfloat16, on the CPU, every request
    whole), plus 1e-3.  Measured on MI355X the kernels' error is 1.0 to 1.2
    times the emulation's (tiny model A 3.4e-3 against 2.8e-3, B 6.5e-3 against
    6.9e-3, two layers of the 7B widths 0.089 against 0.107), so the bar says:
    no less exact than rounding makes it.  ``key`` caches the emulation's error
    per model."""
    if key not in _emulated_error:
        import tempfile
        from emulated_ops import EmulatedOps
        from replay_schedules import whole
        steps = whole(requests)
        with tempfile.TemporaryDirectory() as out:
            replay_in_process(folder, steps, out, "bfloat16", max_tokens_needed(steps),
                              ops=EmulatedOps(torch.bfloat16), device="cpu",
                              max_live=max(16, len(requests)))
            _emulated_error[key], _ = compare(out, steps, reference, vocab)
    return min(tolerance("bfloat16", reference), 1.5 * _emulated_error[key] + 1e-3)


PROBE_ABS, PROBE_REL = 0.004, 0.012


def probe_score(got, reference):
    """The bar for the probe model (tests/probe_model.py), whose logits are one-hot reads of the
    final normed row: largest |difference| / (PROBE_ABS + PROBE_REL |reference|); at most 1 passes.
    Relative, because each logit is rounded by itself (2^-9 of its own size per bfloat16 rounding,
    four of them between the attention weights and the logit)."""
    got, reference = torch.as_tensor(got), torch.as_tensor(reference)
    return float(((got - reference).abs() / (PROBE_ABS + PROBE_REL * reference.abs())).max())


def replay_in_process(folder, steps, out_dir, dtype, max_tokens, ops=None, device="cuda:0",
                      block_size=16, max_live=16):
    from servelab_amd.replay import run
    args = argparse.Namespace(model=folder, dtype=dtype, out=out_dir, max_tokens=max_tokens,
                              block_size=block_size, device=device, max_live=max_live)
    stdin = io.StringIO("".join(json.dumps(s) + "\n" for s in steps))
    stdout = io.StringIO()
    assert run(args, stdin, stdout, ops=ops) == 0
    assert stdout.getvalue().split("\n")[:-1] == [f"done {s['step']}" for s in steps]


def replay_program(folder, steps, out_dir, dtype, max_tokens, env=None):
    """Through bin/trace_run, one step at a time, waiting for each 'done'."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder,
           "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", f"got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


def compare(out_dir, steps, reference, vocab, score=None):
    """Largest absolute difference over all written rows (or largest ``score(got row, reference
    row)``)."""
    worst, where = 0.0, None
    rows = expected_rows(steps)
    for step, wanted in rows.items():
        path = os.path.join(out_dir, f"{step}.f32")
        assert os.path.exists(path), f"step {step} wrote no file"
        got = np.fromfile(path, dtype="<f4").reshape(-1, vocab)
        assert got.shape[0] == len(wanted), f"step {step}: {got.shape[0]} rows, wanted {len(wanted)}"
        assert np.isfinite(got).all(), f"step {step}: logits are not finite"
        for row, (rid, p) in zip(got, wanted):
            err = (float(np.abs(row - reference[rid][p]).max()) if score is None
                   else score(row, reference[rid][p]))
            if err > worst:
                worst, where = err, (step, rid, p)
    for st in steps:
        if st["step"] not in rows:
            assert not os.path.exists(os.path.join(out_dir, f"{st['step']}.f32"))
    return worst, where

"""Trace replay on the GPU, in float32 and in bfloat16: the same requests whole,
with the last 32 tokens decoded one by one, in portions of changing size, and
mixed with so few pages that they are used again, all compared with the plain
implementation."""
import os
import random

import pytest
import torch

import replay_schedules as rs
import probe_model as pm
from replay_harness import (bfloat16_bar, compare, plain_logits, probe_score, replay_in_process,
                            replay_program, tolerance)
from tiny_configs import TINY, make_folder

pytestmark = pytest.mark.gpu


def make_requests(vocab, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


LENGTHS = {"A": [37, 70, 49, 96, 130, 41, 66], "B": [41, 109, 56, 200, 33, 77]}


def schedule_steps(name, requests):
    if name == "whole":
        return rs.whole(requests)
    if name == "tail":
        return rs.tail_decoded(requests)
    if name == "portions":
        return rs.portions(requests)
    return rs.mixed(requests, {r: max(2, len(t) - 32) for r, t in requests.items()})


def pages_ever_needed(requests, page):
    return sum(-(-len(t) // page) for t in requests.values())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B"])
@pytest.mark.parametrize("schedule,page", [("whole", 16), ("tail", 16), ("portions", 16), ("mixed", 16),
                                           ("portions", 32), ("mixed", 32), ("tail", 64),
                                           ("portions", 64), ("mixed", 64)])
def test_replay_matches_plain(tmp_path, which, schedule, page, dtype):
    folder = make_folder(tmp_path, which, seed=11)
    vocab = TINY[which]["vocab_size"]
    requests = make_requests(vocab, LENGTHS[which], seed=5)
    reference = plain_logits(folder, requests)
    steps = schedule_steps(schedule, requests)
    out = str(tmp_path / "out")
    max_tokens = rs.max_tokens_needed(steps, max(64, page))
    if schedule == "mixed":                   # so few pages that they are used again
        assert pages_ever_needed(requests, page) > -(-max_tokens // page)
    replay_in_process(folder, steps, out, dtype, max_tokens, block_size=page)
    worst, where = compare(out, steps, reference, vocab)
    bar = tolerance(dtype, reference) if dtype == "float32" else \
        bfloat16_bar(folder, requests, reference, vocab, ("replay", which))
    print(f"{which} {schedule} page {page} {dtype}: max abs err {worst:.3e} at {where}, bar {bar:.3e}")
    assert worst < bar, f"max abs err {worst} at {where}"


PROBE_LENGTHS = [150, 61, 333, 97, 260, 48, 129]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page", [16, 32, 64])
@pytest.mark.parametrize("schedule", ["tail", "portions", "mixed"])
def test_replay_of_the_probe_model(tmp_path, schedule, page, dtype):
    """The model whose logits are the weights of the visible keys by token: one key too many or
    too few at a window's or a page's edge, or keys read from a wrong page, exceed the bar many
    times over (tests/test_probe_model.py), in bfloat16 too."""
    folder = pm.write_probe_model(str(tmp_path / "probe"))
    vocab = pm.PROBE["vocab_size"]
    requests = make_requests(vocab, PROBE_LENGTHS, seed=8)
    reference = plain_logits(folder, requests)
    steps = schedule_steps(schedule, requests)
    out = str(tmp_path / "out")
    max_tokens = rs.max_tokens_needed(steps, max(64, page))
    if schedule == "mixed":
        assert pages_ever_needed(requests, page) > -(-max_tokens // page)
    replay_in_process(folder, steps, out, dtype, max_tokens, block_size=page)
    worst, where = compare(out, steps, reference, vocab, score=probe_score)
    print(f"probe {schedule} page {page} {dtype}: worst score {worst:.3f} at {where}")
    assert worst <= (1.0 if dtype == "bfloat16" else 0.02), f"score {worst} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    """The bin/trace_run program itself, fed step by step over a pipe."""
    folder = make_folder(tmp_path, "B", seed=2)
    vocab = TINY["B"]["vocab_size"]
    requests = make_requests(vocab, [50, 35, 81], seed=9)
    reference = plain_logits(folder, requests)
    steps = rs.mixed(requests, {r: len(t) - 8 for r, t in requests.items()}, max_live=2)
    out = str(tmp_path / "out")
    replay_program(folder, steps, out, dtype, rs.max_tokens_needed(steps))
    worst, where = compare(out, steps, reference, vocab)
    bar = tolerance(dtype, reference) if dtype == "float32" else \
        bfloat16_bar(folder, requests, reference, vocab, "program")
    assert worst < bar, f"max abs err {worst} at {where}, bar {bar}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_without_attention_bias(tmp_path, dtype):
    """``attention_bias: false``: q, k and v have no bias tensors at all."""
    folder = make_folder(tmp_path, "B", seed=13, attention_bias=False)
    vocab = TINY["B"]["vocab_size"]
    requests = make_requests(vocab, [50, 35, 81, 120], seed=9)
    reference = plain_logits(folder, requests)
    steps = rs.mixed(requests, {r: len(t) - 8 for r, t in requests.items()}, max_live=3)
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, dtype, rs.max_tokens_needed(steps))
    worst, where = compare(out, steps, reference, vocab)
    bar = tolerance(dtype, reference) if dtype == "float32" else \
        bfloat16_bar(folder, requests, reference, vocab, "nobias")
    assert worst < bar, f"max abs err {worst} at {where}"

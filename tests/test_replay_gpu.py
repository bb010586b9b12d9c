"""Trace replay on the GPU, in float32 and in bfloat16: the same requests whole,
with the last 32 tokens decoded one by one, in portions of changing size, and
mixed with so few pages that they are used again, all compared with the plain
implementation."""
import os
import random

import pytest
import torch

import replay_schedules as rs
from replay_harness import compare, plain_logits, replay_in_process, replay_program, tolerance
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B"])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(tmp_path, which, schedule, dtype):
    folder = make_folder(tmp_path, which, seed=11)
    vocab = TINY[which]["vocab_size"]
    requests = make_requests(vocab, LENGTHS[which], seed=5)
    reference = plain_logits(folder, requests)
    steps = schedule_steps(schedule, requests)
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, dtype, rs.max_tokens_needed(steps))
    worst, where = compare(out, steps, reference, vocab)
    print(f"{which} {schedule} {dtype}: max abs err {worst:.3e} at {where}")
    assert worst < tolerance(dtype, reference), f"max abs err {worst} at {where}"


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
    assert worst < tolerance(dtype, reference), f"max abs err {worst} at {where}"

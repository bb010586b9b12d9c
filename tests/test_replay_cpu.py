"""The replay tool over the engine's host side (cache manager, batch packing,
step function) with the kernels emulated in torch on the CPU: every cutting of
the same requests gives the plain implementation's logits."""
import random

import pytest
import torch

import replay_schedules as rs
from emulated_ops import EmulatedOps
from replay_harness import compare, plain_logits, replay_in_process
from tiny_configs import TINY, make_folder


def make_requests(vocab, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


@pytest.mark.parametrize("which", ["A", "B"])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(tmp_path, which, schedule):
    folder = make_folder(tmp_path, which, seed=11)
    vocab = TINY[which]["vocab_size"]
    lengths = [37, 70, 49, 96, 130, 41, 66] if which == "A" else [41, 109, 56, 200, 33, 77]
    requests = make_requests(vocab, lengths, seed=5)
    reference = plain_logits(folder, requests)
    if schedule == "whole":
        steps = rs.whole(requests)
    elif schedule == "tail":
        steps = rs.tail_decoded(requests)
    elif schedule == "portions":
        steps = rs.portions(requests)
    else:
        steps = rs.mixed(requests, {r: max(2, len(t) - 32) for r, t in requests.items()})
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "float32", rs.max_tokens_needed(steps),
                      ops=EmulatedOps(torch.float32), device="cpu")
    worst, where = compare(out, steps, reference, vocab)
    assert worst < 1e-4, f"max abs err {worst} at {where}"


@pytest.mark.parametrize("page", [16, 32, 64])
def test_replay_of_the_probe_model_at_every_page_size(tmp_path, page):
    import probe_model as pm
    from replay_harness import probe_score
    folder = pm.write_probe_model(str(tmp_path / "probe"))
    vocab = pm.PROBE["vocab_size"]
    requests = make_requests(vocab, [150, 61, 333, 97, 260, 48, 129], seed=8)
    reference = plain_logits(folder, requests)
    steps = rs.mixed(requests, {r: max(2, len(t) - 32) for r, t in requests.items()})
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "float32", rs.max_tokens_needed(steps, max(64, page)),
                      ops=EmulatedOps(torch.float32), device="cpu", block_size=page)
    worst, where = compare(out, steps, reference, vocab, score=probe_score)
    assert worst <= 0.02, f"score {worst} at {where}"


def test_replay_without_attention_bias(tmp_path):
    folder = make_folder(tmp_path, "B", seed=13, attention_bias=False)
    from safetensors import safe_open
    with safe_open(folder + "/model.safetensors", "pt") as f:
        assert not any(name.endswith("_proj.bias") for name in f.keys())
    requests = make_requests(TINY["B"]["vocab_size"], [50, 35, 81], seed=9)
    reference = plain_logits(folder, requests)
    steps = rs.mixed(requests, {r: len(t) - 8 for r, t in requests.items()}, max_live=2)
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "float32", rs.max_tokens_needed(steps),
                      ops=EmulatedOps(torch.float32), device="cpu")
    worst, where = compare(out, steps, reference, TINY["B"]["vocab_size"])
    assert worst < 1e-4, f"max abs err {worst} at {where}"

"""The layer sizes of the Qwen2.5-7B shape (hidden 3584, 28 query heads in 4
groups of 7, head size 128, intermediate 18944, vocabulary 152064) with two
layers and random weights: float32 logits equal the plain implementation's to
1e-4 for a whole prompt, token by token and in portions; bfloat16 stays within
its bar.  Reductions of 3584 and 18944 terms and a group size that is no power
of two show what the tiny models cannot."""
import random

import pytest
import torch

import replay_schedules as rs
from replay_harness import compare, plain_logits, replay_in_process, tolerance
from servelab_amd import Qwen2Config, write_random_model

pytestmark = pytest.mark.gpu

WIDE = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=2, hidden_size=3584,
    num_attention_heads=28, num_key_value_heads=4, head_dim=128, intermediate_size=18944,
    vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
    use_sliding_window=False, max_position_embeddings=32768, torch_dtype="float32", eos_token_id=151645)


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("wide") / "model")
    write_random_model(Qwen2Config.from_hf(WIDE), folder, seed=5)
    rng = random.Random(1)
    requests = {"p": [rng.randrange(152064) for _ in range(50)],
                "q": [rng.randrange(152064) for _ in range(21)]}
    return folder, requests, plain_logits(folder, requests)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wide_shape_matches_plain(tmp_path, wide, dtype):
    folder, requests, reference = wide
    steps = [{"step": 0, "entries": [{"id": "p", "tokens": requests["p"][:40], "want": [0, 17, 39]}], "end": []}]
    for i in range(40, 50):                                   # tail token by token, q beside it in portions
        entries = [{"id": "p", "tokens": [requests["p"][i]], "want": [0]}]
        j = i - 40
        if j < 7:
            entries.append({"id": "q", "tokens": requests["q"][3 * j:3 * j + 3], "want": [2]})
        steps.append({"step": len(steps), "entries": entries, "end": ["p"] if i == 49 else []})
    steps[-1]["end"] = ["p", "q"]
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, dtype, rs.max_tokens_needed(steps))
    worst, where = compare(out, steps, reference, 152064)
    print(f"wide {dtype}: max abs err {worst:.3e} at {where}")
    assert worst < tolerance(dtype, reference), f"max abs err {worst} at {where}"


@pytest.fixture(scope="module")
def crowd(wide):
    """One long request and 39 short ones, with the tokens they will be fed."""
    folder, _, _ = wide
    rng = random.Random(2)
    decoded = {"L": 11}
    decoded.update({f"s{i}": 8 if i < 7 else 5 if i < 15 else 2 for i in range(39)})
    requests = {"L": [rng.randrange(152064) for _ in range(1400 + decoded["L"])]}
    for i in range(39):
        requests[f"s{i}"] = [rng.randrange(152064) for _ in range(4 + i % 5 + decoded[f"s{i}"])]
    return folder, requests, decoded, plain_logits(folder, requests)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wide_shape_long_prompt_and_growing_batches(tmp_path, crowd, dtype):
    """What only serving sizes reach: a prompt of 1,400 tokens in one step (the
    library products and the prompt attention that shares keys through LDS, in
    bfloat16), then decode steps of 1, 8, 16 and 40 requests (every form of the
    few-rows products, decode attention over a split context beside short
    ones), with the newcomers' prompts beside the decoded tokens."""
    folder, requests, decoded, reference = crowd
    fed = {r: 0 for r in requests}
    steps = []

    def take(r, n):
        toks = requests[r][fed[r]:fed[r] + n]
        fed[r] += n
        return {"id": r, "tokens": toks, "want": [n - 1]}

    def step(entries):
        steps.append({"step": len(steps), "entries": entries, "end": []})

    live = ["L"]
    step([take("L", 1400)])
    for newcomers in ([], [f"s{i}" for i in range(7)], [f"s{i}" for i in range(7, 15)],
                      [f"s{i}" for i in range(15, 39)]):
        if newcomers:
            step([take(r, len(requests[r]) - decoded[r]) for r in newcomers] + [take(r, 1) for r in live])
            live += newcomers
        step([take(r, 1) for r in live])
        step([take(r, 1) for r in live])
    assert all(fed[r] == len(requests[r]) for r in requests)
    steps[-1]["end"] = list(requests)
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, dtype, rs.max_tokens_needed(steps), max_live=40)
    worst, where = compare(out, steps, reference, 152064)
    print(f"wide, long prompt and batches, {dtype}: max abs err {worst:.3e} at {where}")
    assert worst < tolerance(dtype, reference), f"max abs err {worst} at {where}"

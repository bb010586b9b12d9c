"""The layer sizes of the Qwen2.5-7B shape (hidden 3584, 28 query heads in 4
groups of 7, head size 128, intermediate 18944, vocabulary 152064) with two
layers and random weights: float32 logits equal the plain implementation's to
1e-4 for a whole prompt, token by token and in portions; bfloat16 stays within
its bar.  Reductions of 3584 and 18944 terms and a group size that is no power
of two show what the tiny models cannot.  The widths of the smallest and of the
two largest models of the family (a width that is no multiple of 256, head size
64 and a tied head; 8 kv heads of 5 and of 8 query heads; streams for which the
fused few-rows kernels end at 8 rows, or are not taken at all) run the same kind
of schedule."""
import random

import pytest
import torch

import replay_schedules as rs
from replay_harness import bfloat16_bar, compare, plain_logits, replay_in_process, tolerance
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
    bar = tolerance(dtype, reference) if dtype == "float32" else \
        bfloat16_bar(folder, requests, reference, 152064, "wide")
    print(f"wide {dtype}: max abs err {worst:.3e} at {where}, bar {bar:.3e}")
    assert worst < bar, f"max abs err {worst} at {where}"


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
    bar = tolerance(dtype, reference) if dtype == "float32" else \
        bfloat16_bar(folder, requests, reference, 152064, "crowd")
    print(f"wide, long prompt and batches, {dtype}: max abs err {worst:.3e} at {where}, bar {bar:.3e}")
    assert worst < bar, f"max abs err {worst} at {where}, bar {bar}"


def test_float32_error_at_depth():
    """The float32 path against a float64 run of the plain implementation at 2, 4, 8 and all 28
    layers of the 7B widths (vocabulary cut to 4,099 rows: depth is what is looked at).  The weights are made
    on the device and shared by both sides; the plain implementation runs on the device in float64
    and in float32 (library products, no reduced-precision mode), the latter to show what float32
    arithmetic itself costs at that depth.  Prompt of 48 tokens, then 16 tokens one by one.
    At every depth the error stays below 1e-4 (the bar of the reference's own cross-checks,
    tests/test_parallel.py:103-104) and below what the plain implementation loses by computing
    in float32 itself: the kernels keep their sums of products in segments of 512 terms (and a
    wavefront's lanes each their own share), where a running sum over 3,584 to 18,944 terms
    loses more.  The error grows like the square root of the depth for both."""
    import plain_qwen2 as plain
    from servelab_amd.engine import ModelRunner, StepEntry
    from servelab_amd.engine.session import random_model_on_device
    torch.backends.cuda.matmul.allow_tf32 = False
    rng = random.Random(4)
    toks = [rng.randrange(4099) for _ in range(64)]
    report = {}
    for layers in (2, 4, 8, 28):
        raw = dict(WIDE, num_hidden_layers=layers, vocab_size=4099, eos_token_id=4098)
        cfg = Qwen2Config.from_hf(raw)
        model = random_model_on_device(cfg, 7, "float32")
        from servelab_amd.weights import RandomCheckpoint
        weights = RandomCheckpoint(model.spec.param_specs(), 7, "cuda:0", torch.float32).state_dict()
        exact = plain.forward(raw, weights, toks, dtype=torch.float64)
        plain32 = plain.forward(raw, weights, toks, dtype=torch.float32).double()
        runner = ModelRunner(model, 8, 16)
        rows = [runner.step([StepEntry("a", toks[:48], list(range(48)))])]
        rows += [runner.step([StepEntry("a", [t], [0])]).clone() for t in toks[48:]]
        got = torch.cat(rows).double()
        report[layers] = ((got - exact).abs().max().item(), (plain32 - exact).abs().max().item(),
                          exact.abs().max().item())
        if layers == 28:
            # at the full depth also in portions and mixed: a second request whose portions (down to two
            # tokens) run beside the first one's, which is cut at other places than above
            other = [rng.randrange(4099) for _ in range(41)]
            exact_other = plain.forward(raw, weights, other, dtype=torch.float64)
            runner.close("a")
            cuts_a, cuts_b = [0, 30, 31, 33, 50, 64], [0, 5, 25, 27, 28, 41]
            mixed = 0.0
            for i in range(5):
                ta, tb = toks[cuts_a[i]:cuts_a[i + 1]], other[cuts_b[i]:cuts_b[i + 1]]
                out = runner.step([StepEntry("a", ta, list(range(len(ta)))),
                                   StepEntry("b", tb, list(range(len(tb))))]).double()
                mixed = max(mixed, (out[:len(ta)] - exact[cuts_a[i]:cuts_a[i + 1]]).abs().max().item(),
                            (out[len(ta):] - exact_other[cuts_b[i]:cuts_b[i + 1]]).abs().max().item())
            print(f"float32 at 28 layers, two requests in portions side by side: {mixed:.2e}")
            assert mixed <= 1e-4, mixed
        del model, runner, weights
        torch.cuda.empty_cache()
    for layers, (engine, arithmetic, top) in report.items():
        print(f"float32 at {layers} layers of the 7B widths: engine {engine:.2e}, plain float32 "
              f"{arithmetic:.2e} off the float64 logits (largest {top:.2f})")
    assert all(engine <= 1e-4 for engine, _, _ in report.values()), report
    assert all(engine <= arithmetic for engine, arithmetic, _ in report.values()), report


OTHER_WIDTHS = {
    # hidden 896 is no multiple of 256 (no resident form of the consumer products), head size 64, tied head
    "0.5b": dict(hidden_size=896, num_attention_heads=14, num_key_value_heads=2, head_dim=64, intermediate_size=4864,
                 tie_word_embeddings=True),
    # 8 kv heads of 5 query heads, tiles of 10 rows for the producers of a width of 5,120
    "32b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, head_dim=128, intermediate_size=27648),
    # a stream so wide that no step takes the fused few-rows kernels
    "72b": dict(hidden_size=8192, num_attention_heads=64, num_key_value_heads=8, head_dim=128, intermediate_size=29568),
}


@pytest.mark.parametrize("which", sorted(OTHER_WIDTHS))
def test_other_widths_of_the_family(tmp_path, which):
    """Two layers of the widths of the smallest and of the two largest models of the family (vocabulary cut to
    5,003 rows): a prompt of 300 tokens, then newcomers beside decoded tokens and decode steps of 1, 8,
    16 and 40 requests, in float32 and in bfloat16 against the plain implementation."""
    raw = dict(WIDE, vocab_size=5003, eos_token_id=5002, **OTHER_WIDTHS[which])
    folder = str(tmp_path / "model")
    write_random_model(Qwen2Config.from_hf(raw), folder, seed=6)
    rng = random.Random(3)
    decoded = {"L": 7}
    decoded.update({f"s{i}": 6 if i < 7 else 4 if i < 15 else 2 for i in range(39)})
    requests = {"L": [rng.randrange(5003) for _ in range(300 + decoded["L"])]}
    for i in range(39):
        requests[f"s{i}"] = [rng.randrange(5003) for _ in range(4 + i % 5 + decoded[f"s{i}"])]
    reference = plain_logits(folder, requests)
    fed = {r: 0 for r in requests}
    steps = []

    def take(r, n):
        toks = requests[r][fed[r]:fed[r] + n]
        fed[r] += n
        return {"id": r, "tokens": toks, "want": [n - 1]}

    live = ["L"]
    steps.append({"step": 0, "entries": [take("L", 300)], "end": []})
    for newcomers in ([], [f"s{i}" for i in range(7)], [f"s{i}" for i in range(7, 15)], [f"s{i}" for i in range(15, 39)]):
        if newcomers:
            steps.append({"step": len(steps), "end": [],
                          "entries": [take(r, len(requests[r]) - decoded[r]) for r in newcomers] + [take(r, 1) for r in live]})
            live += newcomers
        steps.append({"step": len(steps), "entries": [take(r, 1) for r in live], "end": []})
    while any(fed[r] < len(requests[r]) for r in requests):
        steps.append({"step": len(steps), "entries": [take(r, 1) for r in live if fed[r] < len(requests[r])], "end": []})
    steps[-1]["end"] = list(requests)
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / ("out_" + dtype))
        replay_in_process(folder, steps, out, dtype, rs.max_tokens_needed(steps), max_live=40)
        worst, where = compare(out, steps, reference, 5003)
        bar = tolerance(dtype, reference) if dtype == "float32" else \
            bfloat16_bar(folder, requests, reference, 5003, ("other widths", which))
        print(f"{which} widths, {dtype}: max abs err {worst:.3e} at {where}, bar {bar:.3e}")
        assert worst < bar, f"{dtype}: max abs err {worst} at {where}, bar {bar}"

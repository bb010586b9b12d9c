"""The whole engine on the GPU, in float32 and in bfloat16: greedy generation
through the entry point, long decoding across graph captures, the first tokens
of a sequence, preemption, sampling with a temperature."""
import random

import pytest
import torch

import plain_qwen2 as plain
import replay_schedules as rs
from replay_harness import bfloat16_bar, compare, plain_logits, replay_in_process, tolerance
from servelab_amd import CacheConfig, LLMEngine, SamplingParams, SchedulerConfig, load_config
from servelab_amd.engine import ModelRunner, StepEntry
from servelab_amd.engine.session import load_model_on_device
from tiny_configs import TINY, make_folder

pytestmark = pytest.mark.gpu
PROMPTS = [list(range(10, 40)), [5, 9, 200, 31], list(range(300, 377)), [7]]


def make_engine(folder, dtype, num_blocks=64, max_batched=256, max_seqs=8):
    return LLMEngine(load_config(folder), CacheConfig(num_blocks=num_blocks),
                     SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=max_batched),
                     dtype=dtype)


def check_greedy(folder, cfg, w, prompt, tokens, dtype):
    """float32: the plain implementation's tokens exactly.  bfloat16: every
    chosen token is, for the plain implementation fed the same tokens, within
    twice the bfloat16 bar of the best logit (each of the two logits may be off
    by the bar; rounding may flip near ties, nothing else may)."""
    if dtype == "float32":
        assert tokens == plain.greedy_generate(cfg, w, prompt, len(tokens))
        return
    whole = list(prompt) + tokens
    logits = plain.forward(cfg, w, whole)
    slack = 2 * bfloat16_bar(folder, {"x": whole}, {"x": logits.numpy()}, cfg["vocab_size"],
                             ("greedy", folder, tuple(whole)))
    for i, t in enumerate(tokens):
        row = logits[len(prompt) - 1 + i]
        assert row[t] >= row.max() - slack, f"token {i}: {row[t]} vs best {row.max()}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_through_the_entry_point(tmp_path, which, dtype):
    folder = make_folder(tmp_path, which, seed=21)
    cfg, w = plain.load_folder(folder)
    vocab = TINY[which]["vocab_size"]
    prompts = [[t % vocab for t in p] for p in PROMPTS]
    outs = make_engine(folder, dtype).generate(prompts, SamplingParams.greedy(12))
    for p, o in zip(prompts, outs):
        assert o.finished and o.outputs[0].finish_reason == "length" and len(o.outputs[0].token_ids) == 12
        check_greedy(folder, cfg, w, p, o.outputs[0].token_ids, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cutting_and_preemption_do_not_change_the_tokens(tmp_path, dtype):
    folder = make_folder(tmp_path, "B", seed=22)
    cfg, w = plain.load_folder(folder)
    base = [o.outputs[0].token_ids for o in
            make_engine(folder, dtype).generate(PROMPTS, SamplingParams.greedy(12))]
    for p, t in zip(PROMPTS, base):
        check_greedy(folder, cfg, w, p, t, dtype)
    if dtype == "float32":
        small = make_engine(folder, dtype, max_batched=8)
        assert [o.outputs[0].token_ids for o in small.generate(PROMPTS, SamplingParams.greedy(12))] == base
        tight = make_engine(folder, dtype, num_blocks=9, max_batched=64)
        assert [o.outputs[0].token_ids for o in tight.generate(PROMPTS, SamplingParams.greedy(12))] == base
        assert tight.stats()["num_preemptions_total"] > 0
        tight.runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,page", [("A", 16), ("B", 16), ("B", 32), ("A", 64), ("B", 64)])
def test_long_decoding_across_graph_captures(tmp_path, which, page, dtype, monkeypatch):
    """A short prompt, then 200 tokens one by one: the context outgrows the
    captured graphs' capacity several times (64 -> 128 -> 256), and two requests
    decode side by side in one graph."""
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 64)
    folder = make_folder(tmp_path, which, seed=23)
    vocab = TINY[which]["vocab_size"]
    rng = random.Random(3)
    requests = {r: [rng.randrange(vocab) for _ in range(n)] for r, n in (("x", 230), ("y", 215))}
    reference = plain_logits(folder, requests)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": requests["x"][:20], "want": [19]},
                                     {"id": "y", "tokens": requests["y"][:5], "want": [4]}], "end": []}]
    for i in range(210):
        steps.append({"step": i + 1, "entries": [
            {"id": "x", "tokens": [requests["x"][20 + i]], "want": [0]},
            {"id": "y", "tokens": [requests["y"][5 + i]], "want": [0]}],
            "end": ["x", "y"] if i == 209 else []})
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, dtype, rs.max_tokens_needed(steps), block_size=page)
    worst, where = compare(out, steps, reference, vocab)
    bar = tolerance(dtype, reference) if dtype == "float32" else \
        bfloat16_bar(folder, requests, reference, vocab, ("long", which))
    assert worst < bar, f"max abs err {worst} at {where}, bar {bar}"


def test_long_decoding_in_shares_of_one_length(tmp_path, monkeypatch):
    """Four requests of very different lengths decoded side by side through the captured graphs with the
    single tokens' keys in shares of one length for all sequences (a table told that it has 2 CUs, so
    that four pairs are more than it has; the sums the kernel balances by change with every replay)."""
    from servelab_amd.kernels import HipOps, Tuning
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 64)
    folder = make_folder(tmp_path, "B", seed=31, use_sliding_window=False)
    vocab = TINY["B"]["vocab_size"]
    rng = random.Random(6)
    starts = {"p": 400, "q": 3, "r": 70, "s": 33}
    requests = {r: [rng.randrange(vocab) for _ in range(n + 100)] for r, n in starts.items()}
    reference = plain_logits(folder, requests)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": requests[r][:n], "want": [n - 1]} for r, n in starts.items()],
              "end": []}]
    for i in range(100):
        steps.append({"step": i + 1, "entries": [{"id": r, "tokens": [requests[r][n + i]], "want": [0]}
                                                 for r, n in starts.items()],
                      "end": list(starts) if i == 99 else []})
    ops = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(shares_of_one_length=True))
    ops._num_cus = 2
    told = []
    call = ops._call
    ops._call = lambda stem, name, *args: (told.append(args[-1]) if name.startswith("sl_attention_mfma@") and args[10] == 1
                                           else None, call(stem, name, *args))[1]
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "bfloat16", rs.max_tokens_needed(steps), block_size=16, ops=ops)
    assert told and any(told)                        # (launches that were told the wavefronts to aim at)
    worst, where = compare(out, steps, reference, vocab)
    bar = bfloat16_bar(folder, requests, reference, vocab, "one length")
    assert worst < bar, f"max abs err {worst} at {where}, bar {bar}"


@pytest.mark.parametrize("page,other", [(32, {}), (16, dict(head_dim=64, num_key_value_heads=2, use_sliding_window=False))])
def test_long_decoding_with_the_keys_merged_inside_the_workgroup(tmp_path, page, other, monkeypatch):
    """The decode attention that a large batch takes by itself (a workgroup of eight wavefronts per
    request and kv head, merged in LDS), asked for at four requests: a prompt each, then 150 tokens
    one by one through the captured graphs, contexts from 3 to 190 keys (fewer key blocks than
    wavefronts for most of the run); the configuration whose head size the matrix-core kernels take, with
    its window in one layer, and the same with two kv heads of 64 and no window."""
    from servelab_amd.kernels import HipOps, Tuning
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 64)
    folder = make_folder(tmp_path, "B", seed=29, **other)
    vocab = TINY["B"]["vocab_size"]
    rng = random.Random(5)
    starts = {"p": 40, "q": 3, "r": 17, "s": 33}
    requests = {r: [rng.randrange(vocab) for _ in range(n + 150)] for r, n in starts.items()}
    reference = plain_logits(folder, requests)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": requests[r][:n], "want": [n - 1]} for r, n in starts.items()],
              "end": []}]
    for i in range(150):
        steps.append({"step": i + 1, "entries": [{"id": r, "tokens": [requests[r][n + i]], "want": [0]}
                                                 for r, n in starts.items()],
                      "end": list(starts) if i == 149 else []})
    ops = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(group_attention_fill=0.0))
    merged = []
    call = ops._call
    ops._call = lambda stem, name, *args: (merged.append(args[-3]) if name.startswith("sl_attention_mfma@") and args[10] == 1
                                           else None, call(stem, name, *args))[1]
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "bfloat16", rs.max_tokens_needed(steps), block_size=page, ops=ops)
    assert merged and all(merged)                    # (every launch over single tokens took that form)
    worst, where = compare(out, steps, reference, vocab)
    bar = bfloat16_bar(folder, requests, reference, vocab, ("merged", page))
    assert worst < bar, f"max abs err {worst} at {where}, bar {bar}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_equals_eager(tmp_path, dtype):
    """The same decode steps with and without graphs; the graph is replayed
    several times with the program's own eager work between the replays."""
    folder = make_folder(tmp_path, "B", seed=24)
    _, model = load_model_on_device(folder, dtype)
    runs = {}
    for use_graphs in (False, True):
        runner = ModelRunner(model, 64, 16, use_graphs=use_graphs)
        rows = []
        runner.step([StepEntry("a", list(range(50)), []), StepEntry("b", list(range(7)), [])])
        for i in range(12):
            rows.append(runner.step([StepEntry("a", [100 + i], [0]), StepEntry("b", [200 + i], [0])]).clone())
            if i % 4 == 3:            # an eager mixed step in between
                rows.append(runner.step([StepEntry("c", [1, 2, 3 + i], [2])]).clone())
                runner.close("c")
        runs[use_graphs] = torch.cat(rows)
        if use_graphs:
            assert runner.graph_replays >= 10
    if dtype == "float32":
        assert torch.equal(runs[True], runs[False])
    else:        # the captured decode attention splits the context differently: rounding only
        assert (runs[True] - runs[False]).abs().max().item() < 1e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_graphs_are_bounded(tmp_path, dtype, monkeypatch):
    """More graph keys (requests x context capacity) than the memory limit holds: the graphs used
    longest ago are dropped and captured again when their shape returns; logits equal those of a
    runner without graphs throughout, and device memory does not grow from one round to the next."""
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 32)
    folder = make_folder(tmp_path, "B", seed=28)
    _, model = load_model_on_device(folder, dtype)
    vocab = TINY["B"]["vocab_size"]
    eager = ModelRunner(model, 64, 16, use_graphs=False)
    graphs = ModelRunner(model, 64, 16, use_graphs=True)
    per_graph = vocab * 4 * 3 + 4096
    graphs.graph_memory_limit = 3 * per_graph            # the six keys together need four times a graph of 3
    rng = random.Random(5)

    def one_round(tag):
        worst = 0.0
        for batch in (1, 2, 3, 2, 1, 3):                  # with two context capacities each: 6 keys
            ids = [f"{tag}{batch}_{i}" for i in range(batch)]
            prompt = [[rng.randrange(vocab) for _ in range(20 + 3 * i)] for i in range(batch)]
            for r in (eager, graphs):
                r.step([StepEntry(i, p, []) for i, p in zip(ids, prompt)])
            for _ in range(16):                           # contexts cross 32: a second capacity
                toks = [rng.randrange(vocab) for _ in ids]
                a = eager.step([StepEntry(i, [t], [0]) for i, t in zip(ids, toks)])
                b = graphs.step([StepEntry(i, [t], [0]) for i, t in zip(ids, toks)])
                worst = max(worst, (a - b).abs().max().item())
            for i in ids:
                eager.close(i), graphs.close(i)
        return worst

    assert one_round("a") <= (0.0 if dtype == "float32" else 1e-2)
    torch.cuda.synchronize()
    held, evicted = torch.cuda.memory_allocated(), graphs.graph_evictions
    assert evicted > 0 and len(graphs._graphs) < 6 and graphs._graph_bytes <= graphs.graph_memory_limit
    assert one_round("b") <= (0.0 if dtype == "float32" else 1e-2)
    torch.cuda.synchronize()
    assert graphs.graph_evictions > evicted and graphs._graph_bytes <= graphs.graph_memory_limit
    assert torch.cuda.memory_allocated() <= held + (1 << 20)
    assert graphs.graph_replays > 100


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B"])
def test_first_tokens_of_a_sequence(tmp_path, which, dtype):
    """Position 0 alone, then 1, 2, 3...: a prompt of one token, portions of one."""
    folder = make_folder(tmp_path, which, seed=25)
    vocab = TINY[which]["vocab_size"]
    requests = {"s": [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7, 9, 3, 2, 3, 8, 4]}
    reference = plain_logits(folder, requests)
    steps = [{"step": i, "entries": [{"id": "s", "tokens": [t], "want": [0]}],
              "end": ["s"] if i == 19 else []} for i, t in enumerate(requests["s"])]
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, dtype, 64)
    worst, where = compare(out, steps, reference, vocab)
    bar = tolerance(dtype, reference) if dtype == "float32" else \
        bfloat16_bar(folder, requests, reference, vocab, ("first", which))
    assert worst < bar, f"max abs err {worst} at {where}, bar {bar}"


def test_temperature_sampling_through_the_engine(tmp_path):
    folder = make_folder(tmp_path, "A", seed=26)
    eng = make_engine(folder, "float32")
    sp = SamplingParams(temperature=0.8, max_tokens=8, seed=7, ignore_eos=True)
    a = eng.generate([PROMPTS[0]], sp)[0].outputs[0].token_ids
    b = eng.generate([PROMPTS[0], PROMPTS[1]], sp)[0].outputs[0].token_ids
    assert a == b                                    # a seeded request does not depend on its batch
    hot = SamplingParams(temperature=1.5, max_tokens=8, ignore_eos=True)
    c = eng.generate([PROMPTS[0]], hot)[0].outputs[0].token_ids
    d = eng.generate([PROMPTS[0]], hot)[0].outputs[0].token_ids
    assert c != d                                    # unseeded requests draw from the engine's stream
    k1 = SamplingParams(temperature=1.0, top_k=1, max_tokens=8, ignore_eos=True)
    greedy = eng.generate([PROMPTS[0]], SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))
    assert eng.generate([PROMPTS[0]], k1)[0].outputs[0].token_ids == greedy[0].outputs[0].token_ids


def test_tiled_only_weight_layout_runs_the_whole_model(tmp_path, monkeypatch):
    """A model too large for two copies of its matrices keeps only the tiled
    one: prompts go through the row-major scratch, decode straight to the matrix
    cores; logits equal those with both copies.  (No further copies in lower
    tiles here, which only the model with two copies would make: they group
    the sums of squares of the stream differently; the products in tiles
    over the row-major copy, which a model without that copy cannot take, are
    for larger matrices than this model has.)"""
    from servelab_amd.kernels import HipOps, Tuning
    folder = make_folder(tmp_path, "B", seed=27)
    toks = list(range(100, 180))
    rows = {}
    for share in (0.45, 0.0):
        ops = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(dual_memory_share=share, lower_tiles_min_gain=1.0,
                                                             rows_copies_memory_share=0.0))
        _, model = load_model_on_device(folder, "bfloat16", ops=ops)
        assert model.rt.ops.layout_summary() == ("dual" if share else "tiled")
        runner = ModelRunner(model, 16, 16)
        out = [runner.step([StepEntry("a", toks[:70], [0, 69])])]
        out += [runner.step([StepEntry("a", [t], [0])]).clone() for t in toks[70:]]
        rows[share] = torch.cat(out)
    assert torch.equal(rows[0.45], rows[0.0])
    # with room for some row-major copies beside the tiled ones, the first matrices loaded keep theirs
    # (here: room for four of the model's matrices) and their many-row products skip the scratch buffer
    total = torch.cuda.get_device_properties(0).total_memory
    cfg = load_config(folder)
    sizes = [s.shape[0] * s.shape[1] * 2 for s in model.spec.param_specs().values() if len(s.shape) == 2]
    room = (sum(sizes) + 2.5 * max(sizes)) / total
    ops = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(dual_memory_share=0.0, lower_tiles_min_gain=1.0,
                                                         rows_copies_memory_share=room))
    _, some = load_model_on_device(folder, "bfloat16", ops=ops, config=cfg)
    assert ops.weight_layout == "tiled" and 0 < ops._matrices_with_rows < ops._matrices
    assert "also row-major" in ops.layout_summary()
    runner = ModelRunner(some, 16, 16)
    out = [runner.step([StepEntry("a", toks[:70], [0, 69])])]
    out += [runner.step([StepEntry("a", [t], [0])]).clone() for t in toks[70:]]
    assert torch.equal(torch.cat(out), rows[0.0])


def test_tuned_library_products_keep_the_logits(tmp_path):
    """Start-up tuning of the library's kernels for a prompt portion of a given
    size: the portion's logits stay within rounding of the untuned ones and of
    the plain implementation, the choices land in a file under the temporary
    folder, and lengths the pool cannot hold are left out."""
    import os
    import tempfile
    folder = make_folder(tmp_path, "B", seed=31)
    cfg, weights = plain.load_folder(folder)
    toks = [(7 * i + 3) % cfg["vocab_size"] for i in range(96)]
    _, model = load_model_on_device(folder, "bfloat16")
    runner = ModelRunner(model, 16, 16)
    before = runner.step([StepEntry("a", toks, [0, 50, 95])]).clone()
    runner.close("a")
    assert runner.tune_products([96, 100000], max_ms=3) == [96]
    assert runner.manager.num_free_pages() == 16
    after = runner.step([StepEntry("b", toks, [0, 50, 95])])
    whole = plain.forward(cfg, weights, toks)
    tol = bfloat16_bar(folder, {"a": toks}, {"a": whole.numpy()}, cfg["vocab_size"], "tuned")
    assert (after.cpu() - whole[[0, 50, 95]]).abs().max().item() < tol
    assert (after - before).abs().max().item() < tol
    name = os.path.join(tempfile.gettempdir(), f"servelab_amd_tunableop_{os.getuid()}.csv")
    assert os.path.exists(name)


@pytest.mark.parametrize("pattern", ["fixed", "poisson"])
def test_load_benchmark_on_a_tiny_model(tmp_path, pattern):
    """The load benchmark drives the real engine: every request comes back with
    its number of tokens, and the figures are those of its outputs."""
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench_serving as bs
    folder = make_folder(tmp_path, "B", seed=31)
    args = bs.parser().parse_args([
        "--model", folder, "--num-prompts", "9", "--input-mean", "60", "--output-tokens", "10",
        "--load-pattern", pattern, "--concurrency", "3", "--request-rate", "400",
        "--num-blocks", "96", "--max-num-seqs", "4", "--max-batched-tokens", "64",
        "--warmup-requests", "2", "--temperature", "0.7", "--top-p", "0.9"])
    res = bs.run(args)
    want = bs.synthetic_requests(9, TINY["B"]["vocab_size"], 60, 10, 42,
                                 longest=TINY["B"]["max_position_embeddings"])
    assert res["requests"] == 9 and res["output_tokens"] == sum(r.output_tokens for r in want)
    assert res["output_throughput_tok_s"] > 0 and res["ttft_ms_p50"] > 0 and res["tpot_ms_p50"] > 0
    assert res["ttft_ms_p99"] >= res["ttft_ms_p50"] and res["steps"] > 0


def test_decode_graphs_of_a_hundred_requests():
    """With matrices large enough for the LDS-staged kernel, decode steps of 65
    to 128 requests hold no library product and replay a graph: same logits as
    the eager steps, and as each request stepped alone."""
    from servelab_amd import Qwen2Config
    from servelab_amd.engine.session import random_model_on_device
    raw = dict(TINY["B"], num_hidden_layers=1, hidden_size=3072, num_attention_heads=24,
               num_key_value_heads=4, head_dim=128, intermediate_size=3072, vocab_size=4096,
               use_sliding_window=False, max_position_embeddings=4096)
    model = random_model_on_device(Qwen2Config.from_hf(raw), 5, "bfloat16")
    assert model.rt.ops.graph_rows_limit == 128
    B = 100
    rng = random.Random(9)
    prompts = {f"r{i}": [rng.randrange(4096) for _ in range(3 + i % 5)] for i in range(B)}
    runs = {}
    for use_graphs in (False, True):
        runner = ModelRunner(model, 2 * B + 8, 16, max_num_seqs=B, use_graphs=use_graphs)
        for r, p in prompts.items():
            assert runner.open(r)
        runner.step([StepEntry(r, p, []) for r, p in prompts.items()])
        rows = [runner.step([StepEntry(r, [(7 * i + j) % 4096], [0]) for j, r in enumerate(prompts)]).clone()
                for i in range(4)]
        runs[use_graphs] = torch.stack(rows)
        assert runner.graph_replays == (3 if use_graphs else 0)
    assert torch.equal(runs[True], runs[False])
    # request 17 alone: the few-rows kernels of one row, not the 128-row one
    runner = ModelRunner(model, 16, 16, use_graphs=False)
    runner.open("solo")
    runner.step([StepEntry("solo", prompts["r17"], [])])
    for i in range(4):
        alone = runner.step([StepEntry("solo", [(7 * i + 17) % 4096], [0])])[0]
        assert (alone - runs[True][i, 17]).abs().max().item() < 0.05 * alone.abs().max().item()


def test_many_requests_under_three_regimes_generate_the_same_tokens(tmp_path):
    """Sixty requests of random lengths, float32, greedy: with room for all, with
    a fifth of the pages (preemption and recomputation) and with few requests
    and small portions at a time, every request generates the same tokens; no
    page is left held."""
    folder = make_folder(tmp_path, "B", seed=41)
    vocab = TINY["B"]["vocab_size"]
    rng = random.Random(12)
    prompts = [[rng.randrange(vocab) for _ in range(max(1, int(rng.gauss(60, 35))))] for _ in range(60)]
    lengths = [max(1, int(rng.gauss(20, 9))) for _ in prompts]
    need = sum(-(-(len(p) + n) // 16) for p, n in zip(prompts, lengths))
    results = {}
    for name, seqs, budget, blocks in (("roomy", 32, 512, need + 8), ("tight", 32, 128, need // 5),
                                       ("narrow", 4, 24, need // 3)):
        eng = LLMEngine(load_config(folder), CacheConfig(num_blocks=blocks),
                        SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=budget), dtype="float32")
        ids = [eng.add_request(prompt_token_ids=p, sampling_params=SamplingParams.greedy(n))
               for p, n in zip(prompts, lengths)]
        done = {}
        while eng.has_unfinished():
            for o in eng.step():
                done[o.request_id] = o
        eng.runner.manager.check()
        stats = eng.stats()
        assert set(stats["pages_in_use"]) == {0}
        results[name] = [done[i].outputs[0].token_ids for i in ids]
        # EOS may end a request early; otherwise it has its number of tokens
        assert all(len(t) == n or done[i].outputs[0].finish_reason == "eos"
                   for t, n, i in zip(results[name], lengths, ids))
        if name == "tight":
            assert stats["num_preemptions_total"] > 0
    assert results["tight"] == results["roomy"]
    assert results["narrow"] == results["roomy"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_command_line_generates_the_plain_tokens(dtype, capsys, tmp_path):
    """``run_engine`` itself on the GPU, on its tiny default model with random weights made on the
    device (examples/run_engine.py:27-72): the printed tokens are the plain implementation's."""
    import re
    import servelab_amd.cli as cli
    from servelab_amd import Qwen2Config
    from servelab_amd.parts import build_model_spec
    from servelab_amd.weights import RandomCheckpoint
    assert cli.main(["--random-weights", "3", "--temperature", "0", "--max-tokens", "10",
                     "--dtype", dtype, "--num-blocks", "32"]) == 0
    printed = capsys.readouterr().out
    got = [int(t) for t in re.search(r"\[req-1\] finish=(\w+) -> \[([0-9, ]+)\]", printed).group(2).split(",")]
    raw = dict(cli.TINY_DEFAULT)
    spec = build_model_spec(Qwen2Config.from_hf(raw))
    weights = {n: t.float().cpu() for n, t in RandomCheckpoint(
        spec.param_specs(), 3, "cuda:0",
        torch.float32 if dtype == "float32" else torch.bfloat16).state_dict().items()}
    prompt = [t % raw["vocab_size"] for t in range(10, 40)]
    assert "stats:" in printed and "[step 1]" in printed
    if dtype == "float32":
        want = plain.greedy_generate(raw, weights, prompt, 10)
        assert got == want[:len(got)] and (len(got) == 10 or got[-1] == raw["eos_token_id"])
    else:
        # the same weights as a folder, for the bar: every token within twice the bfloat16 bar of the best
        import json
        from servelab_amd.weights.safetensors_io import write_safetensors
        folder = str(tmp_path)
        write_safetensors(str(tmp_path / "model.safetensors"),
                          {n: t.to(torch.bfloat16) for n, t in weights.items()})
        with open(tmp_path / "config.json", "w") as f:
            json.dump(raw, f)
        check_greedy(folder, raw, weights, prompt, got, dtype)


def test_graphs_captured_at_start_up_are_the_ones_requests_then_replay(tmp_path, monkeypatch):
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 32)
    folder = make_folder(tmp_path, "B", seed=29)
    cfg, w = plain.load_folder(folder)
    eng = LLMEngine(load_config(folder), CacheConfig(num_blocks=64),
                    SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64), dtype="float32",
                    capture_graphs_up_to=128)
    assert eng.graphs_captured == 4 * 3 and len(eng.runner._graphs) == 12     # 1..4 requests x {32, 64, 128}
    assert eng.runner.manager.num_free_pages() == 64
    eng.runner.manager.check()
    outs = eng.generate(PROMPTS, SamplingParams.greedy(12))
    for p, o in zip(PROMPTS, outs):
        assert o.outputs[0].token_ids == plain.greedy_generate(cfg, w, p, 12)
    assert len(eng.runner._graphs) == 12 and eng.runner.graph_replays >= 10   # nothing new was captured


def test_graphs_captured_at_start_up_stop_at_the_memory_limit(tmp_path, monkeypatch):
    """Start-up capture counts what a graph really keeps (logits and metadata) and drops nothing
    to make room: it stops before the limit, and the count it reports is what is held."""
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 32)
    folder = make_folder(tmp_path, "B", seed=29)
    _, model = load_model_on_device(folder, "float32")
    runner = ModelRunner(model, 64, 16, max_num_seqs=4)
    vocab = TINY["B"]["vocab_size"]
    runner.graph_memory_limit = 5 * (2 * vocab * 4) + 2048       # logits of five graphs of two rows, no more
    made = runner.capture_graphs(range(1, 5), 128)
    assert 0 < made < 12 and made == len(runner._graphs) and runner.graph_evictions == 0
    assert runner._graph_bytes <= runner.graph_memory_limit
    assert runner._graph_bytes == sum(runner._entry_bytes(e[1], k[0]) for k, e in runner._graphs.items())
    assert runner.manager.num_free_pages() == 64
    runner.manager.check()


def test_seeded_draws_with_and_without_the_step_ahead(tmp_path):
    """Temperature, top-k and top-p requests of different lengths, one ended by a stop token: the
    engine that decodes a step ahead (draw counters of tokens the host has not seen, rows gathered
    once a request has left) gives the tokens of the engine that waits for every step."""
    folder = make_folder(tmp_path, "B", seed=33)
    params = [SamplingParams(temperature=0.9, max_tokens=24, seed=11),
              SamplingParams(temperature=1.3, top_k=5, max_tokens=7, seed=12),
              SamplingParams(temperature=0.8, top_p=0.7, max_tokens=15, seed=13),
              SamplingParams(temperature=0.0, max_tokens=19),
              SamplingParams(temperature=1.1, max_tokens=30)]              # unseeded: the engine's stream
    prompts = PROMPTS + [[3, 1, 4, 1, 5, 9, 2, 6]]

    def run(ahead, stop=()):
        eng = LLMEngine(load_config(folder), CacheConfig(num_blocks=64),
                        SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=64), dtype="float32",
                        run_ahead=ahead, seed=77)
        ids = []
        for p, sp in zip(prompts, params):
            sp = SamplingParams(temperature=sp.temperature, top_k=sp.top_k, top_p=sp.top_p,
                                max_tokens=sp.max_tokens, seed=sp.seed, stop_token_ids=tuple(stop))
            ids.append(eng.add_request(prompt_token_ids=p, sampling_params=sp))
        done = {o.request_id: o.outputs[0] for o in eng.run()}
        assert eng._flight is None and set(eng.stats()["pages_in_use"]) == {0}
        eng.runner.manager.check()
        return [(done[i].token_ids, done[i].finish_reason) for i in ids], eng.runner.graph_replays

    waited, _ = run(False)
    ahead, replays = run(True)
    assert ahead == waited and replays > 20
    assert len({tuple(t) for t, _ in waited}) == 5
    stop = waited[0][0][9]
    cut, _ = run(False, stop=(stop,))
    assert cut[0][1] == "eos" and len(cut[0][0]) <= 10
    assert run(True, stop=(stop,))[0] == cut


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_abort_while_two_steps_are_queued(tmp_path, dtype):
    """A request is aborted while a step and the step ahead of it are still queued on the
    device: its pages are free at once and go to a newcomer, whose prompt is written after those
    steps in stream order.  The others' tokens and the newcomer's are the plain ones."""
    folder = make_folder(tmp_path, "B", seed=34)
    cfg, w = plain.load_folder(folder)
    vocab = TINY["B"]["vocab_size"]
    rng = random.Random(9)
    prompts = [[rng.randrange(vocab) for _ in range(n)] for n in (60, 45, 30, 58)]
    eng = LLMEngine(load_config(folder), CacheConfig(num_blocks=14),       # 224 tokens: tight for four
                    SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=128), dtype=dtype)
    ids = [eng.add_request(prompt_token_ids=p, sampling_params=SamplingParams.greedy(16))
           for p in prompts[:3]]
    done = {}
    for _ in range(5):
        for o in eng.step():
            done[o.request_id] = o
    assert eng._flight is not None                    # a step ahead is queued; the device may still run the one before
    free = eng.runner.manager.num_free_pages()
    assert eng.abort_request(ids[0]) and eng.runner.manager.num_free_pages() > free
    ids.append(eng.add_request(prompt_token_ids=prompts[3], sampling_params=SamplingParams.greedy(16)))
    for o in eng.run():
        done[o.request_id] = o
    assert done[ids[0]].outputs[0].finish_reason == "aborted"
    # the newcomer took pages the aborted request had held
    assert eng.runner.manager.page_groups[0].allocator.high_water <= 14
    for i in (1, 2, 3):
        out = done[ids[i]].outputs[0]
        assert out.finish_reason == "length" and len(out.token_ids) == 16
        check_greedy(folder, cfg, w, prompts[i], out.token_ids, dtype)
    part = done[ids[0]].outputs[0].token_ids
    check_greedy(folder, cfg, w, prompts[0], part, dtype)
    assert set(eng.stats()["pages_in_use"]) == {0}
    eng.runner.manager.check()

"""The engine above the kernels (entry point, scheduler, step function, cache)
with the kernels emulated on the CPU: greedy generation equals the plain
implementation's however the work is cut (no GPU).  After the reference's
tests/test_engine_smoke.py:57-134 and tests/test_speculative.py:41-49."""
import pytest
import torch

import plain_qwen2 as plain
from emulated_ops import EmulatedOps
from servelab_amd import CacheConfig, LLMEngine, SamplingParams, SchedulerConfig, load_config
from servelab_amd.engine import ModelRunner, OutOfPages, StepEntry
from servelab_amd.engine.session import load_model_on_device
from tiny_configs import make_folder


def make_engine(folder, num_blocks=64, max_batched=256, max_seqs=8, block_size=16, chunked=True,
                policy="fcfs", run_ahead=True, predictor=None):
    return LLMEngine(load_config(folder), CacheConfig(block_size=block_size, num_blocks=num_blocks),
                     SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=max_batched,
                                     chunked_prefill=chunked, policy=policy),
                     device="cpu", dtype="float32", ops=EmulatedOps(), run_ahead=run_ahead,
                     predictor=predictor)


PROMPTS = [list(range(10, 40)), [5, 9, 200, 31], list(range(300, 377)), [7]]


@pytest.fixture(scope="module")
def folder_and_plain(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("m"), "B", seed=21)
    cfg, w = plain.load_folder(folder)
    want = [plain.greedy_generate(cfg, w, p, 12) for p in PROMPTS]
    return folder, want


def test_greedy_generation_matches_plain(folder_and_plain):
    folder, want = folder_and_plain
    outs = make_engine(folder).generate(PROMPTS, SamplingParams.greedy(12))
    assert [o.outputs[0].token_ids for o in outs] == want
    assert all(o.finished and o.outputs[0].finish_reason == "length" for o in outs)
    assert [o.prompt_token_ids for o in outs] == PROMPTS


@pytest.mark.parametrize("max_batched,max_seqs", [(8, 8), (48, 2), (3, 4)])
def test_any_cutting_gives_the_same_tokens(folder_and_plain, max_batched, max_seqs):
    folder, want = folder_and_plain
    eng = make_engine(folder, max_batched=max_batched, max_seqs=max_seqs)
    outs = eng.generate(PROMPTS, SamplingParams.greedy(12))
    assert [o.outputs[0].token_ids for o in outs] == want


def test_engine_from_one_record(folder_and_plain):
    from servelab_amd import EngineConfig
    folder, want = folder_and_plain
    ec = EngineConfig(cache=CacheConfig(num_blocks=32), scheduler=SchedulerConfig(max_num_seqs=2),
                      seed=5, dtype="float32", device="cpu", run_ahead=False)
    eng = LLMEngine.from_engine_config(load_config(folder), ec, ops=EmulatedOps())
    assert (eng.num_blocks, eng.scheduler.cfg.max_num_seqs, eng.sampler.seed, eng.run_ahead) == (32, 2, 5, False)
    outs = eng.generate(PROMPTS[:2], SamplingParams.greedy(12))
    assert [o.outputs[0].token_ids for o in outs] == want[:2]


def test_preemption_keeps_outputs_whole(folder_and_plain):
    folder, want = folder_and_plain
    eng = make_engine(folder, num_blocks=9, max_batched=64)      # 144 tokens of cache for 4 requests
    outs = eng.generate(PROMPTS, SamplingParams.greedy(12))
    assert [o.outputs[0].token_ids for o in outs] == want
    assert eng.stats()["num_preemptions_total"] > 0
    assert sum(o.metrics["preemptions"] for o in outs) == eng.stats()["num_preemptions_total"]
    eng.runner.manager.check()
    assert eng.runner.manager.num_free_pages() == 9


def test_running_requests_keep_the_invariant(folder_and_plain):
    folder, _ = folder_and_plain
    eng = make_engine(folder, max_batched=16)
    for p in PROMPTS:
        eng.add_request(prompt_token_ids=p, sampling_params=SamplingParams.greedy(5))
    while eng.has_unfinished():
        eng.step()
        ahead = {it.request.request_id for it in eng._flight.plan.items()} if eng._flight else set()
        for r in eng.scheduler.active:                # tests/test_engine_smoke.py:113-127
            # (a request in the step that runs ahead has that step's token in the cache already)
            assert r.owed >= 1
            assert eng.runner.manager.length(r.request_id) == r.cached + (r.request_id in ahead)


@pytest.mark.parametrize("max_seqs,num_blocks", [(2, 64), (8, 9)])
def test_whole_prompts_mode_finishes_under_full_slots_and_a_tight_pool(folder_and_plain, max_seqs,
                                                                       num_blocks):
    """chunked_prefill off with more requests than slots, and with a pool that cannot hold them
    all: prompts run whole, decoding goes on while nothing can be admitted, tokens are plain's."""
    folder, want = folder_and_plain
    eng = make_engine(folder, chunked=False, max_seqs=max_seqs, num_blocks=num_blocks, max_batched=32)
    outs = eng.generate(PROMPTS, SamplingParams.greedy(12))
    assert [o.outputs[0].token_ids for o in outs] == want
    eng.runner.manager.check()
    assert eng.runner.manager.num_free_pages() == num_blocks


def test_priority_policy_serves_the_smaller_value_first(folder_and_plain):
    folder, want = folder_and_plain
    eng = make_engine(folder, policy="priority", max_seqs=1)
    ids = [eng.add_request(prompt_token_ids=p, sampling_params=SamplingParams.greedy(12),
                           priority=pr) for p, pr in zip(PROMPTS, (3, 0, 2, 1))]
    order, done = [], {}
    while eng.has_unfinished():
        for out in eng.step():
            order.append(out.request_id)
            done[out.request_id] = out.outputs[0].token_ids
    assert order == [ids[1], ids[3], ids[2], ids[0]]
    assert [done[i] for i in ids] == want


def test_predicted_shortest_job_first_through_the_engine(folder_and_plain):
    # servelab/engine/engine.py:51,131: the engine hands its predictor to the scheduler
    folder, want = folder_and_plain

    class ByPromptLength:
        def predict_remaining(self, req):
            return req.prompt_len

    with pytest.raises(ValueError, match="requires an output-length predictor"):
        make_engine(folder, policy="sjf-predicted")
    eng = make_engine(folder, policy="sjf-predicted", max_seqs=1, predictor=ByPromptLength())
    ids = [eng.add_request(prompt_token_ids=p, sampling_params=SamplingParams.greedy(12)) for p in PROMPTS]
    order, done = [], {}
    while eng.has_unfinished():
        for out in eng.step():
            order.append(out.request_id)
            done[out.request_id] = out.outputs[0].token_ids
    assert order == [ids[3], ids[1], ids[0], ids[2]]          # prompts of 1, 4, 30 and 77 tokens
    assert [done[i] for i in ids] == want


def test_eos_stops_and_stays_in_the_output(folder_and_plain):
    folder, want = folder_and_plain
    eng = make_engine(folder)
    stop = want[0][3]
    first = want[0].index(stop)
    out = eng.generate([PROMPTS[0]], SamplingParams(temperature=0.0, max_tokens=12,
                                                    stop_token_ids=(stop,)))[0]
    assert out.outputs[0].token_ids == want[0][:first + 1] and out.outputs[0].finish_reason == "eos"


def test_abort_and_oversize(folder_and_plain):
    folder, _ = folder_and_plain
    eng = make_engine(folder, num_blocks=4)
    rid = eng.add_request(prompt_token_ids=PROMPTS[0], sampling_params=SamplingParams.greedy(4))
    eng.step()
    assert eng.abort_request(rid) and not eng.has_unfinished()
    assert eng.runner.manager.num_free_pages() == 4
    outs = eng.generate([list(range(100)), [1, 2, 3]], SamplingParams.greedy(2))
    assert outs[0].outputs[0].finish_reason == "aborted" and outs[0].outputs[0].token_ids == []
    assert outs[1].outputs[0].finish_reason == "length"
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request(prompt_token_ids=[1000])
    with pytest.raises(ValueError, match="tokenizer"):
        eng.add_request(prompt="text")


def test_step_function_errors(folder_and_plain):
    folder, _ = folder_and_plain
    _, model = load_model_on_device(folder, "float32", "cpu", ops=EmulatedOps())
    runner = ModelRunner(model, num_pages=2, page_size=16)
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("a", list(range(40)), [0])])
    with pytest.raises(ValueError, match="twice"):
        runner.step([StepEntry("b", [1], [0]), StepEntry("b", [2], [0])])
    with pytest.raises(ValueError, match="outside"):
        runner.step([StepEntry("c", [1, 2], [2])])
    runner.close("a"), runner.close("b"), runner.close("c")
    out = runner.step([StepEntry("d", [1, 2, 3], [])])           # nothing wanted: no logits
    assert out.shape == (0, 1000)
    out = runner.step([StepEntry("d", [4], [0])])
    assert out.shape == (1, 1000)
    runner.manager.check()


def test_cli_smoke(folder_and_plain, capsys, monkeypatch):
    folder, want = folder_and_plain
    import servelab_amd.cli as cli
    import servelab_amd.engine.llm_engine as le
    real = le.load_model_on_device
    monkeypatch.setattr(le, "load_model_on_device",
                        lambda f, dtype, device, ops=None, config=None:
                        real(f, "float32", "cpu", ops=EmulatedOps(), config=config))
    assert cli.main(["--model", folder, "--max-tokens", "12", "--temperature", "0",
                     "--num-blocks", "32"]) == 0
    printed = capsys.readouterr().out
    assert f"[req-1] finish=length -> {want[0]}" in printed and "stats:" in printed


def test_float16_checkpoints_are_served_in_bfloat16_and_say_so(tmp_path, capsys):
    from servelab_amd.engine.session import resolve_dtype
    cfg = load_config(make_folder(tmp_path, "A", seed=1, torch_dtype="float16"))
    assert resolve_dtype("auto", cfg) == torch.bfloat16
    assert "served in bfloat16" in capsys.readouterr().err
    with pytest.raises(ValueError, match="no kernels"):
        resolve_dtype("float16", cfg)
    assert resolve_dtype("float32", cfg) == torch.float32 and capsys.readouterr().err == ""


def test_decoding_a_step_ahead_changes_nothing_but_the_number_of_model_steps(folder_and_plain):
    """With and without the step ahead: the same tokens; a stop token costs one wasted row, never
    a wrong token; requests that arrive while a step is ahead join after it; an abort while a
    step is ahead leaves nothing held."""
    folder, want = folder_and_plain
    stop = want[0][5]
    cut = [w[:w.index(stop) + 1] if stop in w else w for w in want]
    params = SamplingParams(temperature=0.0, max_tokens=12, stop_token_ids=(stop,))
    runs = {}
    for ahead in (False, True):
        eng = make_engine(folder, run_ahead=ahead)
        outs = eng.generate(PROMPTS, params)
        assert [o.outputs[0].token_ids for o in outs] == cut
        assert eng.runner.manager.num_free_pages() == 64 and eng._flight is None
        runs[ahead] = eng.runner.steps
    assert runs[True] >= runs[False]                      # steps whose every row was void are the difference
    # arrivals during decoding
    eng = make_engine(folder, max_batched=32)
    first = eng.add_request(prompt_token_ids=PROMPTS[0], sampling_params=SamplingParams.greedy(12))
    done = {}
    for i in range(40):
        if i == 3:
            assert eng._flight is not None                # a step is ahead at this point
            second = eng.add_request(prompt_token_ids=PROMPTS[2], sampling_params=SamplingParams.greedy(12))
        if not eng.has_unfinished():
            break
        for out in eng.step():
            done[out.request_id] = out.outputs[0].token_ids
    assert done[first] == want[0] and done[second] == want[2]
    # abort while a step is ahead
    eng = make_engine(folder)
    rid = eng.add_request(prompt_token_ids=PROMPTS[0], sampling_params=SamplingParams.greedy(12))
    eng.step(), eng.step()
    assert eng._flight is not None and eng.abort_request(rid)
    assert not eng.has_unfinished() and eng.runner.manager.num_free_pages() == 64
    other = eng.generate([PROMPTS[1]], SamplingParams.greedy(12))[0]
    assert other.outputs[0].token_ids == want[1]
    eng.runner.manager.check()


def test_decoding_runs_ahead_under_a_standing_queue(folder_and_plain):
    """More requests than slots: while every slot decodes and nobody ends by length, the queue
    cannot move, so the engine keeps a step ahead; the tokens are plain's, and the number of
    model steps is the one without the step ahead (no stop tokens: no row is wasted)."""
    folder, want = folder_and_plain
    steps, ahead_seen = {}, 0
    for ahead in (False, True):
        eng = make_engine(folder, max_seqs=2, run_ahead=ahead)
        for p in PROMPTS:
            eng.add_request(prompt_token_ids=p, sampling_params=SamplingParams.greedy(12))
        done = {}
        while eng.has_unfinished():
            for out in eng.step():
                done[out.request_id] = out.outputs[0].token_ids
            if eng._flight is not None and eng.scheduler.queue:
                ahead_seen += 1
        assert [done[f"req-{i + 1}"] for i in range(4)] == want
        assert eng.runner.manager.num_free_pages() == 64 and eng._flight is None
        eng.runner.manager.check()
        steps[ahead] = eng.runner.steps
    assert steps[True] == steps[False]
    assert ahead_seen >= 8                       # the first pair's decode steps, with two requests waiting


def test_seeded_draws_do_not_depend_on_the_step_ahead_or_the_batch(folder_and_plain):
    """Temperature, top-k and top-p rows with different lengths and a stop token: the step ahead
    draws with the counter of the token before it, gathers the rows of requests that stay, and
    gives the tokens of the engine that waits for every step; so does every request alone."""
    folder, _ = folder_and_plain
    params = [SamplingParams(temperature=0.9, max_tokens=14, seed=11),
              SamplingParams(temperature=1.3, top_k=5, max_tokens=5, seed=12),
              SamplingParams(temperature=0.8, top_p=0.7, max_tokens=9, seed=13),
              SamplingParams(temperature=0.0, max_tokens=11)]

    def run(ahead, which, stop=()):
        eng = make_engine(folder, run_ahead=ahead, max_seqs=3)
        ids = []
        for i in which:
            sp = params[i]
            sp = SamplingParams(temperature=sp.temperature, top_k=sp.top_k, top_p=sp.top_p,
                                max_tokens=sp.max_tokens, seed=sp.seed, stop_token_ids=tuple(stop))
            ids.append(eng.add_request(prompt_token_ids=PROMPTS[i], sampling_params=sp))
        done = {o.request_id: o.outputs[0] for o in eng.run()}
        assert eng.runner.manager.num_free_pages() == 64 and eng._flight is None
        eng.runner.manager.check()
        return [(done[i].token_ids, done[i].finish_reason) for i in ids]

    waited = run(False, range(4))
    assert run(True, range(4)) == waited
    assert len({tuple(t) for t, _ in waited}) == 4 and waited[0][0] != waited[3][0]
    for i in range(4):
        assert run(True, [i]) == [waited[i]]
    stop = waited[0][0][6]                       # ends request 0 part-way, in a step that has a step ahead
    cut = run(False, range(4), stop=(stop,))
    assert cut[0][1] == "eos" and len(cut[0][0]) <= 7
    assert run(True, range(4), stop=(stop,)) == cut


def test_an_aborted_request_is_reported_and_leaves_no_step_behind(folder_and_plain):
    folder, want = folder_and_plain
    eng = make_engine(folder)
    rid = eng.add_request(prompt_token_ids=PROMPTS[0], sampling_params=SamplingParams.greedy(12))
    eng.step(), eng.step()
    assert eng._flight is not None and eng.abort_request(rid)
    assert eng._flight is None                   # the step ahead has nobody left to take its tokens
    assert not eng.abort_request(rid)
    steps = eng.runner.steps
    other = eng.add_request(prompt_token_ids=PROMPTS[1], sampling_params=SamplingParams.greedy(12))
    outs = eng.step()                            # the newcomer's prompt runs in this very step
    assert eng.runner.steps == steps + 2         # (and its first decode step is queued behind it)
    assert [(o.request_id, o.outputs[0].finish_reason) for o in outs] == [(rid, "aborted")]
    assert outs[0].outputs[0].token_ids == want[0][:len(outs[0].outputs[0].token_ids)]
    done = {o.request_id: o.outputs[0].token_ids for o in eng.run()}
    assert done == {other: want[1]}
    # aborts while others go on, through run(): everything is reported once
    eng = make_engine(folder)
    ids = [eng.add_request(prompt_token_ids=p, sampling_params=SamplingParams.greedy(12)) for p in PROMPTS]
    for _ in range(4):
        eng.step()
    assert eng.abort_request(ids[2])
    got = {o.request_id: o.outputs[0] for o in eng.run()}
    assert got[ids[2]].finish_reason == "aborted"
    assert [got[i].token_ids for i in (ids[0], ids[1], ids[3])] == [want[0], want[1], want[3]]
    assert eng.runner.manager.num_free_pages() == 64

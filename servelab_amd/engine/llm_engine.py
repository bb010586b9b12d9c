"""The engine: scheduler, cache manager, step function and sampler together.

Reference: ``LLMEngine`` (servelab/engine/engine.py:42-297) with the same
entry points — add_request, abort_request, has_unfinished, step, generate,
stats — and the same constructor arguments where they apply to one GPU.
"""
import time
from typing import Callable, Dict, List, Optional

import torch

from ..config import CacheConfig, SchedulerConfig
from ..sampling import Sampler
from .batch import StepEntry
from .output import RequestOutput, result_of
from .sampling_params import SamplingParams
from .scheduler import Scheduler
from .request import Request
from .session import load_model_on_device, make_runner, random_model_on_device


class LLMEngine:
    def __init__(self, model_config, cache_config: Optional[CacheConfig] = None,
                 scheduler_config: Optional[SchedulerConfig] = None, seed: int = 1234,
                 device: str = "cuda:0", tokenizer=None,
                 clock: Optional[Callable[[], float]] = None, dtype: str = "auto",
                 model=None, ops=None, tune_products=False, random_weights: Optional[int] = None,
                 capture_graphs_up_to: int = 0):
        """``model_config.path`` names the model folder (as in the reference,
        servelab/engine/engine.py:86-87); ``model`` may pass an already loaded
        DecoderModel instead, and ``random_weights`` a seed: the model of
        ``model_config`` then gets seeded random weights made on the device and
        no folder is read.  ``tune_products``: True, or a list of further
        step sizes (rows) to time the library's matrix kernels for.
        ``capture_graphs_up_to``: a context length up to which the decode graphs
        of 1..max_num_seqs requests are captured now rather than when a request
        first needs them."""
        self.model_config = model_config
        self.cache_config = cache_config or CacheConfig()
        self.scheduler_config = scheduler_config or SchedulerConfig()
        self.tokenizer = tokenizer
        self.clock = clock or time.monotonic
        if device == "auto":
            device = "cuda:0"
        if model is None and random_weights is not None:
            model = random_model_on_device(model_config, random_weights, dtype, device, ops=ops)
        if model is None:
            if not getattr(model_config, "path", ""):
                raise ValueError("model_config.path must name a model folder (or pass "
                                 "random_weights=SEED; write_random_model writes such a folder)")
            _, model = load_model_on_device(model_config.path, dtype, device, ops=ops,
                                            config=model_config)
        self.model = model
        self.device = model.rt.device
        self.dtype = model.rt.act_dtype
        self.runner = make_runner(model, self.cache_config.num_blocks,
                                  self.cache_config.block_size,
                                  self.scheduler_config.max_num_seqs,
                                  self.cache_config.gpu_memory_utilization)
        self.num_blocks = self.runner.manager.num_pages
        if tune_products:
            # a step that uses its whole token budget is the common large step under load;
            # decode steps of more requests than the few-rows kernels take are library products too
            rows = [self.scheduler_config.max_num_batched_tokens]
            if not isinstance(tune_products, bool):
                # further row counts the caller expects often (typical prompt lengths): the
                # library's choices hold for exactly the shapes that were timed
                rows += [int(n) for n in tune_products]
            library_rows = getattr(model.rt.ops, "library_rows", None)
            if library_rows is not None:
                first = model.rt.ops.SKINNY_MAX_M + 1
                rows += sorted({library_rows(n)
                                for n in range(first, self.scheduler_config.max_num_seqs + 1)})
            self.runner.tune_products(rows)
        self.graphs_captured = 0
        if capture_graphs_up_to:
            self.graphs_captured = self.runner.capture_graphs(
                range(1, self.scheduler_config.max_num_seqs + 1), capture_graphs_up_to)
        self.scheduler = Scheduler(self.scheduler_config, self.runner.manager, self.clock,
                                   eos_token_id=model.spec.eos_token_id,
                                   max_positions=model.spec.max_position_embeddings)
        self.sampler = Sampler(model.rt.ops, self.device, seed)
        self._submitted = 0
        self.num_steps = 0

    # -------------------------------------------------------------- intake
    def add_request(self, prompt: Optional[str] = None,
                    sampling_params: Optional[SamplingParams] = None,
                    prompt_token_ids: Optional[List[int]] = None,
                    request_id: Optional[str] = None, priority: int = 0) -> str:
        """servelab/engine/engine.py:138-160."""
        if prompt_token_ids is None:
            if self.tokenizer is None or prompt is None:
                raise ValueError("need prompt_token_ids, or a tokenizer + prompt")
            prompt_token_ids = self.tokenizer.encode(prompt)
        vocab = self.model.spec.vocab_size
        bad = [t for t in prompt_token_ids if not 0 <= int(t) < vocab]
        if bad:
            raise ValueError(f"token id {bad[0]} is outside the vocabulary of {vocab}")
        self._submitted += 1
        request_id = request_id or f"req-{self._submitted}"
        self.scheduler.add_request(Request(
            request_id, prompt_token_ids, sampling_params or SamplingParams(), priority=priority,
            arrived=self.clock(), number=self._submitted))
        return request_id

    def abort_request(self, request_id: str) -> bool:
        return self.scheduler.abort_request(request_id)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished()

    # ---------------------------------------------------------------- step
    def step(self) -> List[RequestOutput]:
        """One scheduler pass, one model step, one sampling call.  Returns the
        requests that finished (or were aborted) in this step
        (servelab/engine/engine.py:169-241)."""
        plan = self.scheduler.schedule()
        outputs = [result_of(r, self._to_text) for r in plan.aborted]
        if plan.is_empty():
            if not outputs and self.scheduler.has_unfinished():
                raise RuntimeError("nothing can be scheduled although requests are unfinished")
            return outputs
        items = plan.items()                     # portions first, then single tokens
        entries = [StepEntry(it.request.request_id, it.token_ids,
                             [it.count - 1] if it.samples else []) for it in items]
        drawing = [it.request for it in items if it.samples]
        logits = self.runner.step(entries)
        tokens = self.sampler.sample(logits, [r.params for r in drawing],
                                     [r.number for r in drawing], [r.num_output for r in drawing])
        finished = self.scheduler.complete(
            plan, {r.request_id: t for r, t in zip(drawing, tokens)}, now=self.clock())
        self.num_steps += 1
        return outputs + [result_of(r, self._to_text) for r in finished]

    @property
    def _to_text(self):
        return self.tokenizer.decode if self.tokenizer is not None else None

    # ------------------------------------------------------------ generate
    def run(self, on_step: Optional[Callable[[dict], None]] = None):
        """Steps until nothing is unfinished, yielding each result as its
        request ends; ``on_step`` is called with ``stats()`` after every step."""
        while self.has_unfinished():
            yield from self.step()
            if on_step is not None:
                on_step(self.stats())

    def generate(self, prompts: List, sampling_params: Optional[SamplingParams] = None,
                 verbose: bool = False) -> List[RequestOutput]:
        """Offline generation of a batch of prompts — strings (needs a tokenizer)
        or lists of token ids — all with the same parameters; results in the
        order of the prompts (the call of servelab/engine/engine.py:249-270).
        ``verbose`` prints a line of queue and cache figures per step."""
        params = sampling_params or SamplingParams()
        order = [self.add_request(p, params) if isinstance(p, str)
                 else self.add_request(None, params, prompt_token_ids=list(p)) for p in prompts]

        def line(st):
            print(f"[step {st['steps']}] running={st['running']} waiting={st['waiting']} "
                  f"cache={st['gpu_cache_usage']:.0%}", flush=True)
        done = {out.request_id: out for out in self.run(line if verbose else None)}
        return [done.get(rid) for rid in order]

    def stats(self) -> dict:
        return {**self.scheduler.stats(), **self.runner.manager.stats(),
                "num_blocks": self.num_blocks, "block_size": self.cache_config.block_size,
                "dtype": str(self.dtype).replace("torch.", ""),
                "checkpoint_dtype": getattr(self.model_config, "dtype", None),
                "device": str(self.device),
                "steps": self.num_steps}

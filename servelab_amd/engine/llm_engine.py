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


class _TokenBuffers:
    """Two pinned host buffers used in turn: for sampled tokens, the step ahead
    copies into one while the host still reads the other; for the rows a step
    ahead gathers, the host fills one while the copy out of the other may still
    be queued."""

    def __init__(self, rows: int, device, dtype=torch.int32):
        self.cuda = torch.device(device).type == "cuda"
        self.dtype = dtype
        self.buffers = [torch.empty(max(1, rows), dtype=dtype) for _ in range(2)]
        if self.cuda:
            self.buffers = [b.pin_memory() for b in self.buffers]
        self.turn = 0

    def take(self, n: int) -> torch.Tensor:
        self.turn ^= 1
        if self.buffers[self.turn].numel() < n:
            grown = torch.empty(2 * n, dtype=self.dtype)
            self.buffers[self.turn] = grown.pin_memory() if self.cuda else grown
        return self.buffers[self.turn][:n]


class _Flight:
    """A step that is queued on the device: its plan, the requests it samples
    for (in row order), the sampled tokens on the device and their copy on the
    way to the host."""

    def __init__(self, plan, drawing, device_tokens, buffers: _TokenBuffers):
        self.plan, self.drawing, self.device_tokens = plan, drawing, device_tokens
        self.host = self.arrived = None
        if device_tokens is not None:
            self.host = buffers.take(len(drawing))
            self.host.copy_(device_tokens, non_blocking=True)
            if device_tokens.is_cuda:
                self.arrived = torch.cuda.Event()
                self.arrived.record()

    def tokens(self) -> List[int]:
        if self.host is None:
            return []
        if self.arrived is not None:
            self.arrived.synchronize()
        return self.host.tolist()


class LLMEngine:
    def __init__(self, model_config, cache_config: Optional[CacheConfig] = None,
                 scheduler_config: Optional[SchedulerConfig] = None, seed: int = 1234,
                 device: str = "cuda:0", tokenizer=None, predictor=None,
                 clock: Optional[Callable[[], float]] = None, dtype: str = "auto",
                 model=None, ops=None, tune_products=False, random_weights: Optional[int] = None,
                 capture_graphs_up_to: int = 0, run_ahead: bool = True):
        """``model_config.path`` names the model folder (as in the reference,
        servelab/engine/engine.py:86-87); ``model`` may pass an already loaded
        DecoderModel instead, and ``random_weights`` a seed: the model of
        ``model_config`` then gets seeded random weights made on the device and
        no folder is read.  ``tune_products``: True, or a list of further
        step sizes (rows) to time the library's matrix kernels for.
        ``capture_graphs_up_to``: a context length up to which the decode graphs
        of 1..max_num_seqs requests are captured now rather than when a request
        first needs them.  ``predictor``: an object with
        ``predict_remaining(request) -> int``, the number of tokens a request
        will generate, for the policy "sjf-predicted"
        (servelab/engine/engine.py:51,131)."""
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
                # decode steps of more requests than the few-rows kernels take, and the steps that
                # carry a newcomer's short prompt beside decoded tokens: below LIBRARY_PADDED_MAX_M
                # rows they run on a multiple of LIBRARY_ROW_STEP rows, so these few shapes cover them
                first = int(getattr(model.rt.ops, "graph_rows_limit", model.rt.ops.SKINNY_MAX_M)) + 1
                top = max(self.scheduler_config.max_num_seqs,
                          min(model.rt.ops.LIBRARY_PADDED_MAX_M, self.scheduler_config.max_num_batched_tokens))
                rows += sorted({library_rows(n) for n in range(first, top + 1)})
            self.runner.tune_products(rows)
        self.graphs_captured = 0
        if capture_graphs_up_to:
            self.graphs_captured = self.runner.capture_graphs(
                range(1, self.scheduler_config.max_num_seqs + 1), capture_graphs_up_to)
        self.scheduler = Scheduler(self.scheduler_config, self.runner.manager, self.clock,
                                   eos_token_id=model.spec.eos_token_id,
                                   max_positions=model.spec.max_position_embeddings, predictor=predictor)
        self.sampler = Sampler(model.rt.ops, self.device, seed)
        self.run_ahead = bool(run_ahead)
        self._flight: Optional[_Flight] = None
        self._token_buffers = _TokenBuffers(self.scheduler_config.max_num_seqs, self.device)
        self._row_buffers = _TokenBuffers(self.scheduler_config.max_num_seqs, self.device, torch.int64)
        self._aborted: List[RequestOutput] = []      # results of abort_request, returned by the next step
        self._submitted = 0
        self.num_steps = 0

    @classmethod
    def from_engine_config(cls, model_config, engine_config, **more) -> "LLMEngine":
        """The engine that an ``EngineConfig`` describes (cache, scheduler, seed,
        dtype, device and the start-up options in one record); ``more`` passes
        on what the record does not hold (``model``, ``ops``, ``tokenizer``,
        ``random_weights``, ...)."""
        ec = engine_config
        return cls(model_config, ec.cache, ec.scheduler, seed=ec.seed, device=ec.device,
                   dtype=ec.dtype, tune_products=ec.tune_products,
                   capture_graphs_up_to=ec.capture_graphs_up_to, run_ahead=ec.run_ahead, **more)

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

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished()

    # ---------------------------------------------------------------- step
    def step(self) -> List[RequestOutput]:
        """One scheduler pass, one model step, one sampling call.  Returns the
        requests that finished (or were aborted) in this step
        (servelab/engine/engine.py:169-241).

        Decoding runs one step ahead of the host: while a step's tokens are
        still on their way, the next decode step of the same requests is
        already queued behind it on the device, taking its token ids from the
        sampler's output there (``run_ahead``; the reference waits for every
        step's tokens before it plans the next).  What the host does between
        two steps then costs no device time.  A request that a stop token ends
        has one wasted row in the step ahead; a newcomer waits for that step."""
        flight, self._flight = self._flight, None
        outputs, self._aborted = self._aborted, []
        if flight is None:
            plan = self.scheduler.schedule()
            outputs += [result_of(r, self._to_text) for r in plan.aborted]
            if plan.is_empty():
                if not outputs and self.scheduler.has_unfinished():
                    raise RuntimeError("nothing can be scheduled although requests are unfinished")
                return outputs
            flight = self._launch(plan, None)
        if self.run_ahead:
            ahead = self.scheduler.plan_ahead(flight.plan)
            if ahead is not None:
                self._flight = self._launch(ahead, flight)
        tokens = flight.tokens()                 # waits for this step's tokens, not for the step ahead
        finished = self.scheduler.complete(
            flight.plan, {r.request_id: t for r, t in zip(flight.drawing, tokens)}, now=self.clock())
        self.num_steps += 1
        if self._flight is not None and all(it.request.done for it in self._flight.plan.items()):
            self._flight = None                  # every request of the step ahead has ended: its result is void
        return outputs + [result_of(r, self._to_text) for r in finished]

    def _launch(self, plan, after: Optional["_Flight"]) -> "_Flight":
        """Queue ``plan`` on the device: the model step, the sampling call and
        the copy of the sampled tokens to the host.  ``after``: the step whose
        tokens this one continues from, not yet known to the host."""
        items = plan.items()                     # portions first, then single tokens
        drawing = [it.request for it in items if it.samples or after is not None]
        if after is None:
            entries = [StepEntry(it.request.request_id, it.token_ids,
                                 [it.count - 1] if it.samples else []) for it in items]
            logits = self.runner.step(entries)
        else:
            entries = [StepEntry(it.request.request_id, [0], [0]) for it in items]
            row_of = {r.request_id: i for i, r in enumerate(after.drawing)}
            rows = [row_of[it.request.request_id] for it in items]
            ids = after.device_tokens
            if rows != list(range(len(after.drawing))):
                # requests have left since that step: gather the rows that stay (the index goes
                # through pinned memory, so nothing here waits for the device)
                index = self._row_buffers.take(len(rows))
                index.copy_(torch.tensor(rows, dtype=torch.int64))
                ids = ids.index_select(0, index.to(ids.device, non_blocking=True))
            logits = self.runner.step(entries, device_ids=ids)
        drawn_before = 1 if after is not None else 0     # the token of the step this one follows
        device_tokens = self.sampler.sample_on_device(
            logits, [r.params for r in drawing], [r.number for r in drawing],
            [r.num_output + drawn_before for r in drawing]) if drawing else None
        return _Flight(plan, drawing, device_tokens, self._token_buffers)

    def abort_request(self, request_id: str) -> bool:
        """servelab/engine/engine.py:162-163.  The request's pages are free at
        once (a step or a step ahead that is still queued on the device may
        write its rows of them; whoever gets the pages next writes after that,
        in stream order); its result, with finish reason "aborted", comes with
        the next ``step``."""
        req = self.scheduler.abort_request(request_id)
        if req is None:
            return False
        self._aborted.append(result_of(req, self._to_text))
        if self._flight is not None and all(it.request.done for it in self._flight.plan.items()):
            self._flight = None                  # nobody is left to take the step ahead's tokens
        return True

    @property
    def _to_text(self):
        return self.tokenizer.decode if self.tokenizer is not None else None

    # ------------------------------------------------------------ generate
    def run(self, on_step: Optional[Callable[[dict], None]] = None):
        """Steps until nothing is unfinished, yielding each result as its
        request ends; ``on_step`` is called with ``stats()`` after every step."""
        while self.has_unfinished() or self._aborted:
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
                "dtype_substituted": (getattr(self.model_config, "dtype", None) == "float16"
                                      and self.dtype == torch.bfloat16),
                "device": str(self.device),
                "steps": self.num_steps}

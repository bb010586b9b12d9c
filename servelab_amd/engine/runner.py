"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.

Reference: the middle of ``LLMEngine.step`` (servelab/engine/engine.py:176-218)
— build the packed batch, ``forward_packed``, ``lm_head_forward`` on the
selected rows, float32 logits.  Here that is a function of its own below the
scheduler, so that trace replay, the benchmark and the engine drive the same
code.  It runs only the tokens it is given, from the cache earlier steps left.
"""
from typing import Dict, Hashable, List, Optional

import torch

from ..cache import CacheManager, CachePool
from ..parts.base import Runtime
from ..parts.model import DecoderModel
from .batch import StepBatch, StepEntry, pack_batch


class OutOfPages(RuntimeError):
    """The cache pool cannot hold the tokens of this step."""


class ModelRunner:
    def __init__(self, model: DecoderModel, num_pages: int, page_size: int,
                 max_num_seqs: int = 64):
        self.model = model
        self.rt: Runtime = model.rt
        self.manager = CacheManager(model.spec.stream_specs(), num_pages, page_size,
                                    num_state_slots=max_num_seqs)
        self.pool = CachePool(self.manager, self.rt.device, self.rt.act_dtype)
        self.bindings = [self.pool.binding(c.stream, c.write) for c in model.spec.run]
        self.max_positions = model.spec.max_position_embeddings
        self.steps = 0
        self.tokens_run = 0

    # ------------------------------------------------------------ requests
    def open(self, request: Hashable) -> bool:
        return self.manager.open(request)

    def close(self, request: Hashable) -> None:
        self.manager.close(request)

    # ---------------------------------------------------------------- step
    def prepare(self, entries: List[StepEntry]):
        """Reserve pages and build the device batch.  Returns (batch, order):
        the entries are packed with multi-token ones first, ``order`` maps the
        packed position back; wanted rows stay in the callers' order."""
        m = self.manager
        seen = set()
        for e in entries:
            if e.request in seen:
                raise ValueError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if len(e.tokens) < 1:
                raise ValueError(f"request {e.request!r} brings no tokens")
            if not m.is_open(e.request) and not m.open(e.request):
                raise OutOfPages(f"no state slot free for request {e.request!r}")
        for e in entries:
            total = m.length(e.request) + len(e.tokens)
            if total > self.max_positions:
                raise ValueError(f"request {e.request!r}: {total} tokens exceed "
                                 f"max_position_embeddings {self.max_positions}")
            if not m.grow(e.request, total):
                raise OutOfPages(
                    f"request {e.request!r} needs {m.pages_needed(e.request, total)} more pages, "
                    f"{m.num_free_pages()} free")
        order = sorted(range(len(entries)), key=lambda i: 0 if len(entries[i].tokens) > 1 else 1)
        packed = [entries[i] for i in order]
        starts = [m.length(e.request) for e in packed]
        offset_of, offset = {}, 0
        for i in order:
            offset_of[i] = offset
            offset += len(entries[i].tokens)
        rows = []
        for i, e in enumerate(entries):          # wanted rows stay in the callers' order
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"request {e.request!r}: wanted place {w} is outside its "
                                     f"{len(e.tokens)} tokens")
                rows.append(offset_of[i] + int(w))
        batch = pack_batch(packed, starts, rows, m, self.rt.device)
        return batch, packed

    @torch.no_grad()
    def step(self, entries: List[StepEntry]) -> torch.Tensor:
        """Run one batch; returns float32 logits [wanted, vocab] in the order of
        the entries and of their ``want``."""
        if not entries:
            return torch.empty((0, self.model.spec.vocab_size), dtype=torch.float32,
                               device=self.rt.device)
        batch, packed = self.prepare(entries)
        logits = self.model.forward(batch, self.bindings)
        for e, start, n in zip(packed, batch.starts, batch.q_lens):
            self.manager.commit(e.request, start + n)
        self.steps += 1
        self.tokens_run += batch.num_tokens
        return logits

"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.

Reference: the middle of ``LLMEngine.step`` (servelab/engine/engine.py:176-218)
— build the packed batch, ``forward_packed``, ``lm_head_forward`` on the
selected rows, float32 logits.  Here that is a function of its own below the
scheduler, so that trace replay, the benchmark and the engine drive the same
code.  It runs only the tokens it is given, from the cache earlier steps left.
"""
from collections import OrderedDict
from typing import Dict, Hashable, List, Optional

import torch

from ..cache import CacheManager, CachePool
from ..parts.base import Runtime
from ..parts.model import DecoderModel
from .batch import Staging, StepBatch, StepEntry, batch_on_device, build_arrays, pack_batch


class OutOfPages(RuntimeError):
    """The cache pool cannot hold the tokens of this step."""


class ModelRunner:
    GRAPH_MAX_SEQS = 64
    GRAPH_MIN_CONTEXT = 512
    # Captured decode graphs keep their outputs (float32 logits [requests, vocabulary]) and metadata
    # buffers for as long as they live; their intermediates share one memory pool.  What they keep
    # is bounded: at most this share of the device memory that is free once the cache pool stands,
    # and at most GRAPH_MEMORY_MAX bytes; the graph used longest ago goes first.
    GRAPH_MEMORY_SHARE = 0.25
    GRAPH_MEMORY_MAX = 4 << 30

    def __init__(self, model: DecoderModel, num_pages: int, page_size: int,
                 max_num_seqs: int = 64, use_graphs: bool = True):
        self.model = model
        self.rt: Runtime = model.rt
        self.manager = CacheManager(model.spec.stream_specs(), num_pages, page_size,
                                    num_state_slots=max_num_seqs)
        self.pool = CachePool(self.manager, self.rt.device, self.rt.act_dtype)
        self.bindings = [[self.pool.binding(s, c.write) for s in c.streams] for c in model.spec.run]
        self.max_positions = model.spec.max_position_embeddings
        self.steps = 0
        self.tokens_run = 0
        # decode steps of up to graph_max_seqs single tokens replay a captured HIP graph; a kernel
        # table says itself up to how many rows its products stay clear of library calls
        self.use_graphs = (use_graphs and self.rt.device.type == "cuda" and model.spec.graph_safe)
        self.graph_max_seqs = int(getattr(self.rt.ops, "graph_rows_limit", self.GRAPH_MAX_SEQS))
        self._graphs: "OrderedDict[tuple, tuple]" = OrderedDict()     # least recently used first
        self._graph_pool = None           # one memory pool for the intermediates of all captures
        self._graph_bytes = 0
        self.graph_memory_limit = self.GRAPH_MEMORY_MAX
        if self.use_graphs:
            free, _ = torch.cuda.mem_get_info(self.rt.device)
            self.graph_memory_limit = min(self.GRAPH_MEMORY_MAX, int(free * self.GRAPH_MEMORY_SHARE))
        self.graph_replays = 0
        self.graph_evictions = 0
        self._staging = Staging()
        self._decoding = None         # the last graph step, for the next one to continue from

    # ------------------------------------------------------------ requests
    def open(self, request: Hashable) -> bool:
        return self.manager.open(request)

    def close(self, request: Hashable) -> None:
        self.manager.close(request)

    # ---------------------------------------------------------------- step
    def reserve(self, entries: List[StepEntry]):
        """Open what is new, reserve pages for every entry, and order the step:
        multi-token entries first.  Returns (packed entries, their cached
        lengths, wanted rows in the callers' order of entries)."""
        m = self.manager
        vocab = self.model.spec.vocab_size
        seen = set()
        for e in entries:
            if e.request in seen:
                raise ValueError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if len(e.tokens) < 1:
                raise ValueError(f"request {e.request!r} brings no tokens")
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                raise ValueError(f"request {e.request!r}: token id outside the vocabulary of {vocab}")
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
        return packed, starts, rows

    def prepare(self, entries: List[StepEntry]):
        """Reserve pages and build the device batch: (batch, packed entries)."""
        packed, starts, rows = self.reserve(entries)
        return pack_batch(packed, starts, rows, self.manager, self.rt.device,
                          staging=self._staging), packed

    # -------------------------------------------------------------- graphs
    def _graph_key(self, packed, starts, rows):
        """(sequences, context capacity) when the step is a pure decode step
        that a captured graph can run, else None."""
        B = len(packed)
        if not self.use_graphs or B > self.graph_max_seqs or len(rows) != B:
            return None
        if any(len(e.tokens) != 1 for e in packed) or rows != list(range(B)):
            return None
        cap = self.GRAPH_MIN_CONTEXT
        need = max(starts) + 1
        while cap < need:
            cap *= 2
        return (B, cap)

    def _step_graph(self, key, packed, starts, rows, device_ids=None, evict=True):
        """Decode step through a HIP graph.  The first step of a shape runs
        eagerly on a side stream (its result is returned) and is then captured;
        later steps overwrite the graph's metadata buffer and replay it.
        Everything a launch depends on besides device memory is fixed by the
        key: the number of sequences and the context capacity, which sets the
        width of the block tables and how the decode attention splits.
        ``evict=False``: a new graph that would not fit beside the others is
        not made (None is returned and nothing ran)."""
        B, cap = key
        pages = cap // self.manager.page_size
        arr = build_arrays(packed, starts, rows, self.manager, fixed_pages=pages)
        host = torch.from_numpy(arr.flat)
        entry = self._graphs.get(key)
        if entry is not None:
            self._graphs.move_to_end(key)
            graph, dev, staging, logits, copied = entry
            copied.synchronize()              # the last copy out of the staging buffer is done
            staging.copy_(host)
            dev.copy_(staging, non_blocking=True)
            copied.record()
            if device_ids is not None:
                dev[arr.offsets[0]:arr.offsets[0] + B].copy_(device_ids)
            graph.replay()
            self.graph_replays += 1
            self._decoding = (key, arr)
            return logits
        need = self._entry_bytes(host, B)
        if not evict and self._graphs and self._graph_bytes + need > self.graph_memory_limit:
            return None
        staging = torch.empty_like(host).pin_memory()
        staging.copy_(host)
        dev = staging.to(self.rt.device, non_blocking=True)
        if device_ids is not None:
            dev[arr.offsets[0]:arr.offsets[0] + B].copy_(device_ids)
        batch = batch_on_device(arr, dev, max_ctx_len=cap)
        side = torch.cuda.Stream(device=self.rt.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            eager = self.model.forward(batch, self.bindings)
        torch.cuda.current_stream().wait_stream(side)
        self._make_room(need)
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits = self.model.forward(batch, self.bindings)
        copied = torch.cuda.Event()
        copied.record()
        self._graphs[key] = (graph, dev, staging, logits, copied)
        self._graph_bytes += need
        self._decoding = (key, arr)
        return eager

    def capture_graphs(self, batch_sizes, max_context: int) -> int:
        """Capture, ahead of use, the decode graphs of ``batch_sizes`` requests
        for every context capacity up to ``max_context`` tokens, so that no
        request meets the two extra passes (an eager step, then the capture) of
        a shape seen for the first time.  Runs on throw-away requests of one
        token; stops when the graphs' memory limit is reached (nothing is
        dropped to make room).  Returns the number of graphs captured."""
        if not self.use_graphs:
            return 0
        caps, cap = [], self.GRAPH_MIN_CONTEXT
        limit = min(int(max_context), self.max_positions)
        while True:
            caps.append(cap)
            if cap >= limit:
                break
            cap *= 2
        made, full = 0, False
        for B in sorted({int(b) for b in batch_sizes if 1 <= int(b) <= self.graph_max_seqs}):
            tags = [("capture_graphs", i) for i in range(B)]
            opened = []
            try:
                for t in tags:
                    if not self.open(t):
                        break
                    opened.append(t)
                if len(opened) < B or not all(self.manager.grow(t, 1) for t in tags):
                    continue
                packed = [StepEntry(t, [0], [0]) for t in tags]
                for cap in caps:
                    if (B, cap) in self._graphs or cap // self.manager.page_size < 1:
                        continue
                    if self._step_graph((B, cap), packed, [0] * B, list(range(B)), evict=False) is None:
                        full = True
                        break
                    made += 1
            finally:
                for t in opened:
                    self.close(t)
                self._decoding = None
            if full:
                break
        if made:
            torch.cuda.synchronize(self.rt.device)
        return made

    def _entry_bytes(self, meta, B) -> int:
        """What a captured graph keeps alive beside the shared pool of
        intermediates: its logits and its metadata buffer (``meta``: that
        buffer, or the host array it is made from)."""
        return B * self.model.spec.vocab_size * 4 + meta.numel() * meta.element_size()

    def _make_room(self, need: int) -> None:
        """Drop the graphs used longest ago until ``need`` more bytes fit the
        limit (a single graph larger than the limit is still kept alone).
        The device is idle for this: a graph's memory must not return to the
        pool while a replay of it is still running."""
        if not self._graphs or self._graph_bytes + need <= self.graph_memory_limit:
            return
        torch.cuda.synchronize(self.rt.device)
        while self._graphs and self._graph_bytes + need > self.graph_memory_limit:
            old_key, (graph, dev, staging, logits, copied) = self._graphs.popitem(last=False)
            self._graph_bytes -= self._entry_bytes(dev, old_key[0])
            self.graph_evictions += 1
            if self._decoding is not None and self._decoding[0] == old_key:
                self._decoding = None
            del graph, dev, staging, logits, copied

    def _continue_decoding(self, entries: List[StepEntry], device_ids=None) -> Optional[torch.Tensor]:
        """The common decode step — the same requests as the last graph step,
        one more token each — without rebuilding the step's arrays: ids are
        replaced, positions and contexts advance by one, slots follow the block
        tables, and a table gains an entry when a request enters a new page.
        Returns None when the step is anything else."""
        if self._decoding is None:
            return None
        key, arr = self._decoding
        B, cap = key
        if len(entries) != B:
            return None
        m = self.manager
        lengths = m.lengths
        vocab = self.model.spec.vocab_size
        for e, request, start in zip(entries, arr.requests, arr.starts):
            if (e.request != request or len(e.tokens) != 1 or len(e.want) != 1 or e.want[0] != 0
                    or lengths.get(request) != start + 1):
                return None
        if max(arr.starts) + 2 > min(cap, self.max_positions):
            return None
        for e in entries:
            if not 0 <= e.tokens[0] < vocab:
                raise ValueError(f"request {e.request!r}: token id outside the vocabulary of {vocab}")
            if not m.grow(e.request, lengths[e.request] + 1):
                raise OutOfPages(
                    f"request {e.request!r} needs a page, {m.num_free_pages()} free")
        flat, off, bs = arr.flat, arr.offsets, m.page_size
        starts = [s + 1 for s in arr.starts]
        flat[off[0]:off[0] + B] = [e.tokens[0] for e in entries]
        flat[off[1]:off[1] + B] += 1                      # positions
        flat[off[4]:off[4] + B] += 1                      # contexts
        for gi, g in enumerate(m.page_groups):
            pages = arr.group_pages[gi]
            slots_at, tables_at = off[7 + 2 * gi], off[8 + 2 * gi]
            for i, (request, p) in enumerate(zip(arr.requests, starts)):
                page = g.tables[request][p // bs]
                flat[slots_at + i] = page * bs + p % bs
                if p % bs == 0:
                    flat[tables_at + i * pages + p // bs] = page
        arr.starts = starts
        self._graphs.move_to_end(key)
        graph, dev, staging, logits, copied = self._graphs[key]
        copied.synchronize()
        staging.copy_(torch.from_numpy(flat))
        dev.copy_(staging, non_blocking=True)
        copied.record()
        if device_ids is not None:
            dev[off[0]:off[0] + B].copy_(device_ids)
        graph.replay()
        self.graph_replays += 1
        for request, p in zip(arr.requests, starts):
            m.commit(request, p + 1)
        self.steps += 1
        self.tokens_run += B
        return logits

    @torch.no_grad()
    def tune_products(self, row_counts, max_ms: int = 30) -> List[int]:
        """Runs one throw-away prompt portion of each given length with the
        kernel table's library tuning on, so that the library products of a
        step with that many rows use the fastest kernel the library has for
        them.  Lengths the empty pool cannot hold are left out; returns the
        lengths tuned.  A no-op for kernel tables without library products."""
        tuning = getattr(self.model.rt.ops, "library_tuning", None)
        if tuning is None or self.model.rt.act_dtype != torch.bfloat16:
            return []
        done = []
        with tuning(max_ms):
            for n in sorted(set(int(r) for r in row_counts)):
                tag = ("tune_products", n)
                if (n < 1 or n > self.max_positions or not self.manager.can_ever_hold(n)
                        or not self.open(tag)):
                    continue
                try:
                    self.step([StepEntry(tag, [0] * n, [n - 1])])
                    done.append(n)
                except OutOfPages:
                    pass
                finally:
                    self.close(tag)
        if self.rt.device.type == "cuda":
            torch.cuda.synchronize(self.rt.device)
        return done

    def step(self, entries: List[StepEntry], device_ids: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run one batch; returns float32 logits [wanted, vocab] in the order of
        the entries and of their ``want``.  The tensor may be a captured graph's
        output buffer: it is valid until the next call of ``step``.

        ``device_ids`` (int32 on the device, one per entry, in the order of the
        entries) gives the token ids of a step whose entries bring one token
        each when the host does not know them yet (the last step's sampled
        tokens, still on the device); the entries' own ids are then ignored."""
        if not entries:
            return torch.empty((0, self.model.spec.vocab_size), dtype=torch.float32,
                               device=self.rt.device)
        if device_ids is not None:
            if any(len(e.tokens) != 1 for e in entries):
                raise ValueError("token ids from the device go with entries of one token each")
            if device_ids.dtype != torch.int32 or tuple(device_ids.shape) != (len(entries),):
                raise ValueError("device_ids must be int32, one per entry")
        logits = self._continue_decoding(entries, device_ids)
        if logits is not None:
            return logits
        self._decoding = None
        packed, starts, rows = self.reserve(entries)
        key = self._graph_key(packed, starts, rows)
        if key is not None:
            logits = self._step_graph(key, packed, starts, rows, device_ids)
        else:
            batch = pack_batch(packed, starts, rows, self.manager, self.rt.device,
                               staging=self._staging)
            if device_ids is not None:           # (one token each: packed order is the callers' order)
                batch.ids.copy_(device_ids)
            logits = self.model.forward(batch, self.bindings)
        for e, start in zip(packed, starts):
            self.manager.commit(e.request, start + len(e.tokens))
        self.steps += 1
        self.tokens_run += sum(len(e.tokens) for e in packed)
        return logits

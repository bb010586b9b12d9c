"""One step's batch: the tokens to run and the metadata the kernels read.

Reference: ``LLMEngine.step`` flattens the scheduled prefill chunks, then the
decode tokens, into parallel lists tokens/positions/slots/metas/logit_rows
(servelab/engine/engine.py:176-209) and copies three of them to the device
(:213-215); block tables stay Python lists and are re-uploaded per layer.
Here every array of a step is packed into one int32 buffer that is copied to
the device once: ids, positions, the sequence of each token, cumulative query
lengths, context lengths, state slots, wanted rows, and per page group the
slot of each token and the block tables.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, Hashable, List, Sequence

import numpy as np
import torch


@dataclass
class StepEntry:
    """A request's next tokens; ``want`` are the places among these tokens
    whose logits are asked for."""
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class GroupMeta:
    slots: torch.Tensor          # [T] flat cache row of each token in this group
    block_tables: torch.Tensor   # [S, max_pages]
    max_pages: int


@dataclass
class StepBatch:
    num_tokens: int
    num_seqs: int
    num_prefill_seqs: int        # sequences with more than one token come first
    num_prefill_tokens: int
    num_logit_rows: int
    max_q_len: int
    max_ctx_len: int
    # device int32
    ids: torch.Tensor
    positions: torch.Tensor
    tok_seq: torch.Tensor        # [T] sequence index of each token
    cu_q: torch.Tensor           # [S + 1]
    ctx_len: torch.Tensor        # [S] tokens cached after this step
    state_slots: torch.Tensor    # [S]
    logit_rows: torch.Tensor     # [R]
    groups: List[GroupMeta]
    # [2] the sum and the largest of the context lengths of the single-token sequences (what a kernel that
    # shares out their keys balances by; on the device because a captured step is fed new lengths)
    ctx_stats: torch.Tensor = None
    # host copies for parts that plan on the host
    q_lens: List[int] = field(default_factory=list)
    starts: List[int] = field(default_factory=list)
    requests: List[Hashable] = field(default_factory=list)
    host_state_slots: List[int] = field(default_factory=list)


@dataclass
class BatchArrays:
    """A step's metadata on the host: one flat int32 array and where each piece
    lies in it.  The layout depends only on (tokens, sequences, rows, pages per
    table), so a captured graph can be fed by overwriting its buffer."""
    flat: np.ndarray
    offsets: List[int]
    sizes: List[int]
    group_pages: List[int]
    q_lens: List[int]
    starts: List[int]
    requests: List[Hashable]
    state_slots: List[int]
    num_rows: int
    max_ctx_len: int


def build_arrays(entries: List[StepEntry], starts: List[int], rows: List[int], manager,
                 pad_pages_to: int = 8, fixed_pages: int = 0) -> BatchArrays:
    """The arrays of ``entries`` (already ordered: multi-token first) whose
    requests have ``starts[i]`` tokens cached and room for the new ones;
    ``rows`` are the packed rows whose logits are wanted.  ``fixed_pages`` sets
    the width of every block table instead of deriving it from the contexts."""
    bs = manager.page_size
    S = len(entries)
    q_lens = [len(e.tokens) for e in entries]
    T = sum(q_lens)
    cu = np.zeros(S + 1, dtype=np.int32)
    np.cumsum(q_lens, out=cu[1:])
    ids = np.empty(T, dtype=np.int32)
    pos = np.empty(T, dtype=np.int32)
    tok_seq = np.empty(T, dtype=np.int32)
    for i, e in enumerate(entries):
        a, b = cu[i], cu[i + 1]
        ids[a:b] = np.asarray(e.tokens, dtype=np.int64)
        pos[a:b] = np.arange(starts[i], starts[i] + q_lens[i], dtype=np.int32)
        tok_seq[a:b] = i
    ctx = np.asarray([starts[i] + q_lens[i] for i in range(S)], dtype=np.int32)
    slots_host = [manager.state_slot(e.request) for e in entries]

    parts = [ids, pos, tok_seq, cu, ctx, np.asarray(slots_host, dtype=np.int32),
             np.asarray(rows, dtype=np.int32)]
    group_pages = []
    for gi, g in enumerate(manager.page_groups):
        max_pages = max(manager.pages_for(int(c)) for c in ctx)
        if not fixed_pages:
            max_pages = -(-max_pages // pad_pages_to) * pad_pages_to
        else:
            if max_pages > fixed_pages:
                raise ValueError(f"a context of {int(ctx.max())} tokens does not fit block tables "
                                 f"of {fixed_pages} pages")
            max_pages = fixed_pages
        tables = np.zeros((S, max_pages), dtype=np.int32)
        slots = np.empty(T, dtype=np.int32)
        for i, e in enumerate(entries):
            table = np.asarray(g.tables[e.request], dtype=np.int32)
            n = min(len(table), max_pages)
            tables[i, :n] = np.maximum(table[:n], 0)     # released entries are never read
            p = pos[cu[i]:cu[i + 1]]
            page = table[p // bs]
            if (page < 0).any():
                raise AssertionError(f"request {e.request!r} writes into a released page")
            slots[cu[i]:cu[i + 1]] = page * bs + p % bs
        parts += [slots, tables.reshape(-1)]
        group_pages.append(max_pages)

    single = ctx[np.asarray(q_lens) == 1]
    parts.append(np.asarray([single.sum(), single.max()] if single.size else [0, 0], dtype=np.int32))
    sizes = [p.size for p in parts]
    offsets = np.concatenate([[0], np.cumsum([-(-s // 4) * 4 for s in sizes])])   # 16-byte aligned
    flat = np.zeros(int(offsets[-1]), dtype=np.int32)
    for p, o in zip(parts, offsets[:-1]):
        flat[o:o + p.size] = p
    return BatchArrays(flat, [int(o) for o in offsets[:-1]], sizes, group_pages, q_lens,
                       list(starts), [e.request for e in entries], slots_host, len(rows),
                       int(ctx.max()))


def batch_on_device(arr: BatchArrays, dev: torch.Tensor, max_ctx_len: int = 0) -> StepBatch:
    """A StepBatch whose arrays are views into ``dev`` (the flat array on the
    device)."""
    views = [dev[o:o + s] for o, s in zip(arr.offsets, arr.sizes)]
    S = len(arr.q_lens)
    groups = []
    for gi, max_pages in enumerate(arr.group_pages):
        groups.append(GroupMeta(views[7 + 2 * gi], views[8 + 2 * gi].view(S, max_pages), max_pages))
    n_prefill = sum(1 for q in arr.q_lens if q > 1)
    return StepBatch(
        num_tokens=sum(arr.q_lens), num_seqs=S, num_prefill_seqs=n_prefill,
        num_prefill_tokens=sum(q for q in arr.q_lens if q > 1), num_logit_rows=arr.num_rows,
        max_q_len=max(arr.q_lens), max_ctx_len=max_ctx_len or arr.max_ctx_len,
        ids=views[0], positions=views[1], tok_seq=views[2], cu_q=views[3], ctx_len=views[4],
        state_slots=views[5], logit_rows=views[6], groups=groups, ctx_stats=views[-1],
        q_lens=arr.q_lens, starts=arr.starts, requests=arr.requests,
        host_state_slots=arr.state_slots)


class Staging:
    """Pinned host memory that a step's arrays pass through on their way to the
    device, kept from step to step (pinning a fresh buffer costs more than the
    copy); ``done`` marks when the last copy out of it has finished."""

    def __init__(self):
        self.buffer = None
        self.done = None

    def upload(self, flat: np.ndarray, device) -> torch.Tensor:
        n = flat.size
        if self.buffer is None or self.buffer.numel() < n:
            self.buffer = torch.empty(max(4096, 2 * n), dtype=torch.int32).pin_memory()
            self.done = torch.cuda.Event()
        else:
            self.done.synchronize()
        self.buffer[:n].copy_(torch.from_numpy(flat))
        dev = self.buffer[:n].to(device, non_blocking=True)
        self.done.record()
        return dev


def pack_batch(entries: List[StepEntry], starts: List[int], rows: List[int], manager, device,
               pad_pages_to: int = 8, staging: "Staging" = None) -> StepBatch:
    """Build the arrays of a step and copy them to the device in one transfer."""
    arr = build_arrays(entries, starts, rows, manager, pad_pages_to)
    if torch.device(device).type != "cuda":
        return batch_on_device(arr, torch.from_numpy(arr.flat).to(device))
    if staging is None:
        return batch_on_device(arr, torch.from_numpy(arr.flat).pin_memory().to(device, non_blocking=True))
    return batch_on_device(arr, staging.upload(arr.flat, device))

"""Device storage behind the cache manager.

Reference: ``KVCachePool`` keeps ``k_store``/``v_store`` of shape
[L, num_blocks * block_size, nkv, D] in the compute dtype, zero-initialised and
never cleared on reuse (servelab/kv_cache/pool.py:49-57).  Here each page group
has one allocation per side, laid out for the attention kernels:
    k [streams, pages, nkv, page_size, D]   (a key is contiguous over D)
    v [streams, pages, nkv, D, page_size]   (a channel is contiguous over the page)
and each state group has [streams, slots, *shape].  Storage dtype is the
activation dtype, so a float32 model keeps a float32 cache
(servelab/kv_cache/pool.py:41-45).
"""
from dataclasses import dataclass
from typing import Any, List

import torch

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


@dataclass
class PageBinding:
    """What a paged mixer gets for one layer call."""
    group: int
    k: torch.Tensor          # [pages, nkv, page_size, D]
    v: torch.Tensor          # [pages, nkv, D, page_size]
    page_size: int
    write: bool


@dataclass
class StateBinding:
    """What a mixer with fixed-size state gets for one layer call: the state
    of all slots; the batch carries each sequence's slot."""
    group: int
    state: torch.Tensor      # [slots, *shape]
    write: bool


class CachePool:
    def __init__(self, manager, device, act_dtype: torch.dtype):
        self.manager = manager
        self.k: List[torch.Tensor] = []
        self.v: List[torch.Tensor] = []
        self.state: List[torch.Tensor] = []
        bs = manager.page_size
        for g in manager.page_groups:
            s = g.spec
            self.k.append(torch.zeros(len(g.streams), manager.num_pages, s.num_kv_heads, bs,
                                      s.head_dim, dtype=act_dtype, device=device))
            self.v.append(torch.zeros(len(g.streams), manager.num_pages, s.num_kv_heads,
                                      s.head_dim, bs, dtype=act_dtype, device=device))
        for g in manager.state_groups:
            self.state.append(torch.zeros(len(g.streams), manager.state_slots.num_slots,
                                          *g.spec.shape, dtype=_STATE_DTYPES[g.spec.dtype],
                                          device=device))

    def binding(self, stream: int, write: bool) -> Any:
        if stream not in self.manager.stream_group:
            return None
        kind, gi, si = self.manager.stream_group[stream]
        if kind == "pages":
            return PageBinding(gi, self.k[gi][si], self.v[gi][si], self.manager.page_size, write)
        return StateBinding(gi, self.state[gi][si], write)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.k + self.v + self.state)

    @staticmethod
    def bytes_per_page(stream_specs, page_size: int, itemsize: int) -> int:
        """Bytes one page index costs over all paged streams (for sizing the
        pool from free memory, servelab/engine/engine.py:273-288)."""
        total = 0
        for spec in stream_specs.values():
            if hasattr(spec, "num_kv_heads"):
                total += 2 * spec.num_kv_heads * spec.head_dim * page_size * itemsize
        return total

"""The device memory behind the cache manager's books."""
from dataclasses import dataclass

import torch

from .. import memory


@dataclass
class PagedView:
    """What a mixer sees of its cache: row ``page * page_tokens + offset`` of ``k`` belongs to
    one token; ``v`` has the same size but holds each page transposed (``[page][column][offset]``,
    so that the attention kernels read the keys of one value column contiguously); ``group``
    names the block table to use. The memory starts as zeros and only ever holds values that
    were stored, so a masked read of a stale row never meets a NaN."""
    group: int
    k: torch.Tensor            # [n_pages * page_tokens, k_width]
    v: torch.Tensor            # [n_pages * page_tokens, v_width]
    page_tokens: int
    window: int


@dataclass
class StateView:
    """Per-request state of fixed size: row ``slot`` of ``state`` ([n_slots, n_floats], fp32)."""
    state: torch.Tensor


class CacheStorage:
    """Key/value rows for every schedule entry that stores, a block table per group
    ([n_slots + 1, max_blocks] int32, row = the request's slot), and the state rows.

    Beyond what the manager hands out there is one more page in every group (``pad_pages[g]``)
    and one more slot (``pad_slot``) whose block tables begin with that page: rows that a step
    adds to fill a batch up to a size it has a graph for live there, apart from every request."""

    def __init__(self, manager, dtype, device):
        self.manager = manager
        self.views = [None] * len(manager.entry_group)
        rows = None
        for g, pool in zip(manager.groups, manager.pools):
            rows = (pool.n_pages + 1) * manager.page_tokens
            for e in g.entries:
                self.views[e] = PagedView(g.index,
                                          memory.zeros((rows, g.k_width), dtype, device, f"keys of schedule entry {e}"),
                                          memory.zeros((rows, g.v_width), dtype, device, f"values of schedule entry {e}"),
                                          manager.page_tokens, g.window)
        for e, n_floats in manager.state_entries.items():
            self.views[e] = StateView(memory.zeros((manager.n_slots + 1, n_floats), torch.float32, device,
                                                    f"state of schedule entry {e}"))
        self.block_tables = [memory.zeros((manager.n_slots + 1, manager.max_blocks), torch.int32, device, f"block table of group {g.index}")
                             for g in manager.groups]
        self.pad_slot = manager.n_slots
        self.pad_pages = [pool.n_pages for pool in manager.pools]
        for table, page in zip(self.block_tables, self.pad_pages):
            table[self.pad_slot, 0] = page

    def clear_slot(self, slot):
        """State starts from zero for a newly admitted request."""
        for v in self.views:
            if isinstance(v, StateView):
                v.state[slot].zero_()

    def nbytes(self):
        n = 0
        for v in self.views:
            if isinstance(v, PagedView):
                n += v.k.numel() * v.k.element_size() + v.v.numel() * v.v.element_size()
            elif isinstance(v, StateView):
                n += v.state.numel() * 4
        return n
